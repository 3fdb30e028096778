// Optimizer state in the reference's on-disk format: OptimizerStateDict / TensorBuffer / SerializableParameterGroup of
// src/nn/optim/mod.rs:51-326, saved with bincode 2 in its standard configuration (save_to_bytes / load_from_bytes,
// mod.rs:315-326).  bincode is a third-party crate; the writer and reader below follow its published wire format:
// little endian; unsigned integers as one byte below 251, else a marker 251 / 252 / 253 followed by u16 / u32 / u64;
// f32 / f64 as their IEEE bytes; String, Vec and HashMap as a length followed by the items; Option as 0 or 1 + value;
// enum as its variant index + fields; struct fields in declaration order.
// The reference builds TensorData from `tensor.as_slice()` (mod.rs:60-75), which fails for device tensors, so its GPU
// moments are skipped on save (adam.rs:428-447 "Skip parameters that cannot be serialized"); here device buffers are
// copied to the host and written, with Device::CUDA(0) as their device tag.
// A Rust HashMap iterates in a random order; maps are written here with sorted keys and read in any order.
#pragma once
#include <cstring>
#include <map>
#include <optional>

#include "hip_storage.hpp"

namespace ferrox {

struct TensorBuffer {  // mod.rs:108-117
    bool is_f64 = false;
    std::vector<float> f32;
    std::vector<double> f64;
    Shape shape;
    bool on_gpu = false;  // Device::CPU (variant 0) or Device::CUDA(id) (variant 1), src/backend/device.rs:8-13
    size_t device_id = 0;
    std::string buffer_type;
    size_t node_id = 0;
    template <typename T> static TensorBuffer from_tensor(const HipStorage<T>& t, const std::string& type, size_t node) {  // mod.rs:119-150
        TensorBuffer b;
        b.is_f64 = sizeof(T) == 8;
        std::vector<T> v = t.to_vec();  // device -> host
        if constexpr (sizeof(T) == 8) b.f64.assign(v.begin(), v.end());
        else b.f32.assign(v.begin(), v.end());
        b.shape = t.shape();
        b.on_gpu = true;
        b.buffer_type = type;
        b.node_id = node;
        return b;
    }
    template <typename T> Tensor<T> to_tensor() const {  // mod.rs:152-177 with TensorData::to_f32_tensor / to_f64_tensor
        if constexpr (sizeof(T) == 8) {
            if (!is_f64) throw Error("Type mismatch: Expected f64 data");
            return HipStorage<T>::from_vec(f64.data(), shape);
        } else {
            if (is_f64) throw Error("Type mismatch: Expected f32 data");
            return HipStorage<T>::from_vec(f32.data(), shape);
        }
    }
};

struct SerializableParameterGroup {  // mod.rs:180-197
    std::vector<size_t> params;
    std::optional<double> lr, weight_decay, momentum;
    std::string name;
};

namespace bincode {
class Writer {
  public:
    std::vector<uint8_t> out;
    void u8(uint8_t v) { out.push_back(v); }
    void le(uint64_t v, int bytes) {
        for (int i = 0; i < bytes; ++i) out.push_back((uint8_t)(v >> (8 * i)));
    }
    void varint(uint64_t v) {
        if (v < 251) u8((uint8_t)v);
        else if (v < (1ull << 16)) { u8(251); le(v, 2); }
        else if (v < (1ull << 32)) { u8(252); le(v, 4); }
        else { u8(253); le(v, 8); }
    }
    void f32(float v) { uint32_t b; std::memcpy(&b, &v, 4); le(b, 4); }
    void f64(double v) { uint64_t b; std::memcpy(&b, &v, 8); le(b, 8); }
    void str(const std::string& s) { varint(s.size()); out.insert(out.end(), s.begin(), s.end()); }
    void opt(const std::optional<double>& v) {
        if (v) { u8(1); f64(*v); }
        else u8(0);
    }
};
class Reader {
  public:
    Reader(const uint8_t* p, size_t n) : p_(p), n_(n) {}
    uint8_t u8() { need(1); return p_[i_++]; }
    uint64_t le(int bytes) {
        need((size_t)bytes);
        uint64_t v = 0;
        for (int i = 0; i < bytes; ++i) v |= (uint64_t)p_[i_ + i] << (8 * i);
        i_ += (size_t)bytes;
        return v;
    }
    uint64_t varint() {
        const uint8_t t = u8();
        if (t < 251) return t;
        if (t == 251) return le(2);
        if (t == 252) return le(4);
        if (t == 253) return le(8);
        throw Error("bincode: integer does not fit 64 bits");
    }
    // a length that is about to be used for an allocation: each item takes at least `min_item` bytes of input
    size_t len(size_t min_item) {
        const uint64_t v = varint();
        if (min_item && v > (n_ - i_) / min_item) throw Error("bincode: length exceeds the remaining input");
        return (size_t)v;
    }
    float f32() { const uint32_t b = (uint32_t)le(4); float v; std::memcpy(&v, &b, 4); return v; }
    double f64() { const uint64_t b = le(8); double v; std::memcpy(&v, &b, 8); return v; }
    std::string str() {
        const size_t n = len(1);
        need(n);
        std::string s(reinterpret_cast<const char*>(p_ + i_), n);
        i_ += n;
        return s;
    }
    std::optional<double> opt() {
        const uint8_t t = u8();
        if (t > 1) throw Error("bincode: invalid Option tag");
        if (!t) return std::nullopt;
        return f64();
    }
    bool done() const { return i_ == n_; }

  private:
    void need(size_t n) const {
        if (n > n_ - i_) throw Error("bincode: unexpected end of data");
    }
    const uint8_t* p_;
    size_t n_, i_ = 0;
};
}  // namespace bincode

struct OptimizerStateDict {  // mod.rs:263-326
    std::string optimizer_type;
    uint64_t step_count = 0;
    std::map<std::string, double> hyperparameters;
    std::map<std::string, TensorBuffer> parameter_buffers;
    std::vector<SerializableParameterGroup> parameter_groups;

    template <typename T> void add_buffer(size_t node_id, const HipStorage<T>& t, const std::string& type) {  // :281-294
        parameter_buffers[std::to_string(node_id) + "_" + type] = TensorBuffer::from_tensor<T>(t, type, node_id);
    }
    const TensorBuffer* get_buffer(size_t node_id, const std::string& type) const {  // :297-300
        auto it = parameter_buffers.find(std::to_string(node_id) + "_" + type);
        return it == parameter_buffers.end() ? nullptr : &it->second;
    }
    std::vector<uint8_t> save_to_bytes() const {  // :315-318
        bincode::Writer w;
        w.str(optimizer_type);
        w.varint(step_count);
        w.varint(hyperparameters.size());
        for (const auto& kv : hyperparameters) { w.str(kv.first); w.f64(kv.second); }
        w.varint(parameter_buffers.size());
        for (const auto& kv : parameter_buffers) {
            const TensorBuffer& b = kv.second;
            w.str(kv.first);
            w.varint(b.is_f64 ? 1 : 0);  // TensorData::F32 = 0, F64 = 1
            if (b.is_f64) { w.varint(b.f64.size()); for (double v : b.f64) w.f64(v); }
            else { w.varint(b.f32.size()); for (float v : b.f32) w.f32(v); }
            w.varint(b.shape.size());
            for (size_t d : b.shape) w.varint(d);
            if (b.on_gpu) { w.varint(1); w.varint(b.device_id); }
            else w.varint(0);
            w.str(b.buffer_type);
            w.varint(b.node_id);
        }
        w.varint(parameter_groups.size());
        for (const auto& g : parameter_groups) {
            w.varint(g.params.size());
            for (size_t p : g.params) w.varint(p);
            w.opt(g.lr); w.opt(g.weight_decay); w.opt(g.momentum);
            w.str(g.name);
        }
        return std::move(w.out);
    }
    static OptimizerStateDict load_from_bytes(const uint8_t* data, size_t n) {  // :321-325
        bincode::Reader r(data, n);
        OptimizerStateDict sd;
        sd.optimizer_type = r.str();
        sd.step_count = r.varint();
        for (size_t k = r.len(9); k-- > 0;) {
            std::string key = r.str();
            sd.hyperparameters[key] = r.f64();
        }
        for (size_t k = r.len(6); k-- > 0;) {
            std::string key = r.str();
            TensorBuffer b;
            const uint64_t variant = r.varint();
            if (variant > 1) throw Error("bincode: unknown TensorData variant");
            b.is_f64 = variant == 1;
            if (b.is_f64) { b.f64.resize(r.len(8)); for (double& v : b.f64) v = r.f64(); }
            else { b.f32.resize(r.len(4)); for (float& v : b.f32) v = r.f32(); }
            b.shape.resize(r.len(1));
            for (size_t& d : b.shape) d = (size_t)r.varint();
            const uint64_t dev = r.varint();
            if (dev > 1) throw Error("bincode: unknown Device variant");
            b.on_gpu = dev == 1;
            if (b.on_gpu) b.device_id = (size_t)r.varint();
            b.buffer_type = r.str();
            b.node_id = (size_t)r.varint();
            if (numel(b.shape) != (b.is_f64 ? b.f64.size() : b.f32.size())) throw Error("optimizer state: buffer shape does not match its data");
            sd.parameter_buffers[key] = std::move(b);
        }
        sd.parameter_groups.resize(r.len(5));
        for (auto& g : sd.parameter_groups) {
            g.params.resize(r.len(1));
            for (size_t& p : g.params) p = (size_t)r.varint();
            g.lr = r.opt(); g.weight_decay = r.opt(); g.momentum = r.opt();
            g.name = r.str();
        }
        if (!r.done()) throw Error("bincode: trailing bytes after the optimizer state");
        return sd;
    }
};

}  // namespace ferrox
