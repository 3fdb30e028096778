// HipStorage<T>: the host-side storage backend that sits behind Ferrox's `trait StorageBackend<T>`
// (src/backend/storage/mod.rs:24-422) and forwards every hot-path method to libferrox_hip.so through the C ABI of
// include/ferrox_hip.h.  It is the C++ twin of the `impl StorageBackend<T> for HipStorage<T>` a Rust build would
// carry (the reference's CUDAStorage, src/backend/storage/cuda.rs:28-1381, is the template): same method names,
// same argument meaning, every compute method returns NEW owned storage, view methods work in place, errors are
// strings with the reference's wording (thrown as ferrox::Error, the stand-in for Result<_, String>).
//
// Ownership follows CudaTensor (src/backend/cuda/context.rs:284-763): one pool allocation per storage, returned to
// the pool on destruction (Drop, :726-742); clone_storage is a device-to-device copy (:744-763).
#pragma once
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <memory>
#include <mutex>
#include <numeric>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/ferrox_hip.h"

namespace ferrox {

using Shape = std::vector<size_t>;

struct Error : std::runtime_error {
    using std::runtime_error::runtime_error;
};

inline std::string fmt_shape(const Shape& s) {  // Rust's {:?} of a usize slice
    std::ostringstream o;
    o << "[";
    for (size_t i = 0; i < s.size(); ++i) o << (i ? ", " : "") << s[i];
    o << "]";
    return o.str();
}
inline size_t numel(const Shape& s) { return std::accumulate(s.begin(), s.end(), size_t(1), std::multiplies<size_t>()); }
inline void fx_ok(int rc) {
    if (rc != FX_OK) throw Error(fx_last_error());
}

// BackendManager (src/backend/manager.rs:22-340): process-wide owner of the device context and the pools.
class BackendManager {
  public:
    static BackendManager& get() {
        static BackendManager m;
        return m;
    }
    // BackendManager::init(Option<PoolConfig>), manager.rs:53
    void init(int device = 0, const fx_pool_config* cfg = nullptr) {
        if (ctx_) return;
        fx_ok(fx_init(device, cfg, &ctx_));
    }
    void shutdown() {
        if (ctx_) fx_destroy(ctx_);
        ctx_ = nullptr;
    }
    bool has_hip() const { return ctx_ != nullptr; }
    fx_ctx* ctx() const {
        if (!ctx_) throw Error("CUDA backend not available");  // with_cuda_context, manager.rs:405-416
        return ctx_;
    }
    // 0: mathematical conv gradients (the reference's GPU semantics); 1: the CPU backend's literal arithmetic
    int conv_grad_mode = 0;
    // clone_storage() as a second owner of the same device block instead of a device-to-device copy.  Nothing reachable through
    // the storage trait writes device memory in place (every op returns new storage, the &mut methods of storage/mod.rs:246-269
    // change the view and materialise into a NEW block), so a shared clone cannot be told from a copied one.  Off for callers
    // that do update tensors in place (the fused optimizers, a recorded step's batch).
    bool share_clones = false;

  private:
    fx_ctx* ctx_ = nullptr;
};

// dtype dispatch onto the _f32 / _f64 entry points
template <typename T> struct Api;
#define FERROX_API(T, S, CODE)                                                                                          \
    template <> struct Api<T> {                                                                                        \
        static constexpr int dtype = CODE;                                                                             \
        static int fill(fx_ctx* c, T* o, T v, int64_t n) { return fx_fill_##S(c, o, v, n); }                           \
        static int materialize(fx_ctx* c, const T* i, T* o, const int64_t* sh, const int64_t* st, int nd, int64_t n) { \
            return fx_materialize_##S(c, i, o, sh, st, nd, n);                                                         \
        }                                                                                                              \
        static int binary(fx_ctx* c, int op, const T* a, const T* b, T* o, int64_t n) { return fx_binary_##S(c, op, a, b, o, n); } \
        static int scalar(fx_ctx* c, int op, const T* a, T s, T* o, int64_t n) { return fx_scalar_##S(c, op, a, s, o, n); } \
        static int unary(fx_ctx* c, int op, const T* a, T* o, int64_t n) { return fx_unary_##S(c, op, a, o, n); }      \
        static int clamp(fx_ctx* c, const T* a, T lo, T hi, T* o, int64_t n) { return fx_clamp_##S(c, a, lo, hi, o, n); } \
        static int in_range(fx_ctx* c, const T* a, T lo, T hi, T* o, int64_t n) { return fx_in_range_##S(c, a, lo, hi, o, n); } \
        static int rmin(fx_ctx* c, const T* i, T* o, int64_t ou, int64_t ax, int64_t in) { return fx_reduce_min_##S(c, i, o, nullptr, ou, ax, in); } \
        static int pool(fx_ctx* c, bool mx, const T* i, T* o, const int64_t* d) {                                      \
            return mx ? fx_maxpool2d_##S(c, i, o, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9])          \
                      : fx_avgpool2d_##S(c, i, o, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9]);         \
        }                                                                                                              \
        static int unpool(fx_ctx* c, bool mx, const T* g, const T* x, const T* p, T* gi, const int64_t* d) {           \
            return mx ? fx_max_unpool2d_##S(c, g, x, p, gi, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9]) \
                      : fx_avg_unpool2d_##S(c, g, gi, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9]);     \
        }                                                                                                              \
        static int softmax(fx_ctx* c, const T* i, T* o, int64_t ou, int64_t ax, int64_t in) { return fx_softmax_axis_##S(c, i, o, ou, ax, in); } \
        static int rsum(fx_ctx* c, const T* i, T* o, int64_t ou, int64_t ax, int64_t in) { return fx_reduce_sum_##S(c, i, o, ou, ax, in); } \
        static int rmean(fx_ctx* c, const T* i, T* o, int64_t ou, int64_t ax, int64_t in) { return fx_reduce_mean_##S(c, i, o, ou, ax, in); } \
        static int rmax(fx_ctx* c, const T* i, T* o, int64_t ou, int64_t ax, int64_t in) { return fx_reduce_max_##S(c, i, o, nullptr, ou, ax, in); } \
        static int gemm(fx_ctx* c, int ta, int tb, int64_t M, int64_t N, int64_t K, const T* A, const T* B, T* C) {    \
            return fx_gemm_##S(c, ta, tb, M, N, K, A, B, C);                                                           \
        }                                                                                                              \
        static int conv_fwd(fx_ctx* c, const T* x, const T* w, T* y, const int64_t* d) {                               \
            return fx_conv2d_fwd_##S(c, x, w, y, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10], nullptr, 0); \
        }                                                                                                              \
        static int conv_dgrad(fx_ctx* c, const T* g, const T* w, T* dx, const int64_t* d, int mode) {                  \
            return fx_conv2d_dgrad_##S(c, g, w, dx, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10], mode, nullptr, 0); \
        }                                                                                                              \
        static int conv_wgrad(fx_ctx* c, const T* x, const T* g, T* dw, const int64_t* d, int mode) {                  \
            return fx_conv2d_wgrad_##S(c, x, g, dw, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], d[8], d[9], d[10], mode, nullptr, 0); \
        }                                                                                                              \
    };
FERROX_API(float, f32, FX_F32)
FERROX_API(double, f64, FX_F64)
#undef FERROX_API

template <typename T> class HipStorage {
  public:
    using Ptr = std::unique_ptr<HipStorage<T>>;

    HipStorage(const HipStorage&) = delete;
    HipStorage& operator=(const HipStorage&) = delete;
    ~HipStorage() { release(); }

    // Set on a gradient that its producer already multiplied by a ReLU's mask: the activation tensor whose (value > 0) was
    // applied.  The operator that owns that activation then skips its own masking.  Never copied: any tensor made from this one
    // (a sum of gradients, a clone) starts without the mark, and is masked again where it matters (the mask is idempotent).
    const void* relu_masked_by = nullptr;

    // ---- factories: BackendManager::{zeros, ones, full, from_vec}, manager.rs:131-339 ------------------------
    // CudaOps::get_tensor (cuda/ops.rs:121-133): output buffers come from the pool and are not cleared.
    static Ptr alloc(const Shape& shape) {
        Ptr s(new HipStorage());
        s->shape_ = shape;
        const size_t n = numel(shape);
        void* p = nullptr;
        fx_ok(fx_alloc(ctx(), Api<T>::dtype, (int64_t)n, &p, &s->granted_, &s->id_));
        s->ptr_ = static_cast<T*>(p);
        return s;
    }
    // A storage that aliases another one's device memory without owning it (the caller keeps the original alive):
    // used by the fused training loop for the batch, which the reference clones every step (training.rs:125-126).
    static Ptr borrow(const HipStorage& src) {
        Ptr s(new HipStorage());
        s->shape_ = src.shape_;
        s->ptr_ = src.ptr_;
        s->borrowed_ = true;
        return s;
    }
    static Ptr full(const Shape& shape, T value) {
        Ptr s = alloc(shape);
        fx_ok(Api<T>::fill(ctx(), s->ptr_, value, (int64_t)s->size()));
        return s;
    }
    static Ptr zeros(const Shape& shape) { return full(shape, T(0)); }
    static Ptr ones(const Shape& shape) { return full(shape, T(1)); }
    static Ptr from_vec(const T* data, const Shape& shape) {  // host_to_device, context.rs:81-97
        Ptr s = alloc(shape);
        fx_ok(fx_h2d(ctx(), s->ptr_, data, (int64_t)(s->size() * sizeof(T))));
        return s;
    }

    // ---- metadata: storage/mod.rs:29-54 ---------------------------------------------------------------------
    const Shape& shape() const { return shape_; }
    size_t ndim() const { return shape_.size(); }
    size_t size() const { return numel(shape_); }
    bool is_gpu() const { return true; }
    bool owns_data() const { return true; }
    const T* data() const { return ptr_; }
    T* data() { return ptr_; }
    [[noreturn]] void cpu_data() const { throw Error("GPU storage has no CPU data. Use to_cpu() first"); }  // storage/cuda.rs:56-62
    Ptr clone_storage() const {  // CudaTensor::clone, context.rs:744-763
        if (BackendManager::get().share_clones && ptr_ && !borrowed_) {
            static std::mutex first_clone;  // two threads may clone one storage through const references at the same time
            std::lock_guard<std::mutex> lk(first_clone);
            if (!owner_) {  // first clone: the block moves to a counted owner, which returns it to the pool when the last storage lets go
                const uint64_t id = id_;
                owner_ = std::shared_ptr<void>(static_cast<void*>(ptr_), [id](void* q) {
                    if (BackendManager::get().has_hip()) fx_free(BackendManager::get().ctx(), Api<T>::dtype, q, id);
                });
            }
            Ptr s(new HipStorage());
            s->shape_ = shape_;
            s->ptr_ = ptr_;
            s->id_ = id_;
            s->granted_ = granted_;
            s->owner_ = owner_;
            return s;
        }
        Ptr s = alloc(shape_);
        fx_ok(fx_d2d(ctx(), s->ptr_, ptr_, (int64_t)(size() * sizeof(T))));
        return s;
    }
    std::vector<T> to_vec() const {  // CudaTensor::to_vec, context.rs:410-426 (truncates an oversized pooled block)
        std::vector<T> v(size());
        fx_ok(fx_d2h(ctx(), v.data(), ptr_, (int64_t)(v.size() * sizeof(T))));
        return v;
    }
    T first() const {  // Tensor::first, tensor.rs:1048-1067: one scalar crosses to the host (synchronises)
        if (size() == 0) throw Error("Empty array");
        T v;
        fx_ok(fx_d2h(ctx(), &v, ptr_, (int64_t)sizeof(T)));
        return v;
    }

    // ---- elementwise: storage/mod.rs add/sub/mul/div/..., CUDAStorage storage/cuda.rs:75-560 ------------------
    Ptr add(const HipStorage& o) const { return binary(FX_ADD, o, "addition"); }
    Ptr sub(const HipStorage& o) const { return binary(FX_SUB, o, "subtraction"); }
    Ptr mul(const HipStorage& o) const { return binary(FX_MUL, o, "multiplication"); }
    Ptr div(const HipStorage& o) const { return binary(FX_DIV, o, "division"); }
    Ptr equal(const HipStorage& o) const { return binary(FX_EQUAL, o, "comparison"); }
    Ptr min(const HipStorage& o) const { return binary(FX_MIN, o, "min operation"); }          // cpu.rs:692-715
    Ptr max(const HipStorage& o) const { return binary(FX_MAX, o, "max operation"); }          // cpu.rs:717-740
    Ptr greater(const HipStorage& o) const { return binary(FX_GREATER, o, "comparison"); }     // cpu.rs:865-885
    Ptr greater_equal(const HipStorage& o) const { return binary(FX_GREATER_EQUAL, o, "comparison"); }
    Ptr less(const HipStorage& o) const { return binary(FX_LESS, o, "comparison"); }
    Ptr less_equal(const HipStorage& o) const { return binary(FX_LESS_EQUAL, o, "comparison"); }
    Ptr powf(const HipStorage& o) const { return binary(FX_POW, o, "powf"); }                  // cpu.rs:1152-1172
    Ptr power_scalar(T s) const { return scalar(FX_POW_SCALAR, s); }                           // cpu.rs:1174-1181
    Ptr less_scalar(T s) const { return scalar(FX_LESS_SCALAR, s); }
    Ptr abs() const { return unary(FX_ABS); }
    Ptr reciprocal() const { return unary(FX_RECIPROCAL); }
    Ptr sign() const { return unary(FX_SIGN); }                                               // cpu.rs:949-965
    Ptr logical_not() const { return unary(FX_LOGICAL_NOT); }                                 // cpu.rs:920-931
    Ptr in_range(T lo, T hi) const {                                                          // cpu.rs:933-947
        Ptr r = alloc(shape_);
        fx_ok(Api<T>::in_range(ctx(), ptr_, lo, hi, r->ptr_, (int64_t)size()));
        return r;
    }
    Ptr add_scalar(T s) const { return scalar(FX_ADD_SCALAR, s); }
    Ptr sub_scalar(T s) const { return scalar(FX_SUB_SCALAR, s); }
    Ptr mul_scalar(T s) const { return scalar(FX_MUL_SCALAR, s); }
    Ptr div_scalar(T s) const { return scalar(FX_DIV_SCALAR, s); }
    Ptr greater_scalar(T s) const { return scalar(FX_GREATER_SCALAR, s); }
    Ptr greater_equal_scalar(T s) const { return scalar(FX_GREATER_EQUAL_SCALAR, s); }
    Ptr less_equal_scalar(T s) const { return scalar(FX_LESS_EQUAL_SCALAR, s); }
    Ptr neg() const { return unary(FX_NEG); }
    Ptr sqrt() const { return unary(FX_SQRT); }
    Ptr exp() const { return unary(FX_EXP); }
    Ptr log() const { return unary(FX_LOG); }
    Ptr relu() const { return unary(FX_RELU); }
    Ptr sigmoid() const { return unary(FX_SIGMOID); }
    Ptr tanh() const { return unary(FX_TANH); }
    Ptr clamp(T lo, T hi) const {
        Ptr r = alloc(shape_);
        fx_ok(Api<T>::clamp(ctx(), ptr_, lo, hi, r->ptr_, (int64_t)size()));
        return r;
    }

    // ---- matmul: storage/cuda.rs:540-600, cpu.rs:967-1002 ----------------------------------------------------
    Ptr matmul(const HipStorage& o) const {
        if (ndim() != 2 || o.ndim() != 2) throw Error("Matrix multiplication requires 2D tensors");
        if (shape_[1] != o.shape_[0]) {
            std::ostringstream m;
            m << "Matrix multiplication shape mismatch: (" << shape_[0] << ", " << shape_[1] << ") @ (" << o.shape_[0] << ", "
              << o.shape_[1] << ")";
            throw Error(m.str());
        }
        Ptr r = alloc({shape_[0], o.shape_[1]});
        fx_ok(Api<T>::gemm(ctx(), 0, 0, (int64_t)shape_[0], (int64_t)o.shape_[1], (int64_t)shape_[1], ptr_, o.ptr_, r->ptr_));
        return r;
    }
    // C = op(self) . op(other) without materialised transposes (not in the trait: used by the fused gradient path)
    Ptr matmul_t(const HipStorage& o, bool ta, bool tb) const {
        if (ndim() != 2 || o.ndim() != 2) throw Error("Matrix multiplication requires 2D tensors");
        const size_t M = ta ? shape_[1] : shape_[0], K = ta ? shape_[0] : shape_[1];
        const size_t Kb = tb ? o.shape_[1] : o.shape_[0], N = tb ? o.shape_[0] : o.shape_[1];
        if (K != Kb) throw Error("Matrix multiplication shape mismatch");
        Ptr r = alloc({M, N});
        fx_ok(Api<T>::gemm(ctx(), ta, tb, (int64_t)M, (int64_t)N, (int64_t)K, ptr_, o.ptr_, r->ptr_));
        return r;
    }

    // ---- softmax_batched: storage/mod.rs, cpu.rs:1037-1068 ----------------------------------------------------
    Ptr softmax_batched(size_t axis) const {
        if (axis >= ndim()) {
            std::ostringstream m;
            m << "Softmax axis " << axis << " out of bounds for tensor with " << ndim() << " dimensions";
            throw Error(m.str());
        }
        int64_t outer, ax, inner;
        oai(shape_, axis, outer, ax, inner);
        Ptr r = alloc(shape_);
        fx_ok(Api<T>::softmax(ctx(), ptr_, r->ptr_, outer, ax, inner));
        return r;
    }

    Ptr softmax() const {  // whole tensor as one row, cpu.rs:1018-1036
        Ptr r = alloc(shape_);
        fx_ok(Api<T>::softmax(ctx(), ptr_, r->ptr_, 1, (int64_t)size(), 1));
        return r;
    }

    // ---- pooling and its gradients: storage/mod.rs:328-420, extensions/pooling.rs; storage/cuda.rs:1127-1290 ----
    Ptr maxpool2d(size_t k, size_t s, size_t p) const { return pool2d(true, k, s, p, "Maxpool2d"); }
    Ptr avgpool2d(size_t k, size_t s, size_t p) const { return pool2d(false, k, s, p, "Avgpool2d"); }
    Ptr maxpool1d(size_t k, size_t s, size_t p) const { return pool1d(true, k, s, p, "Maxpool1d"); }
    Ptr avgpool1d(size_t k, size_t s, size_t p) const { return pool1d(false, k, s, p, "Avgpool1d"); }
    // self is the upstream gradient; original_input / pooled_output as in the trait
    Ptr max_unpool2d(const HipStorage& original_input, const HipStorage& pooled_output, size_t k, size_t s, size_t p) const {
        return unpool(true, original_input, &pooled_output, k, k, s, s, p, p);
    }
    Ptr avg_unpool2d(const HipStorage& original_input, const HipStorage& pooled_output, size_t k, size_t s, size_t p) const {
        return unpool(false, original_input, &pooled_output, k, k, s, s, p, p);
    }
    Ptr max_unpool1d(const HipStorage& original_input, const HipStorage& pooled_output, size_t k, size_t s, size_t p) const {
        return unpool(true, original_input, &pooled_output, 1, k, 1, s, 0, p);
    }
    Ptr avg_unpool1d(const HipStorage& original_input, const HipStorage& pooled_output, size_t k, size_t s, size_t p) const {
        return unpool(false, original_input, &pooled_output, 1, k, 1, s, 0, p);
    }

    // ---- reductions: cpu.rs:60-130, 1183-1238; CudaOps::reduce_axes cuda/ops.rs:2171-2284 ---------------------
    // axes == nullptr reduces everything to a 0-dimensional result (or all-ones shape with keep_dims).
    Ptr sum(const std::vector<size_t>* axes, bool keep_dims) const { return reduce(0, axes, keep_dims); }
    Ptr max_reduce(const std::vector<size_t>* axes, bool keep_dims) const { return reduce(2, axes, keep_dims); }
    Ptr min_reduce(const std::vector<size_t>* axes, bool keep_dims) const { return reduce(3, axes, keep_dims); }  // cpu.rs:1240-1252
    Ptr mean(const std::vector<size_t>* axes, bool keep_dims) const {  // sum * T(1/n), cpu.rs:1193-1221
        Ptr s = reduce(0, axes, keep_dims);
        double n = 1;
        if (axes) for (size_t a : *axes) n *= (double)shape_[a];
        else n = (double)size();
        return s->mul_scalar((T)(1.0 / n));
    }

    // ---- view operations, in place: storage/mod.rs:246-265; CUDAStorage storage/cuda.rs:795-911 -----------------
    void reshape(const Shape& ns) {
        if (numel(ns) != size()) {
            std::ostringstream m;
            m << "Cannot change shape: current size " << size() << " != new size " << numel(ns);
            throw Error(m.str());
        }
        shape_ = ns;  // contiguous storage: metadata only
    }
    void unsqueeze(size_t axis) {
        if (axis > ndim()) {
            std::ostringstream m;
            m << "Axis " << axis << " out of bounds for tensor with " << ndim() << " dimensions";
            throw Error(m.str());
        }
        Shape ns = shape_;
        ns.insert(ns.begin() + axis, 1);
        reshape(ns);
    }
    void squeeze(const size_t* axis) {
        Shape ns;
        if (axis) {
            if (*axis >= ndim()) throw Error("Axis out of bounds for squeeze");
            if (shape_[*axis] != 1) {
                std::ostringstream m;
                m << "Cannot squeeze axis " << *axis << " with size " << shape_[*axis];
                throw Error(m.str());
            }
            ns = shape_;
            ns.erase(ns.begin() + *axis);
        } else {
            for (size_t d : shape_) if (d != 1) ns.push_back(d);
            if (ns.empty()) ns.push_back(1);
        }
        reshape(ns);
    }
    void broadcast_to(const Shape& target) {  // cpu.rs:510-541; materialised like storage/cuda.rs eager materialize
        if (target.size() < ndim()) throw Error("Cannot broadcast to smaller number of dimensions");
        const size_t off = target.size() - ndim();
        std::vector<int64_t> sh(target.begin(), target.end()), st(target.size(), 0);
        int64_t stride = 1;
        for (size_t i = ndim(); i-- > 0;) {
            const size_t cur = shape_[i], tgt = target[off + i];
            if (cur != 1 && cur != tgt) {
                std::ostringstream m;
                m << "Cannot broadcast dimension " << i << " from size " << cur << " to size " << tgt;
                throw Error(m.str());
            }
            st[off + i] = cur == 1 ? 0 : stride;
            stride *= (int64_t)cur;
        }
        materialize_into(target, sh, st);
    }
    void transpose(const std::vector<size_t>* axes) {  // cpu.rs:543-562
        const size_t nd = ndim();
        std::vector<size_t> order(nd);
        if (axes) {
            std::vector<size_t> sorted = *axes;
            std::sort(sorted.begin(), sorted.end());
            bool ok = axes->size() == nd;
            for (size_t i = 0; ok && i < nd; ++i) ok = sorted[i] == i;
            if (!ok) throw Error("Invalid axes permutation");
            order = *axes;
        } else {
            if (nd <= 1) return;
            for (size_t i = 0; i < nd; ++i) order[i] = nd - 1 - i;
        }
        std::vector<int64_t> cst(nd, 1);
        for (size_t i = nd - 1; i-- > 0;) cst[i] = cst[i + 1] * (int64_t)shape_[i + 1];
        Shape ns(nd);
        std::vector<int64_t> sh(nd), st(nd);
        for (size_t i = 0; i < nd; ++i) {
            ns[i] = shape_[order[i]];
            sh[i] = (int64_t)ns[i];
            st[i] = cst[order[i]];
        }
        materialize_into(ns, sh, st);
    }

    // ---- convolution: storage/mod.rs:276-330; cpu.rs:1255-1314; storage/cuda.rs:913-1020 ------------------------
    Ptr conv2d(const HipStorage& filter, std::pair<size_t, size_t> stride, std::pair<size_t, size_t> padding) const {
        if (ndim() != 4 || filter.ndim() != 4) throw Error("Conv2D requires 4D tensors [batch, channels, height, width]");
        int64_t d[11];
        dims(shape_, filter.shape_, stride, padding, d);
        const size_t oh = (shape_[2] + 2 * padding.first - filter.shape_[2]) / stride.first + 1;
        const size_t ow = (shape_[3] + 2 * padding.second - filter.shape_[3]) / stride.second + 1;
        Ptr y = alloc({shape_[0], filter.shape_[0], oh, ow});
        fx_ok(Api<T>::conv_fwd(ctx(), ptr_, filter.ptr_, y->ptr_, d));
        return y;
    }
    // self is the upstream gradient [B, Cout, oh, ow]; returns the gradient w.r.t. the conv input
    Ptr deconv2d(const HipStorage& filter, const Shape& output_shape, std::pair<size_t, size_t> stride,
                 std::pair<size_t, size_t> padding) const {
        if (output_shape.size() != 4 || filter.ndim() != 4 || ndim() != 4)
            throw Error("Deconv2D requires 4D tensors [batch, channels, height, width]");
        int64_t d[11];
        dims(output_shape, filter.shape_, stride, padding, d);
        Ptr dx = alloc(output_shape);
        fx_ok(Api<T>::conv_dgrad(ctx(), ptr_, filter.ptr_, dx->ptr_, d, BackendManager::get().conv_grad_mode));
        return dx;
    }
    // self is the conv input; other the upstream gradient; output_shape the filter shape
    Ptr cross_correlation2d(const HipStorage& other, const Shape& output_shape, std::pair<size_t, size_t> stride,
                            std::pair<size_t, size_t> padding) const {
        if (ndim() != 4 || other.ndim() != 4 || output_shape.size() != 4)
            throw Error("Cross correlation requires 4D tensors [batch, channels, height, width]");
        int64_t d[11];
        dims(shape_, output_shape, stride, padding, d);
        Ptr dw = alloc(output_shape);
        fx_ok(Api<T>::conv_wgrad(ctx(), ptr_, other.ptr_, dw->ptr_, d, BackendManager::get().conv_grad_mode));
        return dw;
    }

  private:
    HipStorage() = default;
    static fx_ctx* ctx() { return BackendManager::get().ctx(); }
    void release() {
        if (owner_) owner_.reset();
        else if (ptr_ && !borrowed_ && BackendManager::get().has_hip()) fx_free(ctx(), Api<T>::dtype, ptr_, id_);
        ptr_ = nullptr;
    }
    static void oai(const Shape& s, size_t axis, int64_t& outer, int64_t& ax, int64_t& inner) {
        outer = inner = 1;
        for (size_t i = 0; i < axis; ++i) outer *= (int64_t)s[i];
        for (size_t i = axis + 1; i < s.size(); ++i) inner *= (int64_t)s[i];
        ax = (int64_t)s[axis];
    }
    static void dims(const Shape& x, const Shape& w, std::pair<size_t, size_t> s, std::pair<size_t, size_t> p, int64_t* d) {
        d[0] = (int64_t)x[0]; d[1] = (int64_t)x[1]; d[2] = (int64_t)x[2]; d[3] = (int64_t)x[3];
        d[4] = (int64_t)w[0]; d[5] = (int64_t)w[2]; d[6] = (int64_t)w[3];
        d[7] = (int64_t)s.first; d[8] = (int64_t)s.second; d[9] = (int64_t)p.first; d[10] = (int64_t)p.second;
    }
    Ptr binary(int op, const HipStorage& o, const char* what) const {
        if (shape_ != o.shape_) throw Error(std::string("Shape mismatch for GPU ") + what + ": " + fmt_shape(shape_) + " vs " + fmt_shape(o.shape_));
        Ptr r = alloc(shape_);
        fx_ok(Api<T>::binary(ctx(), op, ptr_, o.ptr_, r->ptr_, (int64_t)size()));
        return r;
    }
    Ptr scalar(int op, T s) const {
        Ptr r = alloc(shape_);
        fx_ok(Api<T>::scalar(ctx(), op, ptr_, s, r->ptr_, (int64_t)size()));
        return r;
    }
    Ptr unary(int op) const {
        Ptr r = alloc(shape_);
        fx_ok(Api<T>::unary(ctx(), op, ptr_, r->ptr_, (int64_t)size()));
        return r;
    }
    void materialize_into(const Shape& ns, const std::vector<int64_t>& sh, const std::vector<int64_t>& st) {
        Ptr r = alloc(ns);
        fx_ok(Api<T>::materialize(ctx(), ptr_, r->ptr_, sh.data(), st.data(), (int)sh.size(), (int64_t)numel(ns)));
        std::swap(ptr_, r->ptr_);
        std::swap(id_, r->id_);
        std::swap(granted_, r->granted_);
        std::swap(borrowed_, r->borrowed_);
        std::swap(owner_, r->owner_);
        shape_ = ns;
    }
    Ptr pool2d(bool is_max, size_t k, size_t s, size_t p, const char* what) const {
        if (ndim() != 4) throw Error(std::string(what) + " requires 4D tensor [N, C, H, W]");
        const int64_t d[10] = {(int64_t)shape_[0], (int64_t)shape_[1], (int64_t)shape_[2], (int64_t)shape_[3], (int64_t)k, (int64_t)k,
                               (int64_t)s, (int64_t)s, (int64_t)p, (int64_t)p};
        Ptr r = alloc({shape_[0], shape_[1], (shape_[2] + 2 * p - k) / s + 1, (shape_[3] + 2 * p - k) / s + 1});
        fx_ok(Api<T>::pool(ctx(), is_max, ptr_, r->ptr_, d));
        return r;
    }
    Ptr pool1d(bool is_max, size_t k, size_t s, size_t p, const char* what) const {  // [N, C, L] = H of 1, window 1 x k
        if (ndim() != 3) throw Error(std::string(what) + " requires 3D tensor [N, C, L]");
        const int64_t d[10] = {(int64_t)shape_[0], (int64_t)shape_[1], 1, (int64_t)shape_[2], 1, (int64_t)k, 1, (int64_t)s, 0, (int64_t)p};
        Ptr r = alloc({shape_[0], shape_[1], (shape_[2] + 2 * p - k) / s + 1});
        fx_ok(Api<T>::pool(ctx(), is_max, ptr_, r->ptr_, d));
        return r;
    }
    Ptr unpool(bool is_max, const HipStorage& x, const HipStorage* pooled, size_t kh, size_t kw, size_t sh, size_t sw, size_t ph,
               size_t pw) const {
        const bool one_d = x.ndim() == 3;
        if (!one_d && (x.ndim() != 4 || ndim() != 4)) throw Error("Unpool2D requires 4D tensors [N, C, H, W]");
        if (one_d && ndim() != 3) throw Error("Unpool1D requires 3D tensors [N, C, L]");
        const Shape& xs = x.shape_;
        const int64_t d[10] = {(int64_t)xs[0], (int64_t)xs[1], one_d ? 1 : (int64_t)xs[2], (int64_t)xs[one_d ? 2 : 3], (int64_t)kh,
                               (int64_t)kw, (int64_t)sh, (int64_t)sw, (int64_t)ph, (int64_t)pw};
        Ptr r = alloc(xs);
        fx_ok(Api<T>::unpool(ctx(), is_max, ptr_, x.ptr_, pooled ? pooled->ptr_ : nullptr, r->ptr_, d));
        return r;
    }
    // kind 0 sum, 2 max, 3 min.  One kernel per axis, axes in descending order, temporaries between steps
    // (CudaOps::reduce_axes, cuda/ops.rs:2171-2284; the CPU backend uses the same order, cpu.rs:85-95).
    Ptr reduce(int kind, const std::vector<size_t>* axes, bool keep_dims) const {
        auto launch = [&](const T* in, T* out, int64_t outer, int64_t ax, int64_t inner) {
            fx_ok(kind == 0 ? Api<T>::rsum(ctx(), in, out, outer, ax, inner)
                  : kind == 2 ? Api<T>::rmax(ctx(), in, out, outer, ax, inner) : Api<T>::rmin(ctx(), in, out, outer, ax, inner));
        };
        if (!axes) {
            Shape fs = keep_dims ? Shape(ndim(), 1) : Shape{};
            Ptr r = alloc(fs);
            launch(ptr_, r->ptr_, 1, (int64_t)size(), 1);
            return r;
        }
        if (axes->empty()) throw Error("Empty axes list provided");
        for (size_t a : *axes)
            if (a >= ndim()) {
                std::ostringstream m;
                m << "Axis " << a << " is out of bounds for tensor with " << ndim() << " dimensions";
                throw Error(m.str());
            }
        std::vector<size_t> sorted = *axes;
        std::sort(sorted.begin(), sorted.end(), std::greater<size_t>());
        sorted.erase(std::unique(sorted.begin(), sorted.end()), sorted.end());
        Shape final_shape = shape_;
        if (keep_dims) for (size_t a : sorted) final_shape[a] = 1;
        else for (size_t a : sorted) final_shape.erase(final_shape.begin() + a);
        Shape cur = shape_;
        const T* src = ptr_;
        Ptr tmp, out;
        for (size_t i = 0; i < sorted.size(); ++i) {
            int64_t outer, ax, inner;
            oai(cur, sorted[i], outer, ax, inner);
            cur.erase(cur.begin() + sorted[i]);
            out = alloc(i + 1 == sorted.size() ? final_shape : cur);
            launch(src, out->ptr_, outer, ax, inner);
            tmp = std::move(out);
            src = tmp->ptr_;
        }
        return tmp;
    }

    Shape shape_;
    T* ptr_ = nullptr;
    uint64_t id_ = 0;
    int64_t granted_ = 0;
    bool borrowed_ = false;
    mutable std::shared_ptr<void> owner_;  // set once the block has more than one owner (share_clones)
};

// Tensor<T> (src/backend/tensor.rs:20-26) is a device tag plus a boxed storage; every method forwards to the
// storage (e.g. tensor.rs:441-456, 1393-1411).  On this backend the façade adds nothing, so the operator layer
// works on the storage handle directly.
template <typename T> using Tensor = std::unique_ptr<HipStorage<T>>;

}  // namespace ferrox
