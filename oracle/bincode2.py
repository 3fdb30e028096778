"""Optimizer state dictionary in the reference's on-disk format (test infrastructure only).

The reference saves `OptimizerStateDict` (src/nn/optim/mod.rs:263-326) with `bincode::encode_to_vec(self,
config::standard())`; bincode is a third-party crate (Cargo.toml:19, bincode 2.0.1) that is not in the reference tree,
so this restates its published wire format (bincode 2 specification, "standard" configuration):
  * little endian, variable-length integers: u < 251 -> one byte; else a marker byte 251 / 252 / 253 / 254 followed
    by the value as u16 / u32 / u64 / u128 (the smallest that holds it); usize and u64 travel as such varints;
  * f32 / f64: their IEEE-754 bytes; bool / u8: one byte; String: varint length + UTF-8; Vec / HashMap: varint length
    + items / (key, value) pairs; Option: 0u8, or 1u8 + value; enum: variant index as a varint u32 + its fields;
    struct: its fields in declaration order.
Schema (field order as declared): OptimizerStateDict { optimizer_type: String, step_count: u64, hyperparameters:
HashMap<String, f64>, parameter_buffers: HashMap<String, TensorBuffer>, parameter_groups: Vec<SerializableParameter
Group> }; TensorBuffer { data: TensorData (enum F32(Vec<f32>) = 0 | F64(Vec<f64>) = 1), shape: Vec<usize>, device: Device
(enum CPU = 0 | CUDA(usize) = 1, src/backend/device.rs:8-13), buffer_type: String, node_id: usize };
SerializableParameterGroup { params: Vec<usize>, lr, weight_decay, momentum: Option<f64>, name: String } (mod.rs:108-197).

PARITY UNPINNED: the reference holds no serialized bytes (its only use is a round trip, mod.rs:384-398) and no Rust
toolchain exists here to produce any; the integer rule is checked against the examples of the bincode specification,
everything else only by round trips and by agreement between this file and the C++ writer/reader.  A Rust HashMap
iterates in a per-process random order, so the byte stream of the reference is not unique; readers here accept any
order, writers emit keys sorted."""
import struct

import numpy as np


def enc_varint(u):
    u = int(u)
    if u < 0:
        raise ValueError("unsigned value expected")
    if u < 251:
        return bytes([u])
    if u < 1 << 16:
        return b"\xfb" + struct.pack("<H", u)
    if u < 1 << 32:
        return b"\xfc" + struct.pack("<I", u)
    if u < 1 << 64:
        return b"\xfd" + struct.pack("<Q", u)
    return b"\xfe" + u.to_bytes(16, "little")


class Reader:
    def __init__(self, data):
        self.b = memoryview(bytes(data))
        self.i = 0

    def take(self, n):
        if self.i + n > len(self.b):
            raise ValueError("unexpected end of data")
        v = self.b[self.i:self.i + n]
        self.i += n
        return v

    def varint(self):
        t = self.take(1)[0]
        if t < 251:
            return t
        if t == 251:
            return struct.unpack("<H", self.take(2))[0]
        if t == 252:
            return struct.unpack("<I", self.take(4))[0]
        if t == 253:
            return struct.unpack("<Q", self.take(8))[0]
        if t == 254:
            return int.from_bytes(self.take(16), "little")
        raise ValueError("invalid integer marker 255")

    def string(self):
        return bytes(self.take(self.varint())).decode("utf-8")

    def f64(self):
        return struct.unpack("<d", self.take(8))[0]

    def opt_f64(self):
        tag = self.take(1)[0]
        if tag > 1:
            raise ValueError("invalid Option tag")
        return self.f64() if tag else None


def enc_string(s):
    raw = s.encode("utf-8")
    return enc_varint(len(raw)) + raw


def enc_opt_f64(v):
    return b"\x00" if v is None else b"\x01" + struct.pack("<d", v)


def enc_tensor_buffer(buf):
    """buf: dict(data=np.ndarray f32|f64, shape=[...], device=None (CPU) | int (CUDA id), buffer_type=str, node_id=int)."""
    data = np.ascontiguousarray(buf["data"])
    if data.dtype == np.float32:
        out = enc_varint(0)
    elif data.dtype == np.float64:
        out = enc_varint(1)
    else:
        raise TypeError("f32 / f64 only")
    out += enc_varint(data.size) + data.astype(data.dtype.newbyteorder("<")).tobytes()
    out += enc_varint(len(buf["shape"])) + b"".join(enc_varint(d) for d in buf["shape"])
    out += enc_varint(0) if buf["device"] is None else enc_varint(1) + enc_varint(buf["device"])
    return out + enc_string(buf["buffer_type"]) + enc_varint(buf["node_id"])


def dec_tensor_buffer(r):
    variant = r.varint()
    if variant not in (0, 1):
        raise ValueError("unknown TensorData variant")
    dt = np.dtype("<f4") if variant == 0 else np.dtype("<f8")
    n = r.varint()
    data = np.frombuffer(bytes(r.take(n * dt.itemsize)), dt).astype(dt.newbyteorder("="))
    shape = [r.varint() for _ in range(r.varint())]
    dev = r.varint()
    if dev not in (0, 1):
        raise ValueError("unknown Device variant")
    device = None if dev == 0 else r.varint()
    return dict(data=data, shape=shape, device=device, buffer_type=r.string(), node_id=r.varint())


def encode_state_dict(sd):
    """sd: dict(optimizer_type, step_count, hyperparameters {name: float}, parameter_buffers {key: buffer dict},
    parameter_groups [dict(params=[ids], lr, weight_decay, momentum, name)]).  Map keys are written sorted."""
    out = enc_string(sd["optimizer_type"]) + enc_varint(sd["step_count"])
    out += enc_varint(len(sd["hyperparameters"]))
    for k in sorted(sd["hyperparameters"]):
        out += enc_string(k) + struct.pack("<d", sd["hyperparameters"][k])
    out += enc_varint(len(sd["parameter_buffers"]))
    for k in sorted(sd["parameter_buffers"]):
        out += enc_string(k) + enc_tensor_buffer(sd["parameter_buffers"][k])
    out += enc_varint(len(sd["parameter_groups"]))
    for g in sd["parameter_groups"]:
        out += enc_varint(len(g["params"])) + b"".join(enc_varint(p) for p in g["params"])
        out += enc_opt_f64(g["lr"]) + enc_opt_f64(g["weight_decay"]) + enc_opt_f64(g["momentum"]) + enc_string(g["name"])
    return out


def decode_state_dict(data):
    r = Reader(data)
    sd = dict(optimizer_type=r.string(), step_count=r.varint())
    sd["hyperparameters"] = {}
    for _ in range(r.varint()):
        k = r.string()
        sd["hyperparameters"][k] = r.f64()
    sd["parameter_buffers"] = {}
    for _ in range(r.varint()):
        k = r.string()
        sd["parameter_buffers"][k] = dec_tensor_buffer(r)
    sd["parameter_groups"] = []
    for _ in range(r.varint()):
        params = [r.varint() for _ in range(r.varint())]
        sd["parameter_groups"].append(dict(params=params, lr=r.opt_f64(), weight_decay=r.opt_f64(), momentum=r.opt_f64(),
                                           name=r.string()))
    if r.i != len(r.b):
        raise ValueError("trailing bytes")  # decode_from_slice would report them as unread; the files here have none
    return sd
