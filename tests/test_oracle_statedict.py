"""The optimizer state dictionary's byte format as restated in oracle/bincode2.py (CPU only).
Integer markers and the length-prefixed layouts are checked against the rules and examples of the bincode 2
specification (standard configuration); the reference itself holds no serialized bytes, so the format as a whole is
'parity unpinned' beyond that and round trips."""
import struct

import numpy as np
import pytest

from oracle import bincode2 as bc


def test_varint_markers_follow_the_bincode_specification():
    assert bc.enc_varint(0) == b"\x00" and bc.enc_varint(250) == b"\xfa"
    assert bc.enc_varint(251) == b"\xfb\xfb\x00"                      # first value that needs the u16 form
    assert bc.enc_varint(65535) == b"\xfb\xff\xff"
    assert bc.enc_varint(65536) == b"\xfc\x00\x00\x01\x00"            # u32 form
    assert bc.enc_varint(2 ** 32 - 1) == b"\xfc\xff\xff\xff\xff"
    assert bc.enc_varint(2 ** 32) == b"\xfd" + struct.pack("<Q", 2 ** 32)
    assert bc.enc_varint(2 ** 64) == b"\xfe" + (2 ** 64).to_bytes(16, "little")
    for v in (0, 1, 250, 251, 252, 65535, 65536, 2 ** 32 - 1, 2 ** 32, 2 ** 63 + 5, 2 ** 64 - 1):
        r = bc.Reader(bc.enc_varint(v))
        assert r.varint() == v and r.i == len(r.b)
    with pytest.raises(ValueError):
        bc.Reader(b"\xff").varint()


def test_strings_sequences_and_options():
    assert bc.enc_string("Hello") == b"\x05Hello"                     # length as a varint, then the UTF-8 bytes
    assert bc.enc_string("") == b"\x00"
    assert bc.enc_opt_f64(None) == b"\x00"
    assert bc.enc_opt_f64(1.5) == b"\x01" + struct.pack("<d", 1.5)
    buf = dict(data=np.array([1.0, -2.0], np.float32), shape=[2], device=None, buffer_type="m", node_id=7)
    # TensorData::F32 = variant 0, Vec<f32> of 2, shape Vec<usize> [2], Device::CPU = variant 0, "m", node 7
    assert bc.enc_tensor_buffer(buf) == (b"\x00\x02" + struct.pack("<ff", 1.0, -2.0) + b"\x01\x02" + b"\x00" + b"\x01m" + b"\x07")
    buf = dict(data=np.array([0.5], np.float64), shape=[1, 1], device=3, buffer_type="second_moment", node_id=300)
    assert bc.enc_tensor_buffer(buf) == (b"\x01\x01" + struct.pack("<d", 0.5) + b"\x02\x01\x01" + b"\x01\x03" +
                                         b"\x0dsecond_moment" + b"\xfb\x2c\x01")


def example_state(dtype):
    rng = np.random.default_rng(3)
    bufs = {}
    for node, shape in ((4, [3, 2]), (5, [3]), (260, [2, 1, 2])):
        for kind in ("first_moment", "second_moment"):
            bufs[f"{node}_{kind}"] = dict(data=rng.standard_normal(int(np.prod(shape))).astype(dtype), shape=shape, device=0,
                                          buffer_type=kind, node_id=node)
    return dict(optimizer_type="Adam", step_count=12345, hyperparameters={"lr": 1e-3, "beta1": 0.9, "beta2": 0.999, "eps": 1e-8,
                                                                         "weight_decay": 0.0, "amsgrad": 0.0},
                parameter_buffers=bufs,
                parameter_groups=[dict(params=[4, 5, 260], lr=None, weight_decay=0.01, momentum=None, name="default")])


def same_state(a, b):
    assert a["optimizer_type"] == b["optimizer_type"] and a["step_count"] == b["step_count"]
    assert a["hyperparameters"] == b["hyperparameters"] and a["parameter_groups"] == b["parameter_groups"]
    assert a["parameter_buffers"].keys() == b["parameter_buffers"].keys()
    for k, x in a["parameter_buffers"].items():
        y = b["parameter_buffers"][k]
        assert x["shape"] == y["shape"] and x["device"] == y["device"] and x["buffer_type"] == y["buffer_type"] and x["node_id"] == y["node_id"]
        assert x["data"].dtype == y["data"].dtype and np.array_equal(x["data"], y["data"])


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_state_dict_round_trip_and_layout(dtype):
    sd = example_state(dtype)
    raw = bc.encode_state_dict(sd)
    assert raw.startswith(b"\x04Adam" + b"\xfb\x39\x30" + b"\x06")     # "Adam", 12345 as marker + u16, 6 hyperparameters
    same_state(bc.decode_state_dict(raw), sd)
    assert bc.encode_state_dict(bc.decode_state_dict(raw)) == raw
    with pytest.raises(ValueError):
        bc.decode_state_dict(raw[:-1])
    with pytest.raises(ValueError):
        bc.decode_state_dict(raw + b"\x00")


def test_reader_accepts_any_map_order():
    """A Rust HashMap is written in its iteration order, which differs from run to run."""
    sd = example_state(np.float32)
    out = bc.enc_string(sd["optimizer_type"]) + bc.enc_varint(sd["step_count"])
    out += bc.enc_varint(len(sd["hyperparameters"]))
    for k in sorted(sd["hyperparameters"], reverse=True):
        out += bc.enc_string(k) + struct.pack("<d", sd["hyperparameters"][k])
    out += bc.enc_varint(len(sd["parameter_buffers"]))
    for k in sorted(sd["parameter_buffers"], key=lambda s: s[::-1]):
        out += bc.enc_string(k) + bc.enc_tensor_buffer(sd["parameter_buffers"][k])
    g = sd["parameter_groups"][0]
    out += bc.enc_varint(1) + bc.enc_varint(3) + b"".join(bc.enc_varint(p) for p in g["params"])
    out += bc.enc_opt_f64(None) + bc.enc_opt_f64(0.01) + bc.enc_opt_f64(None) + bc.enc_string("default")
    same_state(bc.decode_state_dict(out), sd)
