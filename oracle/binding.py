"""ctypes binding + numpy conveniences for libferrox_oracle.so (the CPU oracle; test infrastructure only).

Each helper takes and returns numpy arrays.  The C functions they call cite the Ferrox source
lines they restate (see ferrox_oracle.cpp).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libferrox_oracle.so")

BINARY_OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3, "equal": 4, "greater": 5, "greater_equal": 6, "less": 7,
              "less_equal": 8, "min": 9, "max": 10, "pow": 11}
UNARY_OPS = {"neg": 0, "sqrt": 1, "exp": 2, "log": 3, "relu": 4, "sigmoid": 5, "tanh": 6, "abs": 7, "reciprocal": 8,
             "sign": 9, "logical_not": 10}
SCALAR_OPS = {"add_scalar": 0, "sub_scalar": 1, "mul_scalar": 2, "div_scalar": 3, "greater_scalar": 4,
              "greater_equal_scalar": 5, "less_equal_scalar": 6, "less_scalar": 7, "pow_scalar": 8}


def build():
    """Compile the oracle with its Makefile (gcc only; nothing from the reference tree is needed)."""
    subprocess.check_call(["make", "-C", _HERE, "-s"], stdout=subprocess.DEVNULL)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    return C.CDLL(_LIB_PATH)


_lib = _load()
_i64 = C.c_int64


def _sfx(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "f32", C.c_float
    if dtype == np.float64:
        return "f64", C.c_double
    raise TypeError(f"oracle supports float32/float64 only, got {dtype}")


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _c(a, dtype=None):
    return np.ascontiguousarray(a, dtype=dtype)


def _fn(name, dtype):
    s, _ = _sfx(dtype)
    return getattr(_lib, f"{name}_{s}")


def out_hw(H, W, kh, kw, sh, sw, ph, pw):
    return (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1


def im2col(x, kernel, stride, padding):
    x = _c(x)
    B, Cc, H, W = x.shape
    (kh, kw), (sh, sw), (ph, pw) = kernel, stride, padding
    oh, ow = out_hw(H, W, kh, kw, sh, sw, ph, pw)
    col = np.empty((Cc * kh * kw, B * oh * ow), dtype=x.dtype)
    _fn("orc_im2col", x.dtype)(_p(x), *[_i64(v) for v in (B, Cc, H, W, kh, kw, sh, sw, ph, pw)], _p(col))
    return col


def col2im(col, out_shape, kernel, stride, padding, layout):
    """layout 0: row-major [C*kh*kw, B*L] (what im2col produces); 1: the reference's batch-major read."""
    col = _c(col)
    B, Cc, H, W = out_shape
    (kh, kw), (sh, sw), (ph, pw) = kernel, stride, padding
    out = np.empty(out_shape, dtype=col.dtype)
    _fn("orc_col2im", col.dtype)(_p(col), *[_i64(v) for v in (B, Cc, H, W, kh, kw, sh, sw, ph, pw)], _p(out),
                                 C.c_int(layout))
    return out


def gemm(a, b, ta=False, tb=False, naive=False):
    a, b = _c(a), _c(b)
    M = a.shape[1] if ta else a.shape[0]
    K = a.shape[0] if ta else a.shape[1]
    N = b.shape[0] if tb else b.shape[1]
    assert (b.shape[1] if tb else b.shape[0]) == K
    c = np.empty((M, N), dtype=a.dtype)
    _fn("orc_gemm_naive" if naive else "orc_gemm", a.dtype)(C.c_int(ta), C.c_int(tb), _i64(M), _i64(N), _i64(K), _p(a),
                                                           _p(b), _p(c))
    return c


def conv2d_fwd(x, w, stride, padding):
    x, w = _c(x), _c(w)
    B, Cin, H, W = x.shape
    Cout, _, kh, kw = w.shape
    (sh, sw), (ph, pw) = stride, padding
    oh, ow = out_hw(H, W, kh, kw, sh, sw, ph, pw)
    y = np.empty((B, Cout, oh, ow), dtype=x.dtype)
    _fn("orc_conv2d_fwd", x.dtype)(_p(x), _p(w), _p(y), *[_i64(v) for v in (B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw)])
    return y


def conv2d_dgrad(g, w, x_shape, stride, padding, mode):
    """mode 0 = mathematically correct gradient; 1 = literal restatement of the CPU backend (batch-1 only correct)."""
    g, w = _c(g), _c(w)
    B, Cin, H, W = x_shape
    Cout, _, kh, kw = w.shape
    (sh, sw), (ph, pw) = stride, padding
    dx = np.empty(x_shape, dtype=g.dtype)
    _fn("orc_conv2d_dgrad", g.dtype)(_p(g), _p(w), _p(dx), *[_i64(v) for v in (B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw)],
                                     C.c_int(mode))
    return dx


def conv2d_wgrad(x, g, w_shape, stride, padding, mode):
    x, g = _c(x), _c(g)
    B, Cin, H, W = x.shape
    Cout, _, kh, kw = w_shape
    (sh, sw), (ph, pw) = stride, padding
    dw = np.empty(w_shape, dtype=x.dtype)
    _fn("orc_conv2d_wgrad", x.dtype)(_p(x), _p(g), _p(dw), *[_i64(v) for v in (B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw)],
                                     C.c_int(mode))
    return dw


def binary(op, a, b):
    a, b = _c(a), _c(b)
    o = np.empty_like(a)
    _fn("orc_binary", a.dtype)(C.c_int(BINARY_OPS[op]), _p(a), _p(b), _p(o), _i64(a.size))
    return o


def scalar(op, a, s):
    a = _c(a)
    o = np.empty_like(a)
    _, ct = _sfx(a.dtype)
    _fn("orc_scalar", a.dtype)(C.c_int(SCALAR_OPS[op]), _p(a), ct(s), _p(o), _i64(a.size))
    return o


def unary(op, a):
    a = _c(a)
    o = np.empty_like(a)
    _fn("orc_unary", a.dtype)(C.c_int(UNARY_OPS[op]), _p(a), _p(o), _i64(a.size))
    return o


def clamp(a, lo, hi):
    a = _c(a)
    o = np.empty_like(a)
    _, ct = _sfx(a.dtype)
    _fn("orc_clamp", a.dtype)(_p(a), ct(lo), ct(hi), _p(o), _i64(a.size))
    return o


def relu_bwd(g, x):
    g, x = _c(g), _c(x)
    o = np.empty_like(g)
    _fn("orc_relu_bwd", g.dtype)(_p(g), _p(x), _p(o), _i64(g.size))
    return o


def sigmoid_bwd(g, s, literal):
    g, s = _c(g), _c(s)
    o = np.empty_like(g)
    _fn("orc_sigmoid_bwd", g.dtype)(_p(g), _p(s), _p(o), _i64(g.size), C.c_int(int(literal)))
    return o


def tanh_bwd(g, t):
    g, t = _c(g), _c(t)
    o = np.empty_like(g)
    _fn("orc_tanh_bwd", g.dtype)(_p(g), _p(t), _p(o), _i64(g.size))
    return o


def _oai(shape, axis):
    outer = int(np.prod(shape[:axis], dtype=np.int64))
    inner = int(np.prod(shape[axis + 1:], dtype=np.int64))
    return outer, int(shape[axis]), inner


def reduce_axis(kind, x, axis, want_idx=False):
    """kind in {'sum','mean','max','min','prod'} over ONE axis of a contiguous array (keep_dims False)."""
    x = _c(x)
    outer, ax, inner = _oai(x.shape, axis)
    out_shape = x.shape[:axis] + x.shape[axis + 1:]
    out = np.empty(out_shape, dtype=x.dtype)
    if kind in ("max", "min"):
        idx = np.empty(out_shape, dtype=np.int64)
        _fn("orc_reduce_" + kind, x.dtype)(_p(x), _i64(outer), _i64(ax), _i64(inner), _p(out), _p(idx))
        return (out, idx) if want_idx else out
    _fn("orc_reduce_" + kind, x.dtype)(_p(x), _i64(outer), _i64(ax), _i64(inner), _p(out))
    return out


def reduce(kind, x, axes=None, keep_dims=False):
    """Multi-axis reduction in the reference's order: axes sorted descending, one at a time
    (cpu.rs:85-95); None = every axis from last to first (cpu.rs:115-117).  mean = sum * T(1/n)."""
    x = _c(x)
    shape = x.shape
    order = sorted(set(axes), reverse=True) if axes is not None else list(range(x.ndim - 1, -1, -1))
    r = x
    base = "sum" if kind == "mean" else kind
    for ax in order:
        r = reduce_axis(base, r, ax)
    if kind == "mean":
        n = float(np.prod([shape[a] for a in (axes if axes is not None else range(x.ndim))]))
        r = scalar("mul_scalar", r, x.dtype.type(1.0 / n))
    if keep_dims:
        fs = list(shape)
        for a in (axes if axes is not None else range(x.ndim)):
            fs[a] = 1
        r = r.reshape(fs)
    return r


def splitmix64_uniform(seed, n):
    """u_i in [0,1), i < n: the top 53 bits of splitmix64(seed + i) (Steele, Lea & Flood 2014) as a float64."""
    with np.errstate(over="ignore"):
        z = np.uint64(seed) + np.arange(n, dtype=np.uint64) + np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    return (z >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)


def dropout_mask(shape, p, seed, dtype):
    """create_dropout_mask (nn/layers/dropout.rs:56-82): one f64 uniform per element, keep when u < 1 - p,
    mask = T(1/(1-p)) or 0.  The reference draws from an unseeded generator; element i takes splitmix64(seed + i)."""
    n = int(np.prod(shape))
    keep = 1.0 - p
    u = splitmix64_uniform(seed, n)
    return np.where(u < keep, np.dtype(dtype).type(1.0 / keep), np.dtype(dtype).type(0)).astype(dtype).reshape(shape)


def in_range(a, lo, hi):
    a = _c(a)
    o = np.empty_like(a)
    _, ct = _sfx(a.dtype)
    _fn("orc_in_range", a.dtype)(_p(a), ct(lo), ct(hi), _p(o), _i64(a.size))
    return o


def softmax_all(x):
    """Whole-tensor softmax (cpu.rs:1018-1036): the tensor as one row."""
    x = _c(x)
    return softmax_axis(x.reshape(1, -1), 1).reshape(x.shape)


def pool2d(x, kernel, stride, padding, is_max):
    """maxpool2d / avgpool2d (extensions/pooling.rs:154-229) on [N,C,H,W]."""
    x = _c(x)
    N, Cc, H, W = x.shape
    (kh, kw), (sh, sw), (ph, pw) = kernel, stride, padding
    oh, ow = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
    out = np.empty((N, Cc, oh, ow), x.dtype)
    _fn("orc_pool2d", x.dtype)(_p(x), _p(out), *[_i64(v) for v in (N, Cc, H, W, kh, kw, sh, sw, ph, pw)], C.c_int(int(is_max)))
    return out


def unpool2d(grad_out, x, pooled, kernel, stride, padding, is_max):
    """max_unpool2d / avg_unpool2d (extensions/pooling.rs:339-418): gradient w.r.t. the pooling input."""
    x, grad_out, pooled = _c(x), _c(grad_out), _c(pooled)
    N, Cc, H, W = x.shape
    (kh, kw), (sh, sw), (ph, pw) = kernel, stride, padding
    gin = np.empty_like(x)
    _fn("orc_unpool2d", x.dtype)(_p(grad_out), _p(x), _p(pooled), _p(gin), *[_i64(v) for v in (N, Cc, H, W, kh, kw, sh, sw, ph, pw)],
                                 C.c_int(int(is_max)))
    return gin


def softmax_axis(x, axis):
    x = _c(x)
    outer, ax, inner = _oai(x.shape, axis)
    out = np.empty_like(x)
    _fn("orc_softmax_axis", x.dtype)(_p(x), _i64(outer), _i64(ax), _i64(inner), _p(out))
    return out


def materialize(x, shape, strides):
    """Gather a strided view (element strides, 0 for broadcast dims) of flat buffer x into a contiguous array."""
    x = _c(x)
    n = int(np.prod(shape, dtype=np.int64))
    out = np.empty(shape, dtype=x.dtype)
    sh = (C.c_int64 * len(shape))(*shape)
    st = (C.c_int64 * len(shape))(*strides)
    _fn("orc_materialize", x.dtype)(_p(x), _p(out), sh, st, C.c_int(len(shape)), _i64(n))
    return out


# ---------------------------------------------------------------------------------------------
# allocator state machine
# ---------------------------------------------------------------------------------------------
DEFAULT_BUCKETS = [  # src/backend/memory/mod.rs:50-82  (lo, hi, cap, to_evict, threshold_ms or -1)
    (1, 1024, 500, 50, -1),
    (1025, 262144, 50, 15, -1),
    (262145, 16777216, 10, 5, -1),
    (16777217, 2**62, 2, 2, -1),
]

_lib.orc_pool_new.restype = C.c_void_p


class Pool:
    def __init__(self, buckets=None, literal=True):
        b = buckets or DEFAULT_BUCKETS
        arr = lambda k: (C.c_int64 * len(b))(*[row[k] for row in b])  # noqa: E731
        self._h = C.c_void_p(_lib.orc_pool_new(C.c_int(len(b)), arr(0), arr(1), arr(2), arr(3), arr(4),
                                               C.c_int(int(literal))))
        self.nb = len(b)

    def __del__(self):
        if getattr(self, "_h", None):
            _lib.orc_pool_delete(self._h)
            self._h = None

    def tick(self, dt=1):
        _lib.orc_pool_tick(self._h, C.c_uint64(dt))

    def alloc(self, size):
        g, i = C.c_int64(0), C.c_uint64(0)
        rc = _lib.orc_pool_alloc(self._h, _i64(size), C.byref(g), C.byref(i))
        if rc != 0:
            raise ValueError({-1: "Cannot allocate zero-sized CUDA memory", -2: "No bucket configured"}[rc])
        return g.value, i.value

    def free(self, size, alloc_id):
        return _lib.orc_pool_free(self._h, _i64(size), C.c_uint64(alloc_id))

    def cleanup(self):
        _lib.orc_pool_cleanup(self._h)

    def reset(self):
        _lib.orc_pool_reset(self._h)

    def stats(self):
        out = (C.c_int64 * 8)()
        _lib.orc_pool_stats(self._h, out)
        keys = ("total_allocations", "active_allocations", "pool_hits", "pool_misses", "underflow_misses",
                "active_table_len", "device_allocs", "device_frees")
        return dict(zip(keys, list(out)))

    def bucket_stats(self, i):
        out = (C.c_int64 * 5)()
        _lib.orc_pool_bucket_stats(self._h, C.c_int(i), out)
        keys = ("pooled", "total_allocations", "total_evictions", "av_allocations", "max_allocations")
        return dict(zip(keys, list(out)))
