"""ctypes binding of libferrox_hip.so (see include/ferrox_hip.h) plus a small numpy-facing convenience layer.

The binding is deliberately thin: `lib.fx_<name>` are the raw C entry points with argtypes set; `Context`
wraps a `fx_ctx*` and offers upload/download and one Python method per kernel family so tests and the
benchmark read like the C calls they make.  There is no CPU fallback: if the library cannot be loaded the
import raises.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libferrox_hip.so")

FX_F32, FX_F64 = 0, 1
CONV_FWD, CONV_DGRAD, CONV_WGRAD = 0, 1, 2
BINARY_OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3, "equal": 4, "greater": 5, "greater_equal": 6, "less": 7,
              "less_equal": 8, "min": 9, "max": 10, "pow": 11}
UNARY_OPS = {"neg": 0, "sqrt": 1, "exp": 2, "log": 3, "relu": 4, "sigmoid": 5, "tanh": 6, "abs": 7, "reciprocal": 8,
             "sign": 9, "logical_not": 10}
SCALAR_OPS = {"add_scalar": 0, "sub_scalar": 1, "mul_scalar": 2, "div_scalar": 3, "greater_scalar": 4,
              "greater_equal_scalar": 5, "less_equal_scalar": 6, "less_scalar": 7, "pow_scalar": 8}
FX_MAX_BUCKETS = 8


class BucketConfig(C.Structure):
    _fields_ = [("min_elems", C.c_int64), ("max_elems", C.c_int64), ("max_blocks", C.c_int64), ("to_evict", C.c_int64),
                ("eviction_threshold_ms", C.c_int64)]


class PoolConfig(C.Structure):
    _fields_ = [("n_buckets", C.c_int32), ("literal_ids", C.c_int32), ("best_fit", C.c_int32), ("reserved", C.c_int32),
                ("buckets", BucketConfig * FX_MAX_BUCKETS)]


class PoolStats(C.Structure):
    _fields_ = [(n, C.c_int64) for n in ("total_allocations", "active_allocations", "pool_hits", "pool_misses",
                                         "underflow_misses", "allocation_counter", "active_table_len", "device_allocs",
                                         "device_frees", "bytes_in_use", "bytes_pooled", "peak_bytes")]

    def as_dict(self):
        return {n: getattr(self, n) for n, _ in self._fields_}


class BucketStats(C.Structure):
    _fields_ = [(n, C.c_int64) for n in ("pooled_blocks", "total_allocations", "total_evictions", "av_allocations",
                                         "max_allocations")]

    def as_dict(self):
        return {n: getattr(self, n) for n, _ in self._fields_}


def _load():
    if not os.path.exists(LIB_PATH):
        from . import build as _build  # build only when nothing is built yet
        _build.build()
    return C.CDLL(LIB_PATH)


lib = _load()

_vp, _i64, _int, _u64 = C.c_void_p, C.c_int64, C.c_int, C.c_uint64


def _sig(name, *argtypes, restype=C.c_int):
    fn = getattr(lib, name)
    fn.argtypes = list(argtypes)
    fn.restype = restype
    return fn


_sig("fx_init", _int, C.POINTER(PoolConfig), C.POINTER(_vp))
_sig("fx_destroy", _vp)
_sig("fx_sync", _vp)
_sig("fx_device_name", _vp, C.c_char_p, _i64)
_sig("fx_last_error", restype=C.c_char_p)
_sig("fx_stream", _vp, restype=_vp)
_sig("fx_timer_start", _vp)
_sig("fx_timer_stop", _vp, C.POINTER(C.c_float))
_sig("fx_alloc", _vp, _int, _i64, C.POINTER(_vp), C.POINTER(_i64), C.POINTER(_u64))
_sig("fx_free", _vp, _int, _vp, _u64)
_sig("fx_pool_cleanup", _vp, _int)
_sig("fx_pool_reset", _vp, _int)
_sig("fx_pool_stats_get", _vp, _int, C.POINTER(PoolStats))
_sig("fx_pool_bucket_stats_get", _vp, _int, _int, C.POINTER(BucketStats))
_sig("fx_h2d", _vp, _vp, _vp, _i64)
_sig("fx_d2h", _vp, _vp, _vp, _i64)
_sig("fx_d2d", _vp, _vp, _vp, _i64)
_sig("fx_scratch_info", _vp, C.POINTER(_vp), C.POINTER(_i64), C.POINTER(_i64), C.POINTER(_i64))
_sig("fx_device_mem_info", _vp, C.POINTER(_i64), C.POINTER(_i64))
_sig("fx_conv2d_bwd_relu_supported", _vp, _int, _int, *([_i64] * 11))
_sig("fx_conv2d_last_path", _vp, restype=C.c_char_p)
_sig("fx_conv2d_workspace_bytes", _int, _int, _int, *([_i64] * 11), restype=_i64)

_CONV_INTS = [_i64] * 11
for _s, _ct in (("f32", C.c_float), ("f64", C.c_double)):
    _sig(f"fx_fill_{_s}", _vp, _vp, _ct, _i64)
    _sig(f"fx_fill_uniform_{_s}", _vp, _vp, _i64, _u64, _ct, _ct)
    _sig(f"fx_fill_normal_{_s}", _vp, _vp, _i64, _u64, _ct, _ct)
    _sig(f"fx_materialize_{_s}", _vp, _vp, _vp, C.POINTER(_i64), C.POINTER(_i64), _int, _i64)
    _sig(f"fx_binary_{_s}", _vp, _int, _vp, _vp, _vp, _i64)
    for _n in ("add", "sub", "mul", "div", "equal"):
        _sig(f"fx_{_n}_{_s}", _vp, _vp, _vp, _vp, _i64)
    _sig(f"fx_scalar_{_s}", _vp, _int, _vp, _ct, _vp, _i64)
    for _n in ("add_scalar", "sub_scalar", "mul_scalar", "div_scalar", "greater_scalar", "greater_equal_scalar",
               "less_equal_scalar"):
        _sig(f"fx_{_n}_{_s}", _vp, _vp, _ct, _vp, _i64)
    _sig(f"fx_unary_{_s}", _vp, _int, _vp, _vp, _i64)
    for _n in ("neg", "sqrt", "exp", "log", "relu", "sigmoid", "tanh"):
        _sig(f"fx_{_n}_{_s}", _vp, _vp, _vp, _i64)
    _sig(f"fx_clamp_{_s}", _vp, _vp, _ct, _ct, _vp, _i64)
    _sig(f"fx_relu_bwd_{_s}", _vp, _vp, _vp, _vp, _i64)
    _sig(f"fx_sigmoid_bwd_{_s}", _vp, _vp, _vp, _vp, _i64, _int)
    _sig(f"fx_tanh_bwd_{_s}", _vp, _vp, _vp, _vp, _i64)
    _sig(f"fx_softmax_axis_{_s}", _vp, _vp, _vp, _i64, _i64, _i64)
    _sig(f"fx_reduce_sum_{_s}", _vp, _vp, _vp, _i64, _i64, _i64)
    _sig(f"fx_reduce_mean_{_s}", _vp, _vp, _vp, _i64, _i64, _i64)
    _sig(f"fx_reduce_max_{_s}", _vp, _vp, _vp, _vp, _i64, _i64, _i64)
    _sig(f"fx_reduce_min_{_s}", _vp, _vp, _vp, _vp, _i64, _i64, _i64)
    _sig(f"fx_reduce_prod_{_s}", _vp, _vp, _vp, _i64, _i64, _i64)
    _sig(f"fx_in_range_{_s}", _vp, _vp, _ct, _ct, _vp, _i64)
    _sig(f"fx_batchnorm_stats_{_s}", _vp, _vp, _vp, _vp, _vp, _vp, C.c_double, _i64, _i64, _i64)
    _sig(f"fx_batchnorm_fwd_{_s}", _vp, _vp, _vp, _vp, _vp, _vp, C.c_double, _vp, _i64, _i64, _i64, _int)
    _sig(f"fx_batchnorm_bwd_{_s}", _vp, _vp, _vp, _vp, _vp, _vp, _vp, C.c_double, _vp, _vp, _vp, _i64, _i64, _i64, _int)
    _sig(f"fx_dropout_{_s}", _vp, _vp, _vp, _vp, _i64, C.c_double, _u64)
    _sig(f"fx_maxpool2d_{_s}", _vp, _vp, _vp, *([_i64] * 10))
    _sig(f"fx_avgpool2d_{_s}", _vp, _vp, _vp, *([_i64] * 10))
    _sig(f"fx_max_unpool2d_{_s}", _vp, _vp, _vp, _vp, _vp, *([_i64] * 10))
    _sig(f"fx_avg_unpool2d_{_s}", _vp, _vp, _vp, *([_i64] * 10))
    _sig(f"fx_gemm_{_s}", _vp, _int, _int, _i64, _i64, _i64, _vp, _vp, _vp)
    _sig(f"fx_im2col_{_s}", _vp, _vp, _vp, *([_i64] * 10))
    _sig(f"fx_col2im_{_s}", _vp, _vp, _vp, *([_i64] * 10), _int)
    _sig(f"fx_conv2d_fwd_{_s}", _vp, _vp, _vp, _vp, *_CONV_INTS, _vp, _i64)
    _sig(f"fx_conv2d_dgrad_{_s}", _vp, _vp, _vp, _vp, *_CONV_INTS, _int, _vp, _i64)
    _sig(f"fx_conv2d_wgrad_{_s}", _vp, _vp, _vp, _vp, *_CONV_INTS, _int, _vp, _i64)
    _sig(f"fx_conv2d_wgrad_relu_bias_{_s}", _vp, _vp, _vp, _vp, _vp, _vp, *_CONV_INTS, _vp, _i64)
    _sig(f"fx_conv2d_dgrad_relu_{_s}", _vp, _vp, _vp, _vp, _vp, *_CONV_INTS)
    _sig(f"fx_bias_act_{_s}", _vp, _vp, _vp, _i64, _i64, _i64, _int)
    _sig(f"fx_conv2d_fwd_bias_act_{_s}", _vp, _vp, _vp, _vp, _vp, *_CONV_INTS, _int, _vp, _i64)
    _sig(f"fx_gemm_bias_act_{_s}", _vp, _int, _int, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _int)
    _sig(f"fx_gemm_tn_colsum_{_s}", _vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp)
    _sig(f"fx_linear_bwd_{_s}", _vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _int)
    _sig(f"fx_bias_grad_{_s}", _vp, _vp, _vp, _i64, _i64, _i64)
    _sig(f"fx_relu_bwd_bias_grad_{_s}", _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64)
    _sig(f"fx_softmax_ce_fwd_{_s}", _vp, _vp, _vp, _vp, _vp, _i64, _i64)
    _sig(f"fx_softmax_ce_bwd_{_s}", _vp, _vp, _vp, _vp, _vp, _i64, _i64)
    _sig(f"fx_softmax_ce_fwd_unit_grad_{_s}", _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64)
    _sig(f"fx_adam_step_{_s}", _vp, _vp, _vp, _vp, _vp, _i64, *([_ct] * 7))
    _sig(f"fx_sgd_step_{_s}", _vp, _vp, _vp, _i64, _ct)
    _sig(f"fx_adam_step_multi_{_s}", _vp, _int, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_i64),
         *([_ct] * 7))
    _sig(f"fx_sgd_step_multi_{_s}", _vp, _int, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_i64), _ct)
    _sig(f"fx_adam_amsgrad_step_{_s}", _vp, _vp, _vp, _vp, _vp, _vp, _i64, *([_ct] * 7))
    _sig(f"fx_sgd_momentum_step_{_s}", _vp, _vp, _vp, _vp, _i64, _ct, _ct, _ct, _int)
    _sig(f"fx_adam_amsgrad_step_multi_{_s}", _vp, _int, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp),
         C.POINTER(_vp), C.POINTER(_i64), *([_ct] * 7))
    _sig(f"fx_sgd_momentum_step_multi_{_s}", _vp, _int, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_i64),
         _ct, _ct, _ct, _int)

    _sig(f"fx_adam_step_multi_bc_{_s}", _vp, _int, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp),
         C.POINTER(_i64), *([_ct] * 5), _vp)

_sig("fx_graph_begin", _vp)
_sig("fx_graph_end", _vp, C.POINTER(_vp))
_sig("fx_graph_launch", _vp, _vp)
_sig("fx_graph_info", _vp, C.POINTER(_i64), C.POINTER(_i64), C.POINTER(_i64))
_sig("fx_graph_destroy", _vp, _vp)
_sig("fx_host_alloc", _vp, _i64, C.POINTER(_vp))
_sig("fx_host_free", _vp, _vp)
_sig("fx_h2d_async", _vp, _vp, _vp, _i64)
_sig("fx_conv2d_tune_f32", _vp, _int, *([_i64] * 11), _int, _int)
_sig("fx_reduce_max_noalloc_f32", _vp, _vp, _vp, _vp, _i64, _i64, _i64)
NOALLOC_SCRATCH_BYTES = 4 << 20


class FerroxHipError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"[fx error {code}] {message}")
        self.code = code
        self.message = message


def check(rc):
    if rc != 0:
        raise FerroxHipError(rc, lib.fx_last_error().decode("utf-8", "replace"))


def dtype_code(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return FX_F32, "f32"
    if dtype == np.float64:
        return FX_F64, "f64"
    raise TypeError(f"only float32/float64 are supported, got {dtype}")


class DeviceArray:
    """A pool allocation with a shape (row-major).  Returned to the pool by free() or when garbage collected."""

    def __init__(self, ctx, shape, dtype, ptr, granted, alloc_id):
        self.ctx, self.shape, self.dtype = ctx, tuple(int(s) for s in shape), np.dtype(dtype)
        self.ptr, self.granted, self.alloc_id = ptr, granted, alloc_id

    @property
    def size(self):
        return int(np.prod(self.shape, dtype=np.int64))

    @property
    def nbytes(self):
        return self.size * self.dtype.itemsize

    def reshape(self, *shape):
        shape = shape[0] if len(shape) == 1 and isinstance(shape[0], (tuple, list)) else shape
        assert int(np.prod(shape, dtype=np.int64)) == self.size
        v = DeviceArray(self.ctx, shape, self.dtype, self.ptr, self.granted, None)  # non-owning view
        v._base = self
        return v

    def rows(self, lo, hi):
        """Non-owning view of the slices lo:hi along the first axis."""
        assert 0 <= lo <= hi <= self.shape[0]
        inner = int(np.prod(self.shape[1:], dtype=np.int64))
        v = DeviceArray(self.ctx, (hi - lo,) + self.shape[1:], self.dtype, self.ptr + lo * inner * self.dtype.itemsize, 0, None)
        v._base = self
        return v

    def numpy(self):
        out = np.empty(self.shape, dtype=self.dtype)
        if self.size:
            check(lib.fx_d2h(self.ctx.h, out.ctypes.data_as(_vp), self.ptr, self.nbytes))
        return out

    def free(self):
        if self.alloc_id is not None and self.ptr is not None and self.ctx.h:
            code, _ = dtype_code(self.dtype)
            check(lib.fx_free(self.ctx.h, code, self.ptr, self.alloc_id))
        self.ptr = None
        self.alloc_id = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Context:
    def __init__(self, device=0, pool_config=None):
        h = _vp()
        check(lib.fx_init(device, C.byref(pool_config) if pool_config is not None else None, C.byref(h)))
        self.h = h

    def close(self):
        if self.h:
            check(lib.fx_destroy(self.h))
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    # ---- runtime ----
    def graph_begin(self):
        """Starts recording the calls made on this context into a graph (see fx_graph_begin in the header for the rules)."""
        check(lib.fx_graph_begin(self.h))

    def graph_end(self):
        """Ends the recording; returns the graph handle for graph_launch / graph_info / graph_destroy."""
        g = _vp()
        check(lib.fx_graph_end(self.h, C.byref(g)))
        return g

    def graph_launch(self, g):
        check(lib.fx_graph_launch(self.h, g))

    def graph_info(self, g):
        n, k, h = _i64(0), _i64(0), _i64(0)
        check(lib.fx_graph_info(g, C.byref(n), C.byref(k), C.byref(h)))
        return {"nodes": n.value, "kernel_nodes": k.value, "held_blocks": h.value}

    def graph_destroy(self, g):
        check(lib.fx_graph_destroy(self.h, g))

    def scratch_info(self):
        """The library's own scratch region: address, bytes, outgrown regions parked for live graphs, live graphs."""
        cur, b, p, g = _vp(), _i64(0), _i64(0), _i64(0)
        check(lib.fx_scratch_info(self.h, C.byref(cur), C.byref(b), C.byref(p), C.byref(g)))
        return {"current": cur.value or 0, "bytes": b.value, "parked_regions": p.value, "live_graphs": g.value}

    def device_mem_info(self):
        f, t = _i64(0), _i64(0)
        check(lib.fx_device_mem_info(self.h, C.byref(f), C.byref(t)))
        return {"free": f.value, "total": t.value}

    def sync(self):
        check(lib.fx_sync(self.h))

    def device_name(self):
        buf = C.create_string_buffer(256)
        check(lib.fx_device_name(self.h, buf, 256))
        return buf.value.decode()

    def timer_start(self):
        check(lib.fx_timer_start(self.h))

    def timer_stop(self):
        ms = C.c_float(0)
        check(lib.fx_timer_stop(self.h, C.byref(ms)))
        return ms.value

    # ---- memory ----
    def empty(self, shape, dtype=np.float32):
        shape = (shape,) if isinstance(shape, (int, np.integer)) else tuple(shape)
        code, _ = dtype_code(dtype)
        n = int(np.prod(shape, dtype=np.int64))
        ptr, granted, aid = _vp(), _i64(0), _u64(0)
        check(lib.fx_alloc(self.h, code, n, C.byref(ptr), C.byref(granted), C.byref(aid)))
        return DeviceArray(self, shape, dtype, ptr.value, granted.value, aid.value)

    def upload(self, a):
        a = np.ascontiguousarray(a)
        d = self.empty(a.shape, a.dtype)
        check(lib.fx_h2d(self.h, d.ptr, a.ctypes.data_as(_vp), a.nbytes))
        return d

    def pool_stats(self, dtype=np.float32):
        st = PoolStats()
        check(lib.fx_pool_stats_get(self.h, dtype_code(dtype)[0], C.byref(st)))
        return st.as_dict()

    def bucket_stats(self, bucket, dtype=np.float32):
        st = BucketStats()
        check(lib.fx_pool_bucket_stats_get(self.h, dtype_code(dtype)[0], bucket, C.byref(st)))
        return st.as_dict()

    def pool_cleanup(self, dtype=np.float32):
        check(lib.fx_pool_cleanup(self.h, dtype_code(dtype)[0]))

    def pool_reset(self, dtype=np.float32):
        check(lib.fx_pool_reset(self.h, dtype_code(dtype)[0]))

    # ---- kernels (each allocates its output from the pool unless `out` is given) ----
    def _fn(self, name, dtype):
        return getattr(lib, f"fx_{name}_{dtype_code(dtype)[1]}")

    def fill(self, shape, value, dtype=np.float32):
        o = self.empty(shape, dtype)
        check(self._fn("fill", dtype)(self.h, o.ptr, float(value), o.size))
        return o

    def uniform(self, shape, seed, lo, hi, dtype=np.float32):
        o = self.empty(shape, dtype)
        check(self._fn("fill_uniform", dtype)(self.h, o.ptr, o.size, seed, float(lo), float(hi)))
        return o

    def normal(self, shape, seed, mean=0.0, std=1.0, dtype=np.float32):
        o = self.empty(shape, dtype)
        check(self._fn("fill_normal", dtype)(self.h, o.ptr, o.size, seed, float(mean), float(std)))
        return o

    def binary(self, op, a, b, out=None):
        assert a.shape == b.shape, f"Shape mismatch: {a.shape} vs {b.shape}"
        o = out or self.empty(a.shape, a.dtype)
        check(self._fn("binary", a.dtype)(self.h, BINARY_OPS[op], a.ptr, b.ptr, o.ptr, a.size))
        return o

    def scalar(self, op, a, s, out=None):
        o = out or self.empty(a.shape, a.dtype)
        check(self._fn("scalar", a.dtype)(self.h, SCALAR_OPS[op], a.ptr, float(s), o.ptr, a.size))
        return o

    def unary(self, op, a, out=None):
        o = out or self.empty(a.shape, a.dtype)
        check(self._fn("unary", a.dtype)(self.h, UNARY_OPS[op], a.ptr, o.ptr, a.size))
        return o

    def in_range(self, a, lo, hi):
        o = self.empty(a.shape, a.dtype)
        check(self._fn("in_range", a.dtype)(self.h, a.ptr, float(lo), float(hi), o.ptr, a.size))
        return o

    def pool2d(self, x, kernel, stride, padding, is_max):
        N, Cc, H, W = x.shape
        (kh, kw), (sh, sw), (ph, pw) = kernel, stride, padding
        o = self.empty((N, Cc, (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1), x.dtype)
        check(self._fn("maxpool2d" if is_max else "avgpool2d", x.dtype)(self.h, x.ptr, o.ptr, N, Cc, H, W, kh, kw, sh, sw, ph, pw))
        return o

    def unpool2d(self, grad_out, x, pooled, kernel, stride, padding, is_max):
        N, Cc, H, W = x.shape
        (kh, kw), (sh, sw), (ph, pw) = kernel, stride, padding
        gi = self.empty(x.shape, x.dtype)
        if is_max:
            check(self._fn("max_unpool2d", x.dtype)(self.h, grad_out.ptr, x.ptr, pooled.ptr, gi.ptr, N, Cc, H, W, kh, kw, sh, sw, ph, pw))
        else:
            check(self._fn("avg_unpool2d", x.dtype)(self.h, grad_out.ptr, gi.ptr, N, Cc, H, W, kh, kw, sh, sw, ph, pw))
        return gi

    def clamp(self, a, lo, hi):
        o = self.empty(a.shape, a.dtype)
        check(self._fn("clamp", a.dtype)(self.h, a.ptr, float(lo), float(hi), o.ptr, a.size))
        return o

    def relu_bwd(self, g, x, out=None):
        o = out or self.empty(g.shape, g.dtype)
        check(self._fn("relu_bwd", g.dtype)(self.h, g.ptr, x.ptr, o.ptr, g.size))
        return o

    def sigmoid_bwd(self, g, s, literal, out=None):
        o = out or self.empty(g.shape, g.dtype)
        check(self._fn("sigmoid_bwd", g.dtype)(self.h, g.ptr, s.ptr, o.ptr, g.size, int(literal)))
        return o

    def tanh_bwd(self, g, t, out=None):
        o = out or self.empty(g.shape, g.dtype)
        check(self._fn("tanh_bwd", g.dtype)(self.h, g.ptr, t.ptr, o.ptr, g.size))
        return o

    def materialize(self, a, shape, strides):
        n = int(np.prod(shape, dtype=np.int64))
        o = self.empty(shape, a.dtype)
        sh = (_i64 * len(shape))(*shape)
        st = (_i64 * len(shape))(*strides)
        check(self._fn("materialize", a.dtype)(self.h, a.ptr, o.ptr, sh, st, len(shape), n))
        return o

    @staticmethod
    def _oai(shape, axis):
        outer = int(np.prod(shape[:axis], dtype=np.int64))
        inner = int(np.prod(shape[axis + 1:], dtype=np.int64))
        return outer, int(shape[axis]), inner

    def reduce(self, kind, a, axis, want_idx=False, out=None):
        """kind in sum/mean/max/min/prod over ONE axis (keep_dims False)."""
        outer, ax, inner = self._oai(a.shape, axis)
        oshape = a.shape[:axis] + a.shape[axis + 1:]
        o = out or self.empty(oshape if oshape else (1,), a.dtype)
        if kind in ("max", "min"):
            idx = None
            iptr = None
            if want_idx:
                idx = _RawI64(self, max(1, outer * inner))
                iptr = idx.ptr
            check(self._fn("reduce_" + kind, a.dtype)(self.h, a.ptr, o.ptr, iptr, outer, ax, inner))
            o.shape = oshape
            if want_idx:
                return o, idx.numpy().reshape(oshape)
            return o
        check(self._fn("reduce_" + kind, a.dtype)(self.h, a.ptr, o.ptr, outer, ax, inner))
        o.shape = oshape
        return o

    def reduce_max_noalloc(self, a, axis, out, idx):
        """fx_reduce_max_noalloc_f32 into caller-provided `out` (values) and `idx` (a _RawI64 or None)."""
        outer, ax, inner = self._oai(a.shape, axis)
        check(lib.fx_reduce_max_noalloc_f32(self.h, a.ptr, out.ptr, idx.ptr if idx is not None else None, outer, ax, inner))

    def softmax_axis(self, a, axis):
        outer, ax, inner = self._oai(a.shape, axis)
        o = self.empty(a.shape, a.dtype)
        check(self._fn("softmax_axis", a.dtype)(self.h, a.ptr, o.ptr, outer, ax, inner))
        return o

    def gemm(self, a, b, ta=False, tb=False, out=None):
        M = a.shape[1] if ta else a.shape[0]
        K = a.shape[0] if ta else a.shape[1]
        N = b.shape[0] if tb else b.shape[1]
        Kb = b.shape[1] if tb else b.shape[0]
        if K != Kb:
            raise FerroxHipError(1, f"Matrix multiplication shape mismatch: ({M}, {K}) @ ({Kb}, {N})")
        o = out or self.empty((M, N), a.dtype)
        check(self._fn("gemm", a.dtype)(self.h, int(ta), int(tb), M, N, K, a.ptr, b.ptr, o.ptr))
        return o

    def gemm_tn_colsum(self, a, b):
        """a stored [K, M], b stored [K, N]: (a^T . b, column sums of a)."""
        K, M = a.shape
        if b.shape[0] != K:
            raise FerroxHipError(1, f"Matrix multiplication shape mismatch: ({M}, {K}) @ ({b.shape[0]}, {b.shape[1]})")
        N = b.shape[1]
        o, s = self.empty((M, N), a.dtype), self.empty((M,), a.dtype)
        check(self._fn("gemm_tn_colsum", a.dtype)(self.h, M, N, K, a.ptr, b.ptr, o.ptr, s.ptr))
        return o, s

    def linear_bwd(self, dy, w, x, want_db=True, relu_below=False):
        """dy [B, out], w [out, in], x [B, in] -> (dx [B, in], dw [out, in], db [out] or None); relu_below: dx times (x > 0)."""
        Bn, O = dy.shape
        I = w.shape[1]
        dx, dw = self.empty((Bn, I), dy.dtype), self.empty((O, I), dy.dtype)
        db = self.empty((O,), dy.dtype) if want_db else None
        check(self._fn("linear_bwd", dy.dtype)(self.h, Bn, I, O, dy.ptr, w.ptr, x.ptr, dx.ptr, dw.ptr, db.ptr if want_db else None,
                                               int(relu_below)))
        return dx, dw, db

    def im2col(self, x, kernel, stride, padding):
        B, Cc, H, W = x.shape
        (kh, kw), (sh, sw), (ph, pw) = kernel, stride, padding
        oh, ow = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
        col = self.empty((Cc * kh * kw, B * oh * ow), x.dtype)
        check(self._fn("im2col", x.dtype)(self.h, x.ptr, col.ptr, B, Cc, H, W, kh, kw, sh, sw, ph, pw))
        return col

    def col2im(self, col, out_shape, kernel, stride, padding, layout):
        B, Cc, H, W = out_shape
        (kh, kw), (sh, sw), (ph, pw) = kernel, stride, padding
        o = self.empty(out_shape, col.dtype)
        check(self._fn("col2im", col.dtype)(self.h, col.ptr, o.ptr, B, Cc, H, W, kh, kw, sh, sw, ph, pw, layout))
        return o

    def conv2d_fwd(self, x, w, stride, padding, out=None):
        B, Cin, H, W = x.shape
        Cout, _, kh, kw = w.shape
        (sh, sw), (ph, pw) = stride, padding
        oh, ow = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
        y = out or self.empty((B, Cout, oh, ow), x.dtype)
        check(self._fn("conv2d_fwd", x.dtype)(self.h, x.ptr, w.ptr, y.ptr, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, None, 0))
        return y

    def conv2d_tune(self, kind, x_shape, w_shape, stride, padding, with_bias=False, act=0):
        """Times the tile shapes of the f32 3x3 forward (kind CONV_FWD) / data-gradient (CONV_DGRAD) kernel for this layer now."""
        B, Cin, H, W = x_shape
        Cout, _, kh, kw = w_shape
        (sh, sw), (ph, pw) = stride, padding
        check(lib.fx_conv2d_tune_f32(self.h, kind, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, int(with_bias), int(act)))

    def conv2d_dgrad(self, g, w, x_shape, stride, padding, mode=0, out=None):
        B, Cin, H, W = x_shape
        Cout, _, kh, kw = w.shape
        (sh, sw), (ph, pw) = stride, padding
        dx = out or self.empty(x_shape, g.dtype)
        check(self._fn("conv2d_dgrad", g.dtype)(self.h, g.ptr, w.ptr, dx.ptr, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, mode,
                                                None, 0))
        return dx

    # ---- fused sequences
    def bias_act(self, y, bias, outer, C, inner, act=0):
        """In place: y[o, c, i] += bias[c], then ReLU when act == 1."""
        check(self._fn("bias_act", y.dtype)(self.h, y.ptr, bias.ptr, outer, C, inner, act))
        return y

    @staticmethod
    def _channel_view(shape):
        """[N, C, ...] -> (outer, C, inner) of the channel axis."""
        inner = 1
        for d in shape[2:]:
            inner *= d
        return shape[0], shape[1], inner

    def batchnorm_stats(self, x, running_mean=None, running_var=None, momentum=0.1):
        """Per-channel mean and biased variance of x [N, C, ...]; updates the running arrays in place when given."""
        outer, Cc, inner = self._channel_view(x.shape)
        mean, var = self.empty((Cc,), x.dtype), self.empty((Cc,), x.dtype)
        check(self._fn("batchnorm_stats", x.dtype)(self.h, x.ptr, mean.ptr, var.ptr,
                                                   running_mean.ptr if running_mean is not None else None,
                                                   running_var.ptr if running_var is not None else None,
                                                   float(momentum), outer, Cc, inner))
        return mean, var

    def batchnorm_fwd(self, x, mean, var, gamma, beta, eps, relu=False):
        outer, Cc, inner = self._channel_view(x.shape)
        y = self.empty(x.shape, x.dtype)
        check(self._fn("batchnorm_fwd", x.dtype)(self.h, x.ptr, mean.ptr, var.ptr, gamma.ptr, beta.ptr, float(eps), y.ptr,
                                                 outer, Cc, inner, 1 if relu else 0))
        return y

    def batchnorm_bwd(self, dy, x, mean, var, gamma, eps, batch_stats=True, need_dx=True, y_act=None):
        """y_act: the output of batchnorm_fwd(relu=True); dy is then masked where it is zero."""
        outer, Cc, inner = self._channel_view(x.shape)
        dx = self.empty(x.shape, x.dtype) if need_dx else None
        dgamma, dbeta = self.empty((Cc,), x.dtype), self.empty((Cc,), x.dtype)
        check(self._fn("batchnorm_bwd", x.dtype)(self.h, dy.ptr, x.ptr, y_act.ptr if y_act is not None else None,
                                                 mean.ptr, var.ptr, gamma.ptr, float(eps),
                                                 dx.ptr if need_dx else None, dgamma.ptr, dbeta.ptr, outer, Cc, inner,
                                                 1 if batch_stats else 0))
        return dx, dgamma, dbeta

    def dropout(self, x, p, seed):
        """Returns (y, mask): mask = 1/(1-p) or 0 from splitmix64(seed + i), y = x*mask."""
        mask, y = self.empty(x.shape, x.dtype), self.empty(x.shape, x.dtype)
        check(self._fn("dropout", x.dtype)(self.h, x.ptr, mask.ptr, y.ptr, x.size, float(p), int(seed)))
        return y, mask

    def bias_grad(self, g, outer, C, inner):
        o = self.empty((C,), g.dtype)
        check(self._fn("bias_grad", g.dtype)(self.h, g.ptr, o.ptr, outer, C, inner))
        return o

    def relu_bwd_bias_grad(self, g, y, outer, C, inner):
        """(g * (y > 0), its per-channel sum) in one pass."""
        gm, db = self.empty(g.shape, g.dtype), self.empty((C,), g.dtype)
        check(self._fn("relu_bwd_bias_grad", g.dtype)(self.h, g.ptr, y.ptr, gm.ptr, db.ptr, outer, C, inner))
        return gm, db

    def softmax_ce_fwd(self, logits, targets):
        B, Cc = logits.shape
        probs, loss = self.empty((B, Cc), logits.dtype), self.empty((1,), logits.dtype)
        check(self._fn("softmax_ce_fwd", logits.dtype)(self.h, logits.ptr, targets.ptr, probs.ptr, loss.ptr, B, Cc))
        return probs, loss

    def softmax_ce_fwd_unit_grad(self, logits, targets):
        B, Cc = logits.shape
        probs, loss, d = self.empty((B, Cc), logits.dtype), self.empty((1,), logits.dtype), self.empty((B, Cc), logits.dtype)
        check(self._fn("softmax_ce_fwd_unit_grad", logits.dtype)(self.h, logits.ptr, targets.ptr, probs.ptr, loss.ptr, d.ptr, B, Cc))
        return probs, loss, d

    def softmax_ce_bwd(self, probs, targets, grad_loss):
        B, Cc = probs.shape
        d = self.empty((B, Cc), probs.dtype)
        check(self._fn("softmax_ce_bwd", probs.dtype)(self.h, probs.ptr, targets.ptr, grad_loss.ptr, d.ptr, B, Cc))
        return d

    def adam_step(self, p, g, m, v, lr, beta1, beta2, eps, wd, bc1, bc2):
        check(self._fn("adam_step", p.dtype)(self.h, p.ptr, g.ptr, m.ptr, v.ptr, p.size, lr, beta1, beta2, eps, wd, bc1, bc2))

    def adam_step_multi(self, ps, gs, ms, vs, lr, beta1, beta2, eps, wd, bc1, bc2):
        """One launch for a list of parameters (in place on ps, ms, vs)."""
        k = len(ps)
        tab = lambda arrs: (C.c_void_p * k)(*[a.ptr for a in arrs])  # noqa: E731
        ns = (C.c_int64 * k)(*[a.size for a in ps])
        dt = ps[0].dtype if k else np.float32
        check(self._fn("adam_step_multi", dt)(self.h, k, tab(ps), tab(gs), tab(ms), tab(vs), ns, float(lr), float(beta1),
                                              float(beta2), float(eps), float(wd), float(bc1), float(bc2)))

    def sgd_step_multi(self, ps, gs, lr):
        k = len(ps)
        tab = lambda arrs: (C.c_void_p * k)(*[a.ptr for a in arrs])  # noqa: E731
        ns = (C.c_int64 * k)(*[a.size for a in ps])
        dt = ps[0].dtype if k else np.float32
        check(self._fn("sgd_step_multi", dt)(self.h, k, tab(ps), tab(gs), ns, float(lr)))

    def adam_amsgrad_step(self, p, g, m, v, vmax, lr, beta1, beta2, eps, wd, bc1, bc2):
        check(self._fn("adam_amsgrad_step", p.dtype)(self.h, p.ptr, g.ptr, m.ptr, v.ptr, vmax.ptr, p.size, lr, beta1, beta2, eps,
                                                     wd, bc1, bc2))

    def sgd_momentum_step(self, p, g, buf, lr, momentum, wd, nesterov):
        check(self._fn("sgd_momentum_step", p.dtype)(self.h, p.ptr, g.ptr, buf.ptr if buf is not None else None, p.size, lr,
                                                     momentum, wd, int(nesterov)))

    def sgd_step(self, p, g, lr):
        check(self._fn("sgd_step", p.dtype)(self.h, p.ptr, g.ptr, p.size, lr))

    def conv2d_last_path(self):
        """The kernel family the last convolution call on this context ran (a fixed string per dispatch branch)."""
        return lib.fx_conv2d_last_path(self.h).decode()

    def conv2d_bwd_relu_supported(self, kind, dtype, x_shape, w_shape, stride, padding):
        B, Cin, H, W = x_shape
        Cout, _, kh, kw = w_shape
        return bool(lib.fx_conv2d_bwd_relu_supported(self.h, kind, dtype_code(dtype)[0], B, Cin, H, W, Cout, kh, kw, *stride, *padding))

    def conv2d_wgrad_relu_bias(self, x, g, act, w_shape, stride, padding):
        """(dw, db) of a conv + ReLU layer from the unmasked upstream gradient g and the layer's activation."""
        B, Cin, H, W = x.shape
        Cout, _, kh, kw = w_shape
        dw, db = self.empty(w_shape, x.dtype), self.empty((Cout,), x.dtype)
        check(self._fn("conv2d_wgrad_relu_bias", x.dtype)(self.h, x.ptr, g.ptr, act.ptr, dw.ptr, db.ptr, B, Cin, H, W, Cout, kh, kw,
                                                          *stride, *padding, None, 0))
        return dw, db

    def conv2d_dgrad_relu(self, g, act, w, x_shape, stride, padding):
        B, Cin, H, W = x_shape
        Cout, _, kh, kw = w.shape
        dx = self.empty(x_shape, g.dtype)
        check(self._fn("conv2d_dgrad_relu", g.dtype)(self.h, g.ptr, act.ptr, w.ptr, dx.ptr, B, Cin, H, W, Cout, kh, kw, *stride, *padding))
        return dx

    def conv2d_wgrad(self, x, g, w_shape, stride, padding, mode=0, out=None):
        B, Cin, H, W = x.shape
        Cout, _, kh, kw = w_shape
        (sh, sw), (ph, pw) = stride, padding
        dw = out or self.empty(w_shape, x.dtype)
        check(self._fn("conv2d_wgrad", x.dtype)(self.h, x.ptr, g.ptr, dw.ptr, B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw, mode,
                                                None, 0))
        return dw


class _RawI64:
    """int64 device buffer (argmax indices); carved from the f64 pool since both are 8-byte elements."""

    def __init__(self, ctx, n):
        self._a = ctx.empty((n,), np.float64)
        self.ptr, self.n, self.ctx = self._a.ptr, n, ctx

    def numpy(self):
        out = np.empty(self.n, dtype=np.int64)
        check(lib.fx_d2h(self.ctx.h, out.ctypes.data_as(_vp), self.ptr, out.nbytes))
        return out
