"""ctypes binding of libferrox_host.so: the C++ mirror of Ferrox's host stack (HipStorage, autograd tape, layers,
loss, optimizers) with a small C harness to run whole training steps through the C ABI of libferrox_hip.so."""
import ctypes as C
import os
import subprocess

import numpy as np

from . import capi

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libferrox_host.so")


def _load():
    if not os.path.exists(LIB_PATH):
        subprocess.check_call(["make", "-C", os.path.join(_HERE, "host"), "-s"])
    return C.CDLL(LIB_PATH)


lib = _load()
lib.fxh_last_error.restype = C.c_char_p
lib.fxh_init.argtypes = [C.c_int, C.c_int, C.POINTER(capi.PoolConfig)]
lib.fxh_model_create.restype = C.c_void_p
lib.fxh_model_create.argtypes = [C.c_int, C.c_char_p, C.c_char_p, C.c_int, C.POINTER(C.c_void_p), C.c_int]
lib.fxh_model_destroy.argtypes = [C.c_void_p]
lib.fxh_model_num_params.argtypes = [C.c_void_p]
lib.fxh_model_param_numel.argtypes = [C.c_void_p, C.c_int]
lib.fxh_model_param_numel.restype = C.c_int64
lib.fxh_model_set_batch.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(C.c_int64), C.c_int, C.c_void_p, C.POINTER(C.c_int64), C.c_int]
lib.fxh_model_train_step.argtypes = [C.c_void_p, C.POINTER(C.c_double)]
lib.fxh_model_train_steps.argtypes = [C.c_void_p, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double)]
lib.fxh_model_get_param.argtypes = [C.c_void_p, C.c_int, C.c_void_p]
lib.fxh_model_get_grad.argtypes = [C.c_void_p, C.c_int, C.c_void_p]
lib.fxh_model_output_numel.argtypes = [C.c_void_p]
lib.fxh_model_output_numel.restype = C.c_int64
lib.fxh_model_forward.argtypes = [C.c_void_p, C.c_void_p]
lib.fxh_model_set_training.argtypes = [C.c_void_p, C.c_int]
lib.fxh_model_num_state.argtypes = [C.c_void_p]
lib.fxh_model_state_numel.argtypes = [C.c_void_p, C.c_int]
lib.fxh_model_state_numel.restype = C.c_int64
lib.fxh_model_get_state.argtypes = [C.c_void_p, C.c_int, C.c_void_p]
lib.fxh_model_optimizer_state.argtypes = [C.c_void_p, C.POINTER(C.c_void_p), C.POINTER(C.c_int64)]
lib.fxh_free.argtypes = [C.c_void_p]
lib.fxh_free.restype = None
lib.fxh_model_load_optimizer_state.argtypes = [C.c_void_p, C.c_char_p, C.c_int64]
lib.fxh_set_conv_grad_mode.argtypes = [C.c_int]
lib.fxh_set_share_clones.argtypes = [C.c_int]
lib.fxh_set_share_clones.restype = None
lib.fxh_model_configure.argtypes = [C.c_void_p, C.c_int, C.c_int]
lib.fxh_model_enable_graph.argtypes = [C.c_void_p, C.c_int]
lib.fxh_model_graph_info.argtypes = [C.c_void_p, C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.POINTER(C.c_int64)]
lib.fxh_model_backward.argtypes = [C.c_void_p, C.POINTER(C.c_double)]
lib.fxh_model_add_param_group.argtypes = [C.c_void_p, C.POINTER(C.c_int), C.c_int, C.c_double, C.c_double, C.c_double]
lib.fxh_model_input_numel.argtypes = [C.c_void_p]
lib.fxh_model_input_numel.restype = C.c_int64
lib.fxh_model_get_input_grad.argtypes = [C.c_void_p, C.c_void_p]
lib.fxh_pool_stats.argtypes = [C.c_int, C.POINTER(capi.PoolStats)]


class HostError(RuntimeError):
    pass


def _check(rc):
    if rc != 0:
        raise HostError(lib.fxh_last_error().decode("utf-8", "replace"))


def init(device=0, conv_grad_mode=0, pool_config=None):
    _check(lib.fxh_init(device, conv_grad_mode, C.byref(pool_config) if pool_config is not None else None))


def set_share_clones(on):
    """True (default): clone_storage() in the op-by-op engines is a second owner of the same device block (nothing reachable
    through the storage trait writes device memory in place, so it cannot be told from a copy); False: a device-to-device copy
    per clone, as the reference's CUDA backend makes (cuda/context.rs:744-763)."""
    lib.fxh_set_share_clones(1 if on else 0)


def set_conv_grad_mode(mode):
    """0 = mathematical conv gradients (default), 1 = the CPU backend's literal arithmetic."""
    _check(lib.fxh_set_conv_grad_mode(int(mode)))


def shutdown():
    lib.fxh_shutdown()


def pool_stats(dtype=np.float32):
    st = capi.PoolStats()
    _check(lib.fxh_pool_stats(capi.dtype_code(dtype)[0], C.byref(st)))
    return st.as_dict()


class Model:
    """spec: 'conv CIN COUT K S P; bn C EPS MOMENTUM; relu; maxpool K S P; gap; flatten; linear IN OUT; dropout P SEED; ...'
    optimizer: 'sgd LR [MOMENTUM [WEIGHT_DECAY [NESTEROV]]]' | 'adam LR B1 B2 EPS WD [AMSGRAD]'."""

    def __init__(self, spec, params, optimizer, dtype=np.float32, literal_engine=True, fused=False):
        """literal_engine: keep the reference engine's per-node deep clones; fused: fused layers, loss and optimizer."""
        self.dtype = np.dtype(dtype)
        self._params = [np.ascontiguousarray(p, dtype=self.dtype) for p in params]
        self.shapes = [p.shape for p in self._params]
        arr = (C.c_void_p * len(params))(*[p.ctypes.data for p in self._params])
        self.h = lib.fxh_model_create(capi.dtype_code(dtype)[0], spec.encode(), optimizer.encode(), 2 if fused else int(literal_engine), arr,
                                      len(params))
        if not self.h:
            raise HostError(lib.fxh_last_error().decode("utf-8", "replace"))

    def close(self):
        if self.h:
            lib.fxh_model_destroy(self.h)
            self.h = None

    def set_batch(self, x, y):
        x = np.ascontiguousarray(x, dtype=self.dtype)
        y = np.ascontiguousarray(y, dtype=self.dtype)
        xs = (C.c_int64 * x.ndim)(*x.shape)
        ys = (C.c_int64 * y.ndim)(*y.shape)
        _check(lib.fxh_model_set_batch(self.h, x.ctypes.data, xs, x.ndim, y.ctypes.data, ys, y.ndim))

    def train_step(self):
        loss = C.c_double(0)
        _check(lib.fxh_model_train_step(self.h, C.byref(loss)))
        return loss.value

    def configure(self, loss="cce", input_requires_grad=False):
        """loss: 'cce' (softmax cross-entropy against the targets) or 'sum' (sum of every element of the prediction)."""
        _check(lib.fxh_model_configure(self.h, {"cce": 0, "sum": 1}[loss], int(input_requires_grad)))

    def add_param_group(self, indices, lr=None, weight_decay=None, momentum=None):
        """Moves the parameters `indices` into a new optimizer group with its own lr / weight decay / momentum
        (None = the optimizer's value)."""
        nan = float("nan")
        arr = (C.c_int * len(indices))(*indices)
        _check(lib.fxh_model_add_param_group(self.h, arr, len(indices), nan if lr is None else lr,
                                             nan if weight_decay is None else weight_decay, nan if momentum is None else momentum))

    def backward(self):
        """zero_gradients, forward, loss, backward -- no optimizer step.  Returns the loss."""
        loss = C.c_double(0)
        _check(lib.fxh_model_backward(self.h, C.byref(loss)))
        return loss.value

    def input_grad(self, shape):
        out = np.empty(shape, self.dtype)
        assert out.size == lib.fxh_model_input_numel(self.h)
        _check(lib.fxh_model_get_input_grad(self.h, out.ctypes.data))
        return out

    def enable_graph(self, on=True):
        """Later train steps are recorded once (after two eager ones) and replayed as one graph launch where the model
        allows it: fused engine, no Dropout layer, no gradient for the batch.  Same results, bit for bit."""
        _check(lib.fxh_model_enable_graph(self.h, int(on)))

    def graph_info(self):
        n, k, h = C.c_int64(0), C.c_int64(0), C.c_int64(0)
        _check(lib.fxh_model_graph_info(self.h, C.byref(n), C.byref(k), C.byref(h)))
        return {"nodes": n.value, "kernel_nodes": k.value, "held_blocks": h.value}

    def train_steps(self, n):
        loss, ms = C.c_double(0), C.c_double(0)
        _check(lib.fxh_model_train_steps(self.h, n, C.byref(loss), C.byref(ms)))
        return loss.value, ms.value

    def param(self, i):
        out = np.empty(self.shapes[i], self.dtype)
        _check(lib.fxh_model_get_param(self.h, i, out.ctypes.data))
        return out

    def grad(self, i):
        out = np.empty(self.shapes[i], self.dtype)
        _check(lib.fxh_model_get_grad(self.h, i, out.ctypes.data))
        return out

    def set_training(self, training):
        """Module::set_training on every layer (BatchNorm statistics, Dropout)."""
        _check(lib.fxh_model_set_training(self.h, 1 if training else 0))

    def state(self):
        """Persistent non-parameter tensors in layer order (BatchNorm: running mean, running variance)."""
        out = []
        for i in range(lib.fxh_model_num_state(self.h)):
            a = np.empty(lib.fxh_model_state_numel(self.h, i), self.dtype)
            _check(lib.fxh_model_get_state(self.h, i, a.ctypes.data))
            out.append(a)
        return out

    def optimizer_state(self):
        """The optimizer's state dictionary as bytes in the reference's file format (moments copied from the device)."""
        p, n = C.c_void_p(), C.c_int64(0)
        _check(lib.fxh_model_optimizer_state(self.h, C.byref(p), C.byref(n)))
        try:
            return C.string_at(p, n.value)
        finally:
            lib.fxh_free(p)

    def load_optimizer_state(self, data):
        _check(lib.fxh_model_load_optimizer_state(self.h, data, len(data)))

    def forward(self):
        n = lib.fxh_model_output_numel(self.h)
        if n < 0:
            raise HostError(lib.fxh_last_error().decode("utf-8", "replace"))
        out = np.empty(n, self.dtype)
        _check(lib.fxh_model_forward(self.h, out.ctypes.data))
        return out
