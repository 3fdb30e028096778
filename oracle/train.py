"""CPU oracle for one Ferrox training step (test infrastructure only).

Restates, operator by operator and in the reference's order, what `AutoFerroxEngine` + the `nn` layers do for a
Sequential model of Linear / Conv2d / ReLU / Flatten / pooling / BatchNorm / GlobalAvgPool2d / Dropout layers with the softmax cross-entropy loss and SGD or Adam,
using the oracle's C primitives for every storage op so that each intermediate is rounded to the tensor dtype
exactly where the CPU backend rounds it.  References (Ferrox repository paths):
  layers     src/nn/layers/linear.rs:183-279, conv2d.rs:168-214, utils.rs:6-42, activation.rs:47-80, pooling.rs:100-140,
             604-623, norm.rs:127-336, dropout.rs:56-136
  loss       src/nn/losses/classification.rs:191-257
  gradients  src/ops/{basic.rs:10-215, matrix.rs:17-125, unary.rs:60-95,196-236,340-384, comparison.rs:250-297,
             reduction.rs:9-230, reshape.rs:4-115, batched.rs:41-131,154-217}
  optimizers src/nn/optim/sgd.rs:116-245, adam.rs:110-358
`conv_mode` 0 uses the mathematical conv gradients (what the GPU path computes), 1 the CPU backend's literal ones.
"""
import numpy as np

from . import binding as orc


def _bcast(b, shape):
    """Reshape [C] -> [1,C,1,1] / [1,C] and materialise to `shape` (utils.rs:6-42, BroadcastTo)."""
    if len(shape) == 4:
        return orc.materialize(b, shape, (0, 1, 0, 0))
    return orc.materialize(b, shape, (0, 1))


def softmax_ce_forward(pred, y):
    """CCELoss forward (classification.rs:191-257): returns (loss as a 0-d array, softmax probabilities)."""
    dt = pred.dtype.type
    s = orc.softmax_axis(pred, 1)
    c = orc.clamp(s, dt(1e-8), dt(1.0 - 1e-8))
    lp = orc.unary("log", c)
    tl = orc.binary("mul", y, lp)
    ce = orc.reduce("sum", tl, [1], keep_dims=True)
    neg = orc.unary("neg", ce)
    return orc.reduce("mean", neg), s


def softmax_ce_backward(s, y, g_loss):
    """Gradient of the loss w.r.t. the logits from the upstream gradient of the (scalar) loss, op by op."""
    dt = s.dtype.type
    B = s.shape[0]
    c = orc.clamp(s, dt(1e-8), dt(1.0 - 1e-8))
    g = orc.scalar("mul_scalar", np.asarray(g_loss, s.dtype).reshape(1), dt(1.0 / B)).reshape(())   # Mean::gradient scale
    g = np.full((B, 1), g.item(), s.dtype)                                            # expand_reduction(None) -> full
    g = orc.unary("neg", g)                                                           # Neg
    g = orc.materialize(g, s.shape, (1, 0))                                           # Sum(keep_dims): broadcast_to
    g = orc.binary("mul", g, y)                                                       # Mul: grad wrt log-probs
    g = orc.binary("div", g, c)                                                       # Log
    m = orc.binary("mul", orc.scalar("greater_equal_scalar", s, dt(1e-8)),
                   orc.scalar("less_equal_scalar", s, dt(1.0 - 1e-8)))
    g = orc.binary("mul", g, m)                                                       # Clamp
    prod = orc.binary("mul", g, s)                                                    # Softmax batch gradient
    sp = orc.reduce("sum", prod, [1], keep_dims=True)
    diff = orc.binary("sub", g, orc.materialize(sp, s.shape, (1, 0)))
    return orc.binary("mul", s, diff)


def bias_act(y, b, relu=False):
    """Reshape + BroadcastTo + Add (+ ReLU) of a per-channel bias on [B,C] or [B,C,H,W] (utils.rs:6-42)."""
    out = orc.binary("add", y, _bcast(b, y.shape))
    return orc.unary("relu", out) if relu else out


def bias_grad(g):
    """reduce_gradient_for_broadcasting (ops/basic.rs:10-53): axes (3,2,0) for a conv bias, (0) for a linear one."""
    return orc.reduce("sum", g, [3, 2, 0] if g.ndim == 4 else [0])


def adam_update(w, g, m, v, lr, b1, b2, eps, wd, bc1, bc2, vmax=None):
    """One Adam::step for one parameter (adam.rs:288-358); every scalar already in the tensor dtype.  vmax: the AMSGrad
    running maximum of the second moment (adam.rs:203-221) or None.  Returns (w, m, v, vmax)."""
    dt = w.dtype.type
    m = orc.binary("add", orc.scalar("mul_scalar", m, b1), orc.scalar("mul_scalar", g, dt(1) - b1))
    v = orc.binary("add", orc.scalar("mul_scalar", v, b2), orc.scalar("mul_scalar", orc.binary("mul", g, g), dt(1) - b2))
    second = v
    if vmax is not None:
        vmax = orc.binary("max", vmax, v)
        second = vmax
    denom = orc.scalar("add_scalar", orc.unary("sqrt", orc.scalar("div_scalar", second, bc2)), eps)
    upd = orc.scalar("mul_scalar", orc.binary("div", orc.scalar("div_scalar", m, bc1), denom), lr)
    if wd != 0:
        wdt = orc.scalar("mul_scalar", w, wd * lr)
        w = orc.binary("sub", orc.binary("sub", w, upd), wdt)
    else:
        w = orc.binary("sub", w, upd)
    return w, m, v, vmax


def batchnorm_forward(x, gamma, beta, eps, training=True, running_mean=None, running_var=None):
    """BatchNorm::forward (nn/layers/norm.rs:167-336), operator by operator.  Training: statistics of the batch over
    axes (0,2,3) / (0); AddScalar and Sqrt run on the full-size broadcast variance (norm.rs:228-236, 298-311).
    Inference: the running statistics, Sqrt on [C] then broadcast (norm.rs:261-290).  Returns (out, tape record,
    batch mean or None, batch variance or None)."""
    dt = x.dtype.type
    axes = [0, 2, 3] if x.ndim == 4 else [0]
    if training:
        mean = orc.reduce("mean", x, axes)
        cen = orc.binary("sub", x, _bcast(mean, x.shape))
        var = orc.reduce("mean", orc.binary("mul", cen, cen), axes)
        std = orc.unary("sqrt", orc.scalar("add_scalar", _bcast(var, x.shape), dt(eps)))
    else:
        mean = var = None
        cen = orc.binary("sub", x, _bcast(running_mean, x.shape))
        std = _bcast(orc.unary("sqrt", orc.scalar("add_scalar", running_var, dt(eps))), x.shape)
    normalized = orc.binary("div", cen, std)
    wb = _bcast(gamma, x.shape)
    out = orc.binary("add", orc.binary("mul", normalized, wb), _bcast(beta, x.shape))
    return out, (cen, std, normalized, wb, training), mean, var


def batchnorm_running_update(running, batch, momentum):
    """update_running_stats (norm.rs:127-164): running*(1-momentum) + batch*momentum, the biased batch variance."""
    dt = running.dtype.type
    return orc.binary("add", orc.scalar("mul_scalar", running, dt(1.0 - momentum)), orc.scalar("mul_scalar", batch, dt(momentum)))


def batchnorm_backward(g, rec):
    """Gradients (dx, dgamma, dbeta) in the order AutoFerroxEngine::backward visits the nodes (graph/mod.rs:700-783:
    reverse of the depth-first post-order): Add, Mul, Div, Sqrt, AddScalar, BroadcastTo, Mean, Mul(centered, centered)
    twice into `centered`, Sub, BroadcastTo, Mean into x."""
    cen, std, normalized, wb, training = rec
    dt = g.dtype.type
    red = (lambda t: orc.reduce("sum", t, [3, 2, 0])) if g.ndim == 4 else (lambda t: orc.reduce("sum", t, [0]))
    dbeta = red(g)                                                         # Add -> BroadcastTo -> Reshape
    g_norm = orc.binary("mul", g, wb)                                      # Mul::gradient, input 0
    dgamma = red(orc.binary("mul", g, normalized))                         # input 1 -> BroadcastTo -> Reshape
    d_cen = orc.binary("div", g_norm, std)                                 # Div::gradient, input 0 (ops/basic.rs:253)
    if not training:
        return d_cen, dgamma, dbeta
    n = float(cen.size // dbeta.size)
    g_std = orc.binary("mul", g_norm, orc.unary("neg", orc.binary("div", normalized, std)))      # basic.rs:256-257
    g_vpe = orc.binary("div", g_std, orc.scalar("mul_scalar", std, dt(2.0)))                      # Sqrt, unary.rs:138-140
    g_var = red(g_vpe)                                                     # AddScalar passes; BroadcastTo sums; Reshape
    g_sq = _bcast(orc.scalar("mul_scalar", g_var, dt(1.0 / n)), cen.shape)  # Mean::gradient, reduction.rs:178-194
    a = orc.binary("mul", g_sq, cen)                                       # Mul(centered, centered): both inputs
    d_cen = orc.binary("add", orc.binary("add", d_cen, a), a)              # accumulate_gradient, graph/mod.rs:681-690
    g_mean = red(orc.unary("neg", d_cen))                                  # Sub input 1 -> BroadcastTo -> Reshape
    dx = orc.binary("add", d_cen, _bcast(orc.scalar("mul_scalar", g_mean, dt(1.0 / n)), cen.shape))
    return dx, dgamma, dbeta


class Sequential:
    def __init__(self, spec, params, dtype, conv_mode=0):
        self.dtype = np.dtype(dtype)
        self.conv_mode = conv_mode
        self.layers = []
        self.params = [np.ascontiguousarray(p, dtype=self.dtype).copy() for p in params]
        self.training = True
        self.running = {}     # layer index -> [running_mean, running_var]  (zeros / ones, norm.rs:75-84)
        self.dropout_calls = 0
        pi = 0
        for tok in [t.strip() for t in spec.split(";") if t.strip()]:
            parts = tok.split()
            kind = parts[0]
            if kind == "linear":
                self.layers.append(("linear", pi, pi + 1))
                pi += 2
            elif kind == "conv":
                _, cin, cout, k, s, p = parts
                self.layers.append(("conv", pi, pi + 1, (int(s), int(s)), (int(p), int(p))))
                pi += 2
            elif kind in ("maxpool", "avgpool"):
                _, k, st, p = parts
                self.layers.append((kind, (int(k), int(k)), (int(st), int(st)), (int(p), int(p))))
            elif kind == "bn":              # bn C eps momentum
                cfeat = int(parts[1])
                eps = float(parts[2]) if len(parts) > 2 else 1e-5
                mom = float(parts[3]) if len(parts) > 3 else 0.1
                self.running[len(self.layers)] = [np.zeros(cfeat, self.dtype), np.ones(cfeat, self.dtype)]
                self.layers.append(("bn", pi, pi + 1, eps, mom))
                pi += 2
            elif kind == "dropout":         # dropout p seed
                self.layers.append(("dropout", float(parts[1]), int(parts[2])))
            elif kind in ("relu", "flatten", "gap"):
                self.layers.append((kind,))
            else:
                raise ValueError(kind)
        assert pi == len(self.params)

    # ---- forward, recording what backward needs ----
    def forward(self, x):
        tape = []
        h = np.ascontiguousarray(x, dtype=self.dtype)
        for layer in self.layers:
            kind = layer[0]
            if kind == "linear":
                w, b = self.params[layer[1]], self.params[layer[2]]
                wt = np.ascontiguousarray(w.T)                      # Transpose op (owned copy)
                lin = orc.gemm(h, wt)                               # MatMul
                out = orc.binary("add", lin, _bcast(b, lin.shape))  # BroadcastTo + Add
                tape.append(("linear", layer, h, wt))
                h = out
            elif kind == "conv":
                w, b = self.params[layer[1]], self.params[layer[2]]
                y = orc.conv2d_fwd(h, w, layer[3], layer[4])
                out = orc.binary("add", y, _bcast(b, y.shape))
                tape.append(("conv", layer, h))
                h = out
            elif kind in ("maxpool", "avgpool"):
                out = orc.pool2d(h, layer[1], layer[2], layer[3], kind == "maxpool")      # ops/pooling.rs:38-48, 150-162
                tape.append((kind, layer, h, out))
                h = out
            elif kind == "relu":
                tape.append(("relu", h))
                h = orc.unary("relu", h)
            elif kind == "bn":
                li = self.layers.index(layer)
                rm, rv = self.running[li]
                out, rec, mean, var = batchnorm_forward(h, self.params[layer[1]], self.params[layer[2]], layer[3],
                                                        self.training, rm, rv)
                if self.training:
                    self.running[li] = [batchnorm_running_update(rm, mean, layer[4]),
                                        batchnorm_running_update(rv, var, layer[4])]
                tape.append(("bn", layer, rec))
                h = out
            elif kind == "gap":             # GlobalAvgPool2d(flatten = false): Mean over axes (2,3), keep_dims (pooling.rs:604-623)
                tape.append(("gap", h.shape))
                h = orc.reduce("mean", h, [2, 3], keep_dims=True)
            elif kind == "dropout":         # dropout.rs:100-136; call k of a run uses seed + k * 2^32
                if self.training and layer[1] != 0.0:
                    mask = orc.dropout_mask(h.shape, layer[1], layer[2] + (self.dropout_calls << 32), self.dtype)
                    self.dropout_calls += 1
                    tape.append(("dropout", mask))
                    h = orc.binary("mul", h, mask)
                else:
                    tape.append(("dropout", None))
            else:
                tape.append(("flatten", h.shape))
                h = h.reshape(h.shape[0], -1)
        return h, tape

    def loss_and_grads(self, x, y, loss_kind="cce", want_input_grad=False):
        """loss_kind 'cce': CCELoss against y.  'sum': Sum::new() over every element of the prediction
        (ops/reduction.rs:52-140: every axis from last to first, cpu.rs:1183-1211; its gradient is
        expand_reduction(None) = full(input_shape, grad.first()), reduction.rs:9-50).
        want_input_grad: also return the gradient that reaches the batch (a leaf created with requires_grad)."""
        dt = self.dtype.type
        pred, tape = self.forward(x)
        if loss_kind == "sum":
            loss = orc.reduce("sum", pred)
            g = np.full(pred.shape, dt(1), self.dtype)
        else:
            y = np.ascontiguousarray(y, dtype=self.dtype)
            loss, s = softmax_ce_forward(pred, y)
            g = softmax_ce_backward(s, y, np.ones((), self.dtype))
        grads = [None] * len(self.params)
        for rec in reversed(tape):
            kind = rec[0]
            if kind == "linear":
                _, layer, h, wt = rec
                grads[layer[2]] = orc.reduce("sum", g, [0])                               # bias: sum over batch axis
                ga = orc.gemm(g, np.ascontiguousarray(wt.T))                              # grad . B^T (materialised)
                gb = orc.gemm(np.ascontiguousarray(h.T), g)                               # A^T . grad
                grads[layer[1]] = np.ascontiguousarray(gb.T)                              # Transpose::gradient
                g = ga
            elif kind == "conv":
                _, layer, h = rec
                w = self.params[layer[1]]
                grads[layer[2]] = orc.reduce("sum", g, [3, 2, 0])                         # bias: axes (3,2,0)
                gi = orc.conv2d_dgrad(g, w, h.shape, layer[3], layer[4], self.conv_mode)
                grads[layer[1]] = orc.conv2d_wgrad(h, g, w.shape, layer[3], layer[4], self.conv_mode)
                g = gi
            elif kind in ("maxpool", "avgpool"):
                _, layer, h, out = rec
                g = orc.unpool2d(g, h, out, layer[1], layer[2], layer[3], kind == "maxpool")
            elif kind == "relu":
                g = orc.binary("mul", g, orc.scalar("greater_scalar", rec[1], dt(0)))
            elif kind == "bn":
                _, layer, brec = rec
                g, grads[layer[1]], grads[layer[2]] = batchnorm_backward(g, brec)
            elif kind == "gap":
                shape = rec[1]
                g = orc.scalar("mul_scalar", g, dt(1.0 / float(shape[2] * shape[3])))     # Mean::gradient, keep_dims
                g = orc.materialize(g, shape, (shape[1], 1, 0, 0))
            elif kind == "dropout":
                if rec[1] is not None:
                    g = orc.binary("mul", g, rec[1])                                      # Mul::gradient wrt the input
            else:
                g = g.reshape(rec[1])
        if want_input_grad:
            return loss.item(), grads, g
        return loss.item(), grads


class SGD:
    """SGD::step (sgd.rs:116-245): L2 weight decay folded into the gradient, momentum buffer buf = buf*mu + e, Nesterov
    update buf*mu + e, p = p - update*lr.  `groups` maps a parameter index to (lr, weight_decay, momentum) overrides
    (None = the optimizer's value), the ParameterGroup options of optim/mod.rs:203-258."""

    def __init__(self, lr, momentum=0.0, weight_decay=0.0, nesterov=False, groups=None):
        self.lr, self.momentum, self.wd, self.nesterov = lr, momentum, weight_decay, bool(nesterov)
        self.groups = groups or {}
        self.buf = {}

    def step(self, model, grads):
        dt = model.dtype.type
        for i, g in enumerate(grads):
            glr, gwd, gmom = self.groups.get(i, (None, None, None))
            lr = dt(self.lr if glr is None else glr)
            wd = dt(self.wd if gwd is None else gwd)
            mom = dt(self.momentum if gmom is None else gmom)
            w = model.params[i]
            e = g if wd == 0 else orc.binary("add", g, orc.scalar("mul_scalar", w, wd))
            if mom != 0:
                b = self.buf.get(i, np.zeros_like(w))
                b = orc.binary("add", orc.scalar("mul_scalar", b, mom), e)
                self.buf[i] = b
                upd = orc.binary("add", orc.scalar("mul_scalar", b, mom), e) if self.nesterov else b
            else:
                upd = e
            model.params[i] = orc.binary("sub", w, orc.scalar("mul_scalar", upd, lr))


class Adam:
    """Adam::step (adam.rs:110-358); amsgrad keeps vmax = max(vmax, v) (a >= b ? a : b) and divides by it."""

    def __init__(self, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0, amsgrad=False, groups=None):
        self.lr, self.b1, self.b2, self.eps, self.wd = lr, beta1, beta2, eps, weight_decay
        self.amsgrad = bool(amsgrad)
        self.groups = groups or {}
        self.t = 0
        self.m, self.v, self.vmax = {}, {}, {}

    def step(self, model, grads):
        dt = model.dtype.type
        self.t += 1
        b1, b2 = dt(self.b1), dt(self.b2)
        bc1 = dt(1) - max(dt(np.power(b1, dt(self.t))), dt(1e-8))      # adam.rs:110-126
        bc2 = dt(1) - max(dt(np.power(b2, dt(self.t))), dt(1e-8))
        for i, g in enumerate(grads):
            glr, gwd, _ = self.groups.get(i, (None, None, None))
            lr = dt(self.lr if glr is None else glr)
            wd = dt(self.wd if gwd is None else gwd)
            w = model.params[i]
            m = self.m.get(i, np.zeros_like(w))
            v = self.v.get(i, np.zeros_like(w))
            vmax = self.vmax.get(i, np.zeros_like(w)) if self.amsgrad else None
            w, m, v, vmax = adam_update(w, g, m, v, lr, b1, b2, dt(self.eps), wd, bc1, bc2, vmax)
            self.m[i], self.v[i] = m, v
            if self.amsgrad:
                self.vmax[i] = vmax
            model.params[i] = w
