"""Pins the oracle's training step (forward, every gradient, optimizer update) against torch autograd in float64
on small versions of the MLP and CNN configs.  CPU only."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle as orc
from oracle import train as otrain


def make_problem(spec, in_shape, n_classes, seed):
    rng = np.random.default_rng(seed)
    params = []
    for tok in [t.strip() for t in spec.split(";") if t.strip()]:
        p = tok.split()
        if p[0] == "linear":
            i, o = int(p[1]), int(p[2])
            lim = np.sqrt(6.0 / i)
            params += [rng.uniform(-lim, lim, (o, i)), rng.uniform(-0.1, 0.1, (o,))]
        elif p[0] == "conv":
            ci, co, k = int(p[1]), int(p[2]), int(p[3])
            lim = np.sqrt(6.0 / (ci * k * k))
            params += [rng.uniform(-lim, lim, (co, ci, k, k)), rng.uniform(-0.1, 0.1, (co,))]
    x = rng.standard_normal(in_shape)
    labels = rng.integers(0, n_classes, in_shape[0])
    y = np.eye(n_classes)[labels]
    return params, x, y


def torch_step(spec, params, x, y):
    tp = [torch.tensor(p, dtype=torch.float64, requires_grad=True) for p in params]
    h = torch.tensor(x, dtype=torch.float64)
    pi = 0
    for tok in [t.strip() for t in spec.split(";") if t.strip()]:
        p = tok.split()
        if p[0] == "linear":
            h = F.linear(h, tp[pi], tp[pi + 1]); pi += 2
        elif p[0] == "conv":
            h = F.conv2d(h, tp[pi], tp[pi + 1], stride=int(p[4]), padding=int(p[5])); pi += 2
        elif p[0] == "relu":
            h = F.relu(h)
        else:
            h = h.flatten(1)
    s = torch.softmax(h, 1).clamp(1e-8, 1 - 1e-8)
    loss = -(torch.tensor(y) * s.log()).sum(1).mean()
    loss.backward()
    return loss.item(), [t.grad.numpy() for t in tp]


MLP = "linear 20 16; relu; linear 16 12; relu; linear 12 5"
CNN = "conv 3 4 3 1 1; relu; conv 4 6 3 2 1; relu; flatten; linear 96 5"


@pytest.mark.parametrize("spec,in_shape", [(MLP, (9, 20)), (CNN, (5, 3, 8, 8))])
def test_gradients_match_torch_float64(spec, in_shape):
    params, x, y = make_problem(spec, in_shape, 5, 0)
    model = otrain.Sequential(spec, params, np.float64, conv_mode=0)
    loss, grads = model.loss_and_grads(x, y)
    tloss, tgrads = torch_step(spec, params, x, y)
    assert abs(loss - tloss) <= 1e-12 * abs(tloss)
    for g, tg in zip(grads, tgrads):
        assert np.abs(g - tg).max() <= 1e-12 * max(1.0, np.abs(tg).max())


def test_float32_step_close_to_float64_truth():
    params, x, y = make_problem(CNN, (5, 3, 8, 8), 5, 1)
    loss, grads = otrain.Sequential(CNN, params, np.float32).loss_and_grads(x, y)
    tloss, tgrads = torch_step(CNN, params, x, y)
    assert abs(loss - tloss) <= 1e-5 * abs(tloss)
    for g, tg in zip(grads, tgrads):
        assert np.abs(g - tg).max() <= 1e-5 * max(1.0, np.abs(tg).max())


def test_sgd_and_adam_closed_forms():
    # SGD: 2.0 - 0.1 * 1.0 = 1.9 (src/nn/optim/sgd.rs:389-418)
    m = otrain.Sequential("linear 1 1", [np.array([[2.0]]), np.array([0.0])], np.float64)
    otrain.SGD(0.1).step(m, [np.array([[1.0]]), np.array([0.0])])
    assert m.params[0].item() == pytest.approx(1.9, abs=1e-15)
    # Adam, first step: delta = lr * g / (|g| + eps*sqrt(1-b2)) ~ lr * sign(g)
    m = otrain.Sequential("linear 1 1", [np.array([[2.0]]), np.array([0.5])], np.float64)
    otrain.Adam(1e-3).step(m, [np.array([[3.0]]), np.array([-0.25])])
    assert m.params[0].item() == pytest.approx(2.0 - 1e-3, abs=1e-9)
    assert m.params[1].item() == pytest.approx(0.5 + 1e-3, abs=1e-9)
    # against torch.optim.Adam over several steps
    rng = np.random.default_rng(2)
    w0 = rng.standard_normal((4, 3))
    gs = [rng.standard_normal((4, 3)) for _ in range(5)]
    m = otrain.Sequential("linear 3 4", [w0, np.zeros(4)], np.float64)
    opt = otrain.Adam(1e-3)
    tw = torch.tensor(w0, requires_grad=True)
    topt = torch.optim.Adam([tw], lr=1e-3, eps=1e-8)
    for g in gs:
        opt.step(m, [g, np.zeros(4)])
        tw.grad = torch.tensor(g)
        topt.step()
    np.testing.assert_allclose(m.params[0], tw.detach().numpy(), rtol=0, atol=1e-9)


def c1_problem(dtype, batch=32, seed=1):
    """The conv plumbing configuration: x U(-1,1) [B,1,28,28], Kaiming-normal W [8,1,3,3] (std = sqrt(2/9)), zero bias."""
    rng = np.random.default_rng(seed)
    x = rng.uniform(-1, 1, (batch, 1, 28, 28)).astype(dtype)
    w = (rng.standard_normal((8, 1, 3, 3)) * np.sqrt(2.0 / 9.0)).astype(dtype)
    return x, w, np.zeros(8, dtype)


C1 = "conv 1 8 3 1 1; relu"


@pytest.mark.parametrize("dtype,tol", [(np.float64, 1e-12), (np.float32, 1e-5)])
def test_c1_relu_sum_backward_matches_torch(dtype, tol):
    """sum(relu(conv(x) + b)).backward(): loss, input, weight and bias gradients against torch autograd (float64)."""
    x, w, b = c1_problem(dtype)
    model = otrain.Sequential(C1, [w, b], dtype, conv_mode=0)
    loss, grads, gx = model.loss_and_grads(x, None, loss_kind="sum", want_input_grad=True)
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    tw = torch.tensor(w, dtype=torch.float64, requires_grad=True)
    tb = torch.tensor(b, dtype=torch.float64, requires_grad=True)
    tl = F.relu(F.conv2d(tx, tw, tb, stride=1, padding=1)).sum()
    tl.backward()
    assert abs(loss - tl.item()) <= tol * abs(tl.item())
    for got, ref in ((gx, tx.grad), (grads[0], tw.grad), (grads[1], tb.grad)):
        ref = ref.numpy()
        assert got.shape == ref.shape
        assert np.abs(got - ref).max() <= tol * max(1.0, np.abs(ref).max())


def test_c1_literal_mode_gradients_composed():
    """The same graph with the CPU backend's literal conv gradients (batch 32): bias gradient and loss are unchanged,
    the input / weight gradients equal the flat-reinterpretation composition built from torch unfold / fold."""
    x, w, b = c1_problem(np.float64)
    model = otrain.Sequential(C1, [w, b], np.float64, conv_mode=1)
    loss, grads, gx = model.loss_and_grads(x, None, loss_kind="sum", want_input_grad=True)
    ref0 = otrain.Sequential(C1, [w, b], np.float64, conv_mode=0)
    loss0, grads0, _ = ref0.loss_and_grads(x, None, loss_kind="sum", want_input_grad=True)
    assert loss == loss0 and np.array_equal(grads[1], grads0[1])
    B, L = 32, 28 * 28
    pre = F.conv2d(torch.tensor(x), torch.tensor(w), torch.tensor(b), padding=1)
    g = (pre > 0).double().numpy()                                 # d sum(relu(pre)) / d pre
    g2d = g.reshape(8, B * L)
    col = F.unfold(torch.tensor(x), 3, padding=1).numpy().transpose(1, 0, 2).reshape(9, B * L)
    np.testing.assert_allclose(grads[0], (g2d @ col.T).reshape(w.shape), rtol=0, atol=1e-9)
    colm = (w.reshape(8, 9).T @ g2d).reshape(B, 9, L)
    np.testing.assert_allclose(gx, F.fold(torch.tensor(colm.copy()), (28, 28), 3, padding=1).numpy(), rtol=0, atol=1e-11)


@pytest.mark.parametrize("momentum,wd,nesterov", [(0.9, 0.0, False), (0.9, 5e-4, False), (0.9, 5e-4, True), (0.0, 1e-2, False)])
def test_sgd_momentum_weight_decay_nesterov_match_torch(momentum, wd, nesterov):
    """SGD::step in full (sgd.rs:116-245) against torch.optim.SGD (dampening 0: the same recurrences) over several steps."""
    rng = np.random.default_rng(3)
    w0 = rng.standard_normal((4, 3))
    gs = [rng.standard_normal((4, 3)) for _ in range(6)]
    m = otrain.Sequential("linear 3 4", [w0, np.zeros(4)], np.float64)
    opt = otrain.SGD(0.05, momentum, wd, nesterov)
    tw = torch.tensor(w0, requires_grad=True)
    topt = torch.optim.SGD([tw], lr=0.05, momentum=momentum, weight_decay=wd, nesterov=nesterov)
    for g in gs:
        opt.step(m, [g, np.zeros(4)])
        tw.grad = torch.tensor(g)
        topt.step()
        np.testing.assert_allclose(m.params[0], tw.detach().numpy(), rtol=0, atol=1e-13)


def test_adam_amsgrad_and_decoupled_weight_decay_match_torch():
    """AMSGrad (adam.rs:203-221) against torch.optim.Adam(amsgrad=True); the decoupled weight decay against AdamW.
    Gradients shrink over the steps so that the running maximum differs from the current second moment."""
    rng = np.random.default_rng(4)
    w0 = rng.standard_normal((5, 2))
    gs = [rng.standard_normal((5, 2)) * s for s in (3.0, 0.1, 0.05, 2.0, 0.01, 0.01)]
    for amsgrad, wd in ((True, 0.0), (False, 0.1), (True, 0.1)):
        m = otrain.Sequential("linear 2 5", [w0, np.zeros(5)], np.float64)
        opt = otrain.Adam(1e-2, 0.9, 0.999, 1e-8, wd, amsgrad)
        tw = torch.tensor(w0, requires_grad=True)
        topt = torch.optim.AdamW([tw], lr=1e-2, eps=1e-8, weight_decay=wd, amsgrad=amsgrad)
        for g in gs:
            opt.step(m, [g, np.zeros(5)])
            tw.grad = torch.tensor(g)
            topt.step()
            np.testing.assert_allclose(m.params[0], tw.detach().numpy(), rtol=0, atol=1e-9)
        if amsgrad:
            assert np.all(opt.vmax[0] >= opt.v[0]) and np.any(opt.vmax[0] > opt.v[0])


def test_parameter_group_overrides():
    """A group's lr / weight decay / momentum replace the optimizer's for its parameters only (mod.rs:203-258,
    sgd.rs:103-114): closed forms for one step."""
    m = otrain.Sequential("linear 1 1", [np.array([[2.0]]), np.array([1.0])], np.float64)
    otrain.SGD(0.1, groups={1: (0.5, 0.25, None)}).step(m, [np.array([[1.0]]), np.array([1.0])])
    assert m.params[0].item() == pytest.approx(2.0 - 0.1 * 1.0, abs=1e-15)
    assert m.params[1].item() == pytest.approx(1.0 - 0.5 * (1.0 + 0.25 * 1.0), abs=1e-15)
