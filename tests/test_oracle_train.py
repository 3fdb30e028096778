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
