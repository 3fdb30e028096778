"""Pins the oracle's BatchNorm / GlobalAvgPool2d / Dropout / product restatements (CPU only).
BatchNorm: torch.nn.functional.batch_norm and its autograd in float64 (an independent routine) for the forward, the
three gradients and the running mean; the biased running variance and the inference path by closed form.
Dropout: the published splitmix64 first output for seed 0, and the mask definition of nn/layers/dropout.rs:56-82."""
import numpy as np
import pytest
import torch

import oracle as orc
import oracle.train as tr


@pytest.mark.parametrize("shape", [(6, 5, 4, 3), (8, 7), (3, 2, 1, 1)])
def test_batchnorm_matches_torch_autograd_f64(shape):
    rng = np.random.default_rng(5)
    C = shape[1]
    x = rng.standard_normal(shape) * 2 + 1.5
    gamma, beta = rng.uniform(0.5, 1.5, C), rng.standard_normal(C)
    g = rng.standard_normal(shape)
    out, rec, mean, var = tr.batchnorm_forward(x, gamma, beta, 1e-3)
    dx, dg, db = tr.batchnorm_backward(g, rec)
    xt, gt, bt = (torch.tensor(a, requires_grad=True) for a in (x, gamma, beta))
    rm, rv = torch.zeros(C, dtype=torch.float64), torch.ones(C, dtype=torch.float64)
    yt = torch.nn.functional.batch_norm(xt, rm, rv, gt, bt, True, 0.1, 1e-3)
    yt.backward(torch.tensor(g))
    np.testing.assert_allclose(out, yt.detach().numpy(), rtol=0, atol=1e-13)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=0, atol=1e-13)
    np.testing.assert_allclose(dg, gt.grad.numpy(), rtol=0, atol=1e-12)
    np.testing.assert_allclose(db, bt.grad.numpy(), rtol=0, atol=1e-12)
    axes = (0, 2, 3) if len(shape) == 4 else (0,)
    np.testing.assert_allclose(mean, x.mean(axis=axes), atol=1e-14)
    np.testing.assert_allclose(var, x.var(axis=axes), atol=1e-13)                      # biased, as norm.rs:216-224
    np.testing.assert_allclose(tr.batchnorm_running_update(np.zeros(C), mean, 0.1), rm.numpy(), atol=1e-15)
    np.testing.assert_allclose(tr.batchnorm_running_update(np.ones(C), var, 0.1), 0.9 + 0.1 * x.var(axis=axes), atol=1e-14)
    # inference: running statistics, no gradient through them
    out2, rec2, _, _ = tr.batchnorm_forward(x, gamma, beta, 1e-3, False, mean, var)
    yt2 = torch.nn.functional.batch_norm(torch.tensor(x), torch.tensor(mean), torch.tensor(var), torch.tensor(gamma),
                                         torch.tensor(beta), False, 0.1, 1e-3)
    np.testing.assert_allclose(out2, yt2.numpy(), atol=1e-13)
    dx2, dg2, db2 = tr.batchnorm_backward(g, rec2)
    bshape = (1, C) + (1,) * (len(shape) - 2)
    np.testing.assert_allclose(dx2, g * (gamma / np.sqrt(var + 1e-3)).reshape(bshape), atol=1e-13)


def test_sequential_with_batchnorm_gap_dropout_matches_torch():
    """The reference's CNNClassifier block order (examples/common/models.rs:296-318) at toy size, float64."""
    rng = np.random.default_rng(6)
    B, p, seed = 6, 0.3, 42
    spec = "conv 2 4 3 1 1; bn 4 0.001 0.1; relu; gap; flatten; linear 4 5; relu; dropout 0.3 42; linear 5 3"
    params = [rng.standard_normal((4, 2, 3, 3)) * 0.4, rng.standard_normal(4) * 0.1, rng.uniform(0.5, 1.5, 4),
              rng.standard_normal(4) * 0.1, rng.standard_normal((5, 4)) * 0.5, rng.standard_normal(5) * 0.1,
              rng.standard_normal((3, 5)) * 0.5, rng.standard_normal(3) * 0.1]
    x = rng.standard_normal((B, 2, 6, 6))
    y = np.eye(3)[rng.integers(0, 3, B)]
    model = tr.Sequential(spec, params, np.float64)
    loss, grads = model.loss_and_grads(x, y)
    tp = [torch.tensor(a, requires_grad=True) for a in params]
    h = torch.nn.functional.conv2d(torch.tensor(x), tp[0], tp[1], 1, 1)
    h = torch.nn.functional.batch_norm(h, None, None, tp[2], tp[3], True, 0.1, 1e-3).relu()
    h = h.mean(dim=(2, 3))
    h = (h @ tp[4].T + tp[5]).relu()
    h = h * torch.tensor(orc.dropout_mask((B, 5), p, seed, np.float64))
    logits = h @ tp[6].T + tp[7]
    tl = -(torch.tensor(y) * torch.log_softmax(logits, 1)).sum(1).mean()
    tl.backward()
    assert abs(loss - tl.item()) < 1e-12
    for got, t in zip(grads, tp):
        np.testing.assert_allclose(got, t.grad.numpy(), atol=1e-12)
    # evaluation mode: running statistics after one step, dropout off
    model.training = False
    pred, _ = model.forward(x)
    conv = torch.nn.functional.conv2d(torch.tensor(x), tp[0], tp[1], 1, 1).detach()
    rm = 0.1 * conv.mean(dim=(0, 2, 3))
    rv = 0.9 + 0.1 * conv.var(dim=(0, 2, 3), unbiased=False)
    h = torch.nn.functional.batch_norm(conv, rm, rv, tp[2].detach(), tp[3].detach(), False, 0.1, 1e-3).relu().mean(dim=(2, 3))
    h = (h @ tp[4].detach().T + tp[5].detach()).relu()
    np.testing.assert_allclose(pred, (h @ tp[6].detach().T + tp[7].detach()).numpy(), atol=1e-12)


def test_splitmix64_known_answer_and_dropout_mask():
    # first output of splitmix64 seeded with 0 (Vigna's reference implementation): 0xE220A8397B1DCDAF
    u = orc.splitmix64_uniform(0, 3)
    assert u[0] == (0xE220A8397B1DCDAF >> 11) / 2.0 ** 53
    # counter-based: element i of seed s is element 0 of seed s + i
    assert u[2] == orc.splitmix64_uniform(2, 1)[0]
    assert np.all((u >= 0) & (u < 1))
    for dtype in (np.float32, np.float64):
        m = orc.dropout_mask((1000, 7), 0.3, 99, dtype)
        keep = orc.splitmix64_uniform(99, 7000) < 0.7
        assert m.dtype == dtype and np.array_equal(m.ravel() != 0, keep)
        assert np.array_equal(np.unique(m), np.array([0, dtype(1.0 / 0.7)], dtype))
    big = orc.dropout_mask((1 << 18,), 0.25, 1, np.float32)
    assert abs(np.count_nonzero(big) / big.size - 0.75) < 5 * np.sqrt(0.25 * 0.75 / big.size)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_reduce_prod(dtype):
    rng = np.random.default_rng(7)
    m = rng.uniform(0.9, 1.1, (4, 33, 9)).astype(dtype)
    for ax in range(3):
        np.testing.assert_allclose(orc.reduce_axis("prod", m, ax), m.astype(np.float64).prod(axis=ax),
                                   rtol=1e-5 if dtype == np.float32 else 1e-13)
    assert np.array_equal(orc.reduce_axis("prod", np.array([[2, 3, 4], [1, 0, 5]], dtype), 1), np.array([24, 0], dtype))
