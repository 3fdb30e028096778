"""Pins the CPU oracle's GEMM, reductions, activations, softmax and activation gradients against the vectors the
reference's own tests hold (tests/golden/reference_vectors.json), numpy/libm closed forms and finite differences."""
import numpy as np
import pytest

import oracle as orc


def test_reference_vectors(golden):
    a, b, c = (np.array(v, np.float32).reshape(2, 2) for v in golden["matmul"]["arrays"])
    assert np.array_equal(orc.gemm(a, b), c) and np.array_equal(orc.gemm(a, b, naive=True), c)
    m = lambda k: np.array(golden[k]["arrays"][0], np.float32).reshape(2, 2)  # noqa: E731
    e = lambda k: golden[k]["arrays"][1]  # noqa: E731
    assert orc.reduce("sum", m("sum_all")).item() == e("sum_all")[0]
    assert orc.reduce("sum", m("sum_axis0"), [0]).tolist() == e("sum_axis0")
    assert orc.reduce("mean", m("mean_all")).item() == e("mean_all")[0]
    assert orc.reduce("mean", m("mean_axis1"), [1]).tolist() == e("mean_axis1")
    assert orc.reduce("max", m("max_all")).item() == e("max_all")[0]
    assert orc.reduce("max", m("max_axis0"), [0]).tolist() == e("max_axis0")
    for key, op, tol in (("relu", "relu", 1e-6), ("sigmoid", "sigmoid", 1e-4), ("tanh", "tanh", 1e-4), ("neg", "neg", 1e-6)):
        x, y = (np.array(v, np.float32) for v in golden[key]["arrays"])
        np.testing.assert_allclose(orc.unary(op, x), y, atol=tol, rtol=0)
    for key, shape, axis in (("softmax_axis1", (2, 3), 1), ("softmax_axis0", (2, 2), 0)):
        x, y = (np.array(v, np.float32) for v in golden[key]["arrays"])
        np.testing.assert_allclose(orc.softmax_axis(x.reshape(shape), axis).ravel(), y, atol=1e-3, rtol=0)


@pytest.mark.parametrize("dtype,tol", [(np.float32, 1e-5), (np.float64, 1e-12)])
def test_gemm_vs_float64_all_transposes(dtype, tol):
    rng = np.random.default_rng(0)
    for (M, N, K) in ((1, 1, 1), (5, 7, 3), (64, 33, 129), (130, 257, 75), (256, 10, 1000)):
        a = rng.standard_normal((M, K)).astype(dtype)
        b = rng.standard_normal((K, N)).astype(dtype)
        truth = a.astype(np.float64) @ b.astype(np.float64)
        scale = (np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64)).max()
        for ta in (False, True):
            for tb in (False, True):
                for naive in (False, True):
                    got = orc.gemm(a.T.copy() if ta else a, b.T.copy() if tb else b, ta, tb, naive=naive)
                    assert np.abs(got - truth).max() <= tol * scale, (M, N, K, ta, tb, naive)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_reductions_vs_numpy(dtype):
    rng = np.random.default_rng(1)
    tol = 1e-5 if dtype == np.float32 else 1e-12
    for shape in ((2, 2), (7, 13), (3, 5, 7), (4, 3, 6, 5), (1, 1000)):
        x = rng.standard_normal(shape).astype(dtype)
        for axis in range(len(shape)):
            truth = x.astype(np.float64).sum(axis=axis)
            bound = tol * np.abs(x).astype(np.float64).sum(axis=axis).max()
            assert np.abs(orc.reduce_axis("sum", x, axis) - truth).max() <= bound
            assert np.abs(orc.reduce_axis("mean", x, axis) - truth / shape[axis]).max() <= bound
            v, i = orc.reduce_axis("max", x, axis, want_idx=True)
            assert np.array_equal(v, x.max(axis=axis)) and np.array_equal(i, np.argmax(x, axis=axis))
        # multi-axis in the reference's order (descending axes, then keep_dims reshape): bias-gradient pattern (3,2,0)
        if len(shape) == 4:
            got = orc.reduce("sum", x, [0, 2, 3], keep_dims=True)
            assert got.shape == (1, shape[1], 1, 1)
            np.testing.assert_allclose(got.ravel(), x.astype(np.float64).sum(axis=(0, 2, 3)), rtol=tol * 50)
        assert abs(orc.reduce("mean", x).item() - x.astype(np.float64).mean()) <= tol * np.abs(x).mean() * 10 + 1e-30


def test_max_semantics_strict_greater_from_lowest_finite():
    lowest = np.finfo(np.float32).min
    x = np.array([[-np.inf, -np.inf], [np.nan, 3.0], [2.0, 2.0], [lowest, -np.inf]], np.float32)
    v, i = orc.reduce_axis("max", x, 1, want_idx=True)
    assert v[0] == lowest and i[0] == 0          # nothing exceeds the start value (cpu.rs:1231-1234)
    assert v[1] == 3.0 and i[1] == 1             # NaN never selected
    assert i[2] == 0                             # first occurrence on ties
    assert v[3] == lowest and i[3] == 0


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_activations_closed_forms(dtype):
    x = np.linspace(-30, 30, 2001).astype(dtype)
    x64 = x.astype(np.float64)
    tol = 2e-6 if dtype == np.float32 else 1e-14
    np.testing.assert_allclose(orc.unary("sigmoid", x), 1 / (1 + np.exp(-x64)), rtol=tol, atol=tol)
    np.testing.assert_allclose(orc.unary("tanh", x), np.tanh(x64), rtol=0, atol=4 * np.finfo(dtype).eps)
    assert np.all(orc.unary("tanh", x)[x > 20] == 1) and np.all(orc.unary("tanh", x)[x < -20] == -1)
    assert np.array_equal(orc.unary("relu", x), np.maximum(x, 0))
    np.testing.assert_allclose(orc.unary("exp", x), np.exp(x64), rtol=2e-7 if dtype == np.float32 else 1e-15)
    big = np.array([1000.0, -1000.0], dtype)
    assert orc.unary("sigmoid", big).tolist() == [1.0, 0.0] and orc.unary("tanh", big).tolist() == [1.0, -1.0]


def test_activation_gradients_finite_differences_and_literal_sign():
    x = np.linspace(-3, 3, 61)
    g = np.cos(x)
    h = 1e-6
    s, t = orc.unary("sigmoid", x), orc.unary("tanh", x)
    num_s = (orc.unary("sigmoid", x + h) - orc.unary("sigmoid", x - h)) / (2 * h)
    num_t = (orc.unary("tanh", x + h) - orc.unary("tanh", x - h)) / (2 * h)
    np.testing.assert_allclose(orc.sigmoid_bwd(g, s, 0), g * num_s, atol=1e-9)
    np.testing.assert_allclose(orc.sigmoid_bwd(g, s, 1), -g * num_s, atol=1e-9)  # the reference's s*(s-1): sign flipped
    np.testing.assert_allclose(orc.tanh_bwd(g, t), g * num_t, atol=1e-9)
    xr = np.array([-1.0, 0.0, -0.0, 2.0])
    assert orc.relu_bwd(np.ones(4), xr).tolist() == [0.0, 0.0, 0.0, 1.0]  # strict x > 0 (cpu.rs:876-885)


def test_softmax_rows_sum_to_one_and_shift_invariance():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((6, 10)) * 5
    s = orc.softmax_axis(x, 1)
    np.testing.assert_allclose(s.sum(axis=1), 1, atol=1e-14)
    np.testing.assert_allclose(orc.softmax_axis(x + 100.0, 1), s, atol=1e-13)
    np.testing.assert_allclose(orc.softmax_axis(x.T.copy(), 0), s.T, atol=1e-15)


def test_materialize_and_clamp_and_scalar():
    rng = np.random.default_rng(3)
    b = rng.standard_normal(5).astype(np.float32)
    assert np.array_equal(orc.materialize(b, (2, 5, 3), (0, 1, 0)), np.broadcast_to(b.reshape(1, 5, 1), (2, 5, 3)))
    m = rng.standard_normal((4, 6)).astype(np.float32)
    assert np.array_equal(orc.materialize(m, (6, 4), (1, 6)), m.T)
    x = np.array([-1.0, 0.0, 0.5, 1.0, 2.0], np.float32)
    assert orc.clamp(x, 1e-8, 1 - 1e-8).tolist() == [np.float32(1e-8), np.float32(1e-8), 0.5, 1.0, 1.0]  # f32: 1-1e-8 == 1
    assert orc.scalar("greater_equal_scalar", x, 0.5).tolist() == [0, 0, 1, 1, 1]
    assert orc.binary("equal", x, x[::-1].copy()).tolist() == [0, 0, 1, 0, 0]


# ---- oracle functions added for the rest of the storage trait: pinned by the reference's vectors, numpy and torch ----
def test_min_minmax_elementwise_reciprocal_reference_vectors(golden):
    import oracle as orc
    a = np.array(golden["min_all"]["arrays"][0], np.float32).reshape(2, 2)
    assert orc.reduce("min", a).item() == golden["min_all"]["arrays"][1][0]
    assert orc.reduce("min", a, [1]).tolist() == golden["min_axis1"]["arrays"][1]
    for key, op in (("max_elementwise", "max"), ("min_elementwise", "min")):
        x, y, want = (np.array(v, np.float32) for v in golden[key]["arrays"])
        assert np.array_equal(orc.binary(op, x, y), want)
    x, want = (np.array(v, np.float32) for v in golden["reciprocal"]["arrays"])
    assert np.array_equal(orc.unary("reciprocal", x), want)


def test_pooling_reference_vectors(golden):
    import oracle as orc
    for key, is_max in (("maxpool1d", True), ("avgpool1d", False)):
        x, want = (np.array(v, np.float32) for v in golden[key]["arrays"])
        got = orc.pool2d(x.reshape(1, 1, 1, 6), (1, 2), (1, 2), (0, 0), is_max)  # [N,C,L] as H = 1
        assert np.array_equal(got.ravel(), want)
    for key, is_max in (("maxpool2d", True), ("avgpool2d", False)):
        x, want = (np.array(v, np.float32) for v in golden[key]["arrays"])
        assert np.array_equal(orc.pool2d(x.reshape(1, 1, 4, 4), (2, 2), (2, 2), (0, 0), is_max).ravel(), want)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_pooling_vs_torch(dtype):
    """torch as the independent routine: max_pool2d (pads with -inf: same winners), avg_pool2d with
    count_include_pad=False for the forward (the reference divides by the in-bounds count) and with
    count_include_pad=True for the backward (the reference's gradient scale is 1/kernel_area for every window)."""
    import oracle as orc
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(30)
    for (N, Cc, H, W, k, s, p) in [(2, 3, 8, 8, 2, 2, 0), (1, 2, 7, 9, 3, 2, 1), (2, 1, 6, 5, 3, 1, 1), (1, 1, 5, 5, 2, 1, 0), (1, 2, 9, 9, 3, 3, 1)]:
        x = rng.standard_normal((N, Cc, H, W)).astype(dtype)  # no ties
        tx = torch.from_numpy(x).double().requires_grad_(True)
        mp = F.max_pool2d(tx, k, s, p)
        g = rng.standard_normal(tuple(mp.shape)).astype(dtype)
        mp.backward(torch.from_numpy(g).double())
        omp = orc.pool2d(x, (k, k), (s, s), (p, p), True)
        assert np.array_equal(omp, mp.detach().numpy().astype(dtype))
        got = orc.unpool2d(g, x, omp, (k, k), (s, s), (p, p), True)
        assert np.allclose(got, tx.grad.numpy(), rtol=1e-6 if dtype == np.float32 else 1e-14, atol=1e-6 if dtype == np.float32 else 1e-14)
        ap = F.avg_pool2d(torch.from_numpy(x).double(), k, s, p, count_include_pad=False).numpy()
        oap = orc.pool2d(x, (k, k), (s, s), (p, p), False)
        assert np.allclose(oap, ap, rtol=1e-5 if dtype == np.float32 else 1e-13, atol=1e-6 if dtype == np.float32 else 1e-14)
        tx2 = torch.from_numpy(x).double().requires_grad_(True)
        F.avg_pool2d(tx2, k, s, p, count_include_pad=True).backward(torch.from_numpy(g).double())
        got = orc.unpool2d(g, x, oap, (k, k), (s, s), (p, p), False)
        # the reference rounds 1/kernel_area to f32 first, for f64 tensors too (pooling.rs:138): 1/9 is then off by 3e-9 relative
        assert np.allclose(got, tx2.grad.numpy(), rtol=1e-5 if dtype == np.float32 else 1e-7, atol=1e-6 if dtype == np.float32 else 1e-8)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_sign_not_in_range_pow_min_softmax_all_vs_numpy(dtype):
    import oracle as orc
    rng = np.random.default_rng(31)
    a = rng.standard_normal(1000).astype(dtype)
    a[::9] = 0
    assert np.array_equal(orc.unary("sign", a), np.sign(a))
    assert np.array_equal(orc.unary("logical_not", a), (a == 0).astype(dtype))
    assert np.array_equal(orc.in_range(a, -0.5, 0.25), ((a >= dtype(-0.5)) & (a <= dtype(0.25))).astype(dtype))
    b = np.abs(a) + dtype(0.1)
    e = rng.uniform(-2, 3, 1000).astype(dtype)
    tol = 1e-6 if dtype == np.float32 else 1e-14
    assert np.allclose(orc.binary("pow", b, e), np.power(b.astype(np.float64), e.astype(np.float64)), rtol=tol)
    assert np.allclose(orc.scalar("pow_scalar", b, 2.5), np.power(b.astype(np.float64), 2.5), rtol=tol)
    m = rng.standard_normal((6, 7, 5)).astype(dtype)
    m[2, 3, 1] = m[2, 5, 1] = -9.0  # tie: the first index wins
    for ax in range(3):
        v, i = orc.reduce_axis("min", m, ax, want_idx=True)
        assert np.array_equal(v, m.min(axis=ax)) and np.array_equal(i, m.argmin(axis=ax))
    x = (rng.standard_normal((3, 40)) * 4).astype(dtype)
    e64 = np.exp(x.astype(np.float64) - x.max())
    assert np.allclose(orc.softmax_all(x), e64 / e64.sum(), rtol=1e-5 if dtype == np.float32 else 1e-13)
