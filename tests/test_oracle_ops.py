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
