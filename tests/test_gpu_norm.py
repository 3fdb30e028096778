"""GPU parity for the layers of the reference's CNN example beyond conv/linear: BatchNorm (statistics, forward,
backward, running statistics), Dropout and the product reduction, through the C ABI.
Bit for bit where the arithmetic order is defined (BatchNorm forward given mean/var, the running update, the
fixed-statistics dx, dropout); rel 1e-5 (f32) / 1e-12 (f64) of the largest magnitude where a summation order differs."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

DTYPES = [np.float32, np.float64]
TOL = {np.dtype(np.float32): 1e-5, np.dtype(np.float64): 1e-12}
# planar vector path, planar scalar path (odd inner), column paths (inner 9 and inner 1), one slice and many slices
BN_SHAPES = [(64, 8, 16, 16), (5, 3, 5, 5), (6, 4, 3, 3), (64, 10), (1030, 7), (300, 5, 8, 8), (2, 3, 4, 4), (33, 2, 7, 9)]


@pytest.fixture(scope="module")
def ctx():
    from ferrox_amd import capi
    c = capi.Context(0)
    yield c
    c.close()


@pytest.fixture(scope="module")
def orc():
    import oracle
    return oracle


def close(got, ref, tol):
    scale = max(1e-30, float(np.abs(ref).max()))
    return float(np.abs(got - ref).max()) <= tol * scale


@pytest.mark.parametrize("dtype", DTYPES)
def test_batchnorm_stats_match_oracle_and_float64(ctx, orc, dtype):
    import oracle.train as tr
    rng = np.random.default_rng(90)
    tol = TOL[np.dtype(dtype)]
    for shape in BN_SHAPES:
        C = shape[1]
        x = (rng.standard_normal(shape) * rng.uniform(0.5, 3.0, (1, C) + (1,) * (len(shape) - 2))
             + rng.uniform(-2, 2, (1, C) + (1,) * (len(shape) - 2))).astype(dtype)
        axes = (0, 2, 3) if len(shape) == 4 else (0,)
        rm0, rv0 = rng.standard_normal(C).astype(dtype), rng.uniform(0.5, 2, C).astype(dtype)
        drm, drv = ctx.upload(rm0), ctx.upload(rv0)
        mean, var = ctx.batchnorm_stats(ctx.upload(x), drm, drv, 0.1)
        mean, var = mean.numpy(), var.numpy()
        _, _, omean, ovar = tr.batchnorm_forward(x, np.ones(C, dtype), np.zeros(C, dtype), 1e-5)
        x64 = x.astype(np.float64)
        assert close(mean, x64.mean(axis=axes), tol) and close(var, x64.var(axis=axes), 4 * tol), shape
        assert close(mean, omean, tol) and close(var, ovar, 4 * tol), shape
        # the running update is the reference's three operators applied to the batch statistics: bit-exact
        assert np.array_equal(drm.numpy(), tr.batchnorm_running_update(rm0, mean, 0.1)), shape
        assert np.array_equal(drv.numpy(), tr.batchnorm_running_update(rv0, var, 0.1)), shape


def test_batchnorm_stats_large_offset_f32(ctx):
    """mean >> std: a sum-of-squares formula would lose every digit of the variance here."""
    rng = np.random.default_rng(91)
    x = (1000.0 + rng.standard_normal((32, 4, 24, 24))).astype(np.float32)
    x[0, 1, 0, 0] = 5000.0  # an outlier as the first element of a channel
    mean, var = ctx.batchnorm_stats(ctx.upload(x))
    x64 = x.astype(np.float64)
    np.testing.assert_allclose(mean.numpy(), x64.mean(axis=(0, 2, 3)), rtol=1e-6)
    np.testing.assert_allclose(var.numpy(), x64.var(axis=(0, 2, 3)), rtol=1e-4)


@pytest.mark.parametrize("dtype", DTYPES)
def test_batchnorm_forward_bit_exact_given_statistics(ctx, orc, dtype):
    import oracle.train as tr
    rng = np.random.default_rng(92)
    for shape in BN_SHAPES:
        C = shape[1]
        x = (rng.standard_normal(shape) * 2 + 0.5).astype(dtype)
        gamma, beta = rng.uniform(0.5, 1.5, C).astype(dtype), rng.standard_normal(C).astype(dtype)
        ref, _, mean, var = tr.batchnorm_forward(x, gamma, beta, 1e-3)              # training: batch statistics
        got = ctx.batchnorm_fwd(ctx.upload(x), ctx.upload(mean), ctx.upload(var), ctx.upload(gamma), ctx.upload(beta), 1e-3)
        assert np.array_equal(got.numpy(), ref), shape
        rm, rv = rng.standard_normal(C).astype(dtype), rng.uniform(0.5, 2, C).astype(dtype)
        ref, _, _, _ = tr.batchnorm_forward(x, gamma, beta, 1e-3, False, rm, rv)   # inference: running statistics
        got = ctx.batchnorm_fwd(ctx.upload(x), ctx.upload(rm), ctx.upload(rv), ctx.upload(gamma), ctx.upload(beta), 1e-3)
        assert np.array_equal(got.numpy(), ref), shape


@pytest.mark.parametrize("dtype", DTYPES)
def test_batchnorm_backward_matches_composed_autograd(ctx, orc, dtype):
    import oracle.train as tr
    rng = np.random.default_rng(93)
    tol = TOL[np.dtype(dtype)]
    for shape in BN_SHAPES:
        C = shape[1]
        x = (rng.standard_normal(shape) * 2 + 0.5).astype(dtype)
        g = rng.standard_normal(shape).astype(dtype)
        gamma, beta = rng.uniform(0.5, 1.5, C).astype(dtype), rng.standard_normal(C).astype(dtype)
        _, rec, mean, var = tr.batchnorm_forward(x, gamma, beta, 1e-3)
        rdx, rdg, rdb = tr.batchnorm_backward(g, rec)
        dx, dg, db = ctx.batchnorm_bwd(ctx.upload(g), ctx.upload(x), ctx.upload(mean), ctx.upload(var), ctx.upload(gamma), 1e-3)
        # the sums cancel (dx is orthogonal to 1 and to x - mean), so the tolerance is on the scale of the terms: |g|*gamma/std
        scale = float(np.abs(g).max() * np.abs(gamma).max() / np.sqrt(var.min() + 1e-3))
        assert float(np.abs(dx.numpy() - rdx).max()) <= 8 * tol * scale, shape
        n = x.size // C
        assert float(np.abs(dg.numpy() - rdg).max()) <= tol * n * 4 and float(np.abs(db.numpy() - rdb).max()) <= tol * n * 4, shape
        assert close(dg.numpy(), rdg, 20 * tol) or np.abs(rdg).max() < 1e-3 * n
        # fixed statistics (inference graph): dx is two operators, bit-exact
        rm, rv = rng.standard_normal(C).astype(dtype), rng.uniform(0.5, 2, C).astype(dtype)
        _, rec, _, _ = tr.batchnorm_forward(x, gamma, beta, 1e-3, False, rm, rv)
        rdx, rdg, rdb = tr.batchnorm_backward(g, rec)
        dx, dg, db = ctx.batchnorm_bwd(ctx.upload(g), ctx.upload(x), ctx.upload(rm), ctx.upload(rv), ctx.upload(gamma), 1e-3,
                                       batch_stats=False)
        assert np.array_equal(dx.numpy(), rdx), shape
        assert float(np.abs(dg.numpy() - rdg).max()) <= tol * n * 8 and float(np.abs(db.numpy() - rdb).max()) <= tol * n * 4, shape
        _, dg2, db2 = ctx.batchnorm_bwd(ctx.upload(g), ctx.upload(x), ctx.upload(rm), ctx.upload(rv), ctx.upload(gamma), 1e-3,
                                        batch_stats=False, need_dx=False)
        assert np.array_equal(dg2.numpy(), dg.numpy()) and np.array_equal(db2.numpy(), db.numpy())


@pytest.mark.parametrize("dtype", DTYPES)
def test_batchnorm_with_folded_relu_equals_batchnorm_then_relu(ctx, orc, dtype):
    """act = 1 / y_act: the ReLU layer that follows BatchNorm in the reference's models, in the same kernels."""
    import oracle.train as tr
    rng = np.random.default_rng(96)
    tol = TOL[np.dtype(dtype)]
    for shape in BN_SHAPES:
        C = shape[1]
        x = (rng.standard_normal(shape) * 2 + 0.5).astype(dtype)
        g = rng.standard_normal(shape).astype(dtype)
        gamma, beta = rng.uniform(0.5, 1.5, C).astype(dtype), rng.standard_normal(C).astype(dtype)
        pre, rec, mean, var = tr.batchnorm_forward(x, gamma, beta, 1e-3)
        dmean, dvar, dgam, dbet = ctx.upload(mean), ctx.upload(var), ctx.upload(gamma), ctx.upload(beta)
        y = ctx.batchnorm_fwd(ctx.upload(x), dmean, dvar, dgam, dbet, 1e-3, relu=True)
        assert np.array_equal(y.numpy(), orc.unary("relu", pre)), shape
        g_pre = orc.binary("mul", g, orc.scalar("greater_scalar", pre, dtype(0)))       # ReLU::gradient
        rdx, rdg, rdb = tr.batchnorm_backward(g_pre, rec)
        dx, dg, db = ctx.batchnorm_bwd(ctx.upload(g), ctx.upload(x), dmean, dvar, dgam, 1e-3, y_act=y)
        scale = float(np.abs(g).max() * np.abs(gamma).max() / np.sqrt(var.min() + 1e-3))
        n = x.size // C
        assert float(np.abs(dx.numpy() - rdx).max()) <= 8 * tol * scale, shape
        assert float(np.abs(dg.numpy() - rdg).max()) <= tol * n * 4 and float(np.abs(db.numpy() - rdb).max()) <= tol * n * 4, shape
        # the same through the unfused pair of calls: identical bits (same kernels, mask applied at load)
        dx2, dg2, db2 = ctx.batchnorm_bwd(ctx.upload(g_pre), ctx.upload(x), dmean, dvar, dgam, 1e-3)
        assert np.array_equal(dx.numpy(), dx2.numpy()) and np.array_equal(dg.numpy(), dg2.numpy()) and np.array_equal(db.numpy(), db2.numpy())
        rm, rv = rng.standard_normal(C).astype(dtype), rng.uniform(0.5, 2, C).astype(dtype)
        pre, rec, _, _ = tr.batchnorm_forward(x, gamma, beta, 1e-3, False, rm, rv)
        y = ctx.batchnorm_fwd(ctx.upload(x), ctx.upload(rm), ctx.upload(rv), dgam, dbet, 1e-3, relu=True)
        assert np.array_equal(y.numpy(), orc.unary("relu", pre)), shape
        g_pre = orc.binary("mul", g, orc.scalar("greater_scalar", pre, dtype(0)))
        rdx, _, _ = tr.batchnorm_backward(g_pre, rec)
        dx, _, _ = ctx.batchnorm_bwd(ctx.upload(g), ctx.upload(x), ctx.upload(rm), ctx.upload(rv), dgam, 1e-3, batch_stats=False, y_act=y)
        assert np.array_equal(dx.numpy(), rdx), shape


def test_batchnorm_full_size_properties(ctx):
    """[256, 32, 32, 32] f32 (the first activation of the CNN configuration): normalised output has zero mean and unit
    variance per channel; dx sums to zero against 1 and against x - mean."""
    shape = (256, 32, 32, 32)
    x = ctx.normal(shape, 11, 0.7, 1.9)
    g = ctx.normal(shape, 12, 0.0, 1.0)
    ones, zeros = ctx.upload(np.ones(32, np.float32)), ctx.upload(np.zeros(32, np.float32))
    mean, var = ctx.batchnorm_stats(x)
    assert np.abs(mean.numpy() - 0.7).max() < 0.02 and np.abs(var.numpy() - 1.9 ** 2).max() < 0.05
    y = ctx.batchnorm_fwd(x, mean, var, ones, zeros, 0.0)
    m2, v2 = ctx.batchnorm_stats(y)
    assert np.abs(m2.numpy()).max() < 1e-5 and np.abs(v2.numpy() - 1).max() < 1e-5
    dx, dg, db = ctx.batchnorm_bwd(g, x, mean, var, ones, 0.0)
    s1 = ctx.bias_grad(dx, 256, 32, 1024).numpy()
    n = 256 * 1024
    assert np.abs(s1).max() / n < 1e-6
    _, dg2, _ = ctx.batchnorm_bwd(dx, x, mean, var, ones, 0.0, need_dx=False)     # sum dx * xhat
    assert np.abs(dg2.numpy()).max() / n < 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
def test_dropout_mask_bit_exact_and_keep_rate(ctx, orc, dtype):
    rng = np.random.default_rng(94)
    for n, p, seed in [(1, 0.5, 3), (1001, 0.3, 77), (4096, 0.9, 2 ** 40 + 5), (70000, 0.0, 9)]:
        x = rng.standard_normal(n).astype(dtype)
        y, mask = ctx.dropout(ctx.upload(x), p, seed)
        ref = orc.dropout_mask((n,), p, seed, dtype)
        assert np.array_equal(mask.numpy(), ref), (n, p)
        assert np.array_equal(y.numpy(), orc.binary("mul", x, ref)), (n, p)
    n, p = 1 << 22, 0.3
    y, mask = ctx.dropout(ctx.fill((n,), 1.0, dtype), p, 1234)
    kept = np.count_nonzero(mask.numpy()) / n
    assert abs(kept - (1 - p)) < 5 * np.sqrt(p * (1 - p) / n)
    assert np.array_equal(np.unique(mask.numpy()), np.array([0, dtype(1.0 / (1.0 - p))], dtype))
    with pytest.raises(Exception):
        ctx.dropout(ctx.fill((8,), 1.0, dtype), 1.0, 1)


@pytest.mark.parametrize("dtype", DTYPES)
def test_reduce_prod_within_tolerance(ctx, orc, dtype):
    rng = np.random.default_rng(95)
    tol = TOL[np.dtype(dtype)]
    for shape in [(7, 5), (3, 1000), (1000, 3), (4, 33, 9), (1, 70000), (2048, 257), (5, 4099, 3)]:
        m = rng.uniform(0.97, 1.03, shape).astype(dtype) * rng.choice([-1.0, 1.0], shape, p=[0.1, 0.9]).astype(dtype)
        dm = ctx.upload(m)
        for ax in range(len(shape)):
            got = ctx.reduce("prod", dm, ax).numpy()
            ref64 = m.astype(np.float64).prod(axis=ax)
            k = shape[ax]
            np.testing.assert_allclose(got, ref64, rtol=tol * max(1, k / 8), err_msg=str((shape, ax)))
            np.testing.assert_allclose(got, orc.reduce_axis("prod", m, ax), rtol=tol * max(1, k / 4), err_msg=str((shape, ax)))
    z = np.ones((4, 100), dtype)
    z[2, 17] = 0
    assert np.array_equal(ctx.reduce("prod", ctx.upload(z), 1).numpy(), np.array([1, 1, 0, 1], dtype))


def test_new_entry_points_reject_bad_arguments(ctx):
    """Argument checks run on the host before any launch: null pointers, empty or negative views, bad flags."""
    from ferrox_amd import capi
    from ferrox_amd.capi import FerroxHipError
    x = ctx.fill((4, 3, 5, 5), 1.0)
    v3 = ctx.fill((3,), 1.0)
    lib, h = capi.lib, ctx.h

    def fails(rc, text):
        with pytest.raises(FerroxHipError, match=text):
            capi.check(rc)

    fails(lib.fx_batchnorm_stats_f32(h, None, v3.ptr, v3.ptr, None, None, 0.1, 4, 3, 25), "null pointer")
    fails(lib.fx_batchnorm_stats_f32(h, x.ptr, v3.ptr, v3.ptr, None, None, 0.1, 0, 3, 25), "bad view")
    fails(lib.fx_batchnorm_fwd_f32(h, x.ptr, v3.ptr, v3.ptr, v3.ptr, None, 1e-5, x.ptr, 4, 3, 25, 0), "null pointer")
    fails(lib.fx_batchnorm_fwd_f32(h, x.ptr, v3.ptr, v3.ptr, v3.ptr, v3.ptr, 1e-5, x.ptr, 4, 3, 25, 2), "act must be")
    fails(lib.fx_batchnorm_bwd_f32(h, x.ptr, x.ptr, None, v3.ptr, v3.ptr, v3.ptr, 1e-5, x.ptr, v3.ptr, None, 4, 3, 25, 1), "null pointer")
    fails(lib.fx_batchnorm_bwd_f32(h, x.ptr, x.ptr, None, v3.ptr, v3.ptr, v3.ptr, 1e-5, x.ptr, v3.ptr, v3.ptr, 4, 3, 25, 7), "batch_stats")
    fails(lib.fx_dropout_f32(h, x.ptr, x.ptr, x.ptr, 300, 1.0, 1), r"p must be in \[0, 1\)")
    fails(lib.fx_dropout_f32(h, x.ptr, None, x.ptr, 300, 0.5, 1), "null pointer")
    fails(lib.fx_reduce_prod_f32(h, x.ptr, None, 4, 75, 1), "null pointer")
    import ctypes as C
    tab = (C.c_void_p * 2)(x.ptr, None)
    ns = (C.c_int64 * 2)(300, 300)
    fails(lib.fx_adam_step_multi_f32(h, 2, tab, tab, tab, tab, ns, 1e-3, 0.9, 0.999, 1e-8, 0.0, 0.1, 0.001), "null pointer in tensor 1")
    fails(lib.fx_sgd_step_multi_f32(h, -1, tab, tab, ns, 0.1), "negative tensor count")
    assert lib.fx_dropout_f32(h, x.ptr, x.ptr, x.ptr, 0, 0.5, 1) == 0          # nothing to do is not an error
    assert lib.fx_batchnorm_fwd_f32(h, None, None, None, None, None, 1e-5, None, 0, 3, 25, 0) == 0
