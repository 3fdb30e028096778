"""GPU parity for the rest of the storage trait behind the C ABI: elementwise min/max/comparisons of two tensors,
sign, logical_not, in_range, pow, min reduction (+argmin), the block-per-row softmax, and max/avg pooling with
their gradients.  Everything whose arithmetic order is defined is compared bit for bit with the CPU oracle."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

DTYPES = [np.float32, np.float64]
TOL = {np.dtype(np.float32): 1e-5, np.dtype(np.float64): 1e-12}


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


@pytest.mark.parametrize("dtype", DTYPES)
def test_elementwise_extras_bit_exact(ctx, orc, dtype):
    rng = np.random.default_rng(80)
    for n in (1, 5, 1000, 70001):
        a = rng.standard_normal(n).astype(dtype)
        b = rng.standard_normal(n).astype(dtype)
        a[::7] = 0
        b[::5] = a[::5]
        da, db = ctx.upload(a), ctx.upload(b)
        for op in ("min", "max", "greater", "greater_equal", "less", "less_equal", "equal"):
            assert np.array_equal(ctx.binary(op, da, db).numpy(), orc.binary(op, a, b)), (op, n)
        for op in ("sign", "logical_not", "abs", "reciprocal"):
            assert np.array_equal(ctx.unary(op, da).numpy(), orc.unary(op, a)), (op, n)
        assert np.array_equal(ctx.in_range(da, -0.5, 0.25).numpy(), orc.in_range(a, -0.5, 0.25)), n
        assert np.array_equal(ctx.scalar("less_scalar", da, 0.1).numpy(), orc.scalar("less_scalar", a, 0.1)), n


@pytest.mark.parametrize("dtype", DTYPES)
def test_pow_within_tolerance(ctx, orc, dtype):
    rng = np.random.default_rng(81)
    tol = TOL[np.dtype(dtype)]
    a = (np.abs(rng.standard_normal(5000)) + 0.05).astype(dtype)
    e = rng.uniform(-3, 3, 5000).astype(dtype)
    got = ctx.binary("pow", ctx.upload(a), ctx.upload(e)).numpy()
    np.testing.assert_allclose(got, np.power(a.astype(np.float64), e.astype(np.float64)), rtol=tol)
    np.testing.assert_allclose(got, orc.binary("pow", a, e), rtol=tol)
    got = ctx.scalar("pow_scalar", ctx.upload(a), 2.5).numpy()
    np.testing.assert_allclose(got, orc.scalar("pow_scalar", a, 2.5), rtol=tol)
    # squares of negative numbers (what power_scalar(2) is used for)
    b = rng.standard_normal(1000).astype(dtype)
    np.testing.assert_allclose(ctx.scalar("pow_scalar", ctx.upload(b), 2.0).numpy(), b.astype(np.float64) ** 2, rtol=tol)


@pytest.mark.parametrize("dtype", DTYPES)
def test_reduce_min_values_and_first_index(ctx, orc, dtype):
    rng = np.random.default_rng(82)
    for shape in [(7, 5), (3, 1000), (1000, 3), (4, 33, 9), (1, 70000), (2048, 257), (5, 4099, 3)]:
        m = rng.standard_normal(shape).astype(dtype)
        m.flat[rng.integers(0, m.size, 6)] = -50.0  # ties for the minimum
        dm = ctx.upload(m)
        for ax in range(len(shape)):
            v, i = ctx.reduce("min", dm, ax, want_idx=True)
            ov, oi = orc.reduce_axis("min", m, ax, want_idx=True)
            assert np.array_equal(v.numpy(), ov) and np.array_equal(i, oi), (shape, ax)
            assert np.array_equal(ov, m.min(axis=ax)) and np.array_equal(oi, m.argmin(axis=ax))
    big = np.full((3, 5), np.finfo(dtype).max, dtype)  # identity element: nothing is smaller
    v, i = ctx.reduce("min", ctx.upload(big), 1, want_idx=True)
    assert np.array_equal(v.numpy(), big.min(axis=1))


@pytest.mark.parametrize("dtype", DTYPES)
def test_softmax_long_rows_and_whole_tensor(ctx, orc, dtype):
    rng = np.random.default_rng(83)
    tol = TOL[np.dtype(dtype)]
    for shape in [(3, 5000), (1, 100000), (2, 2048)]:
        x = (rng.standard_normal(shape) * 3).astype(dtype)
        got = ctx.softmax_axis(ctx.upload(x), 1).numpy()
        e = np.exp(x.astype(np.float64) - x.max(axis=1, keepdims=True))
        truth = e / e.sum(axis=1, keepdims=True)
        assert np.abs(got - truth).max() <= 4 * tol * truth.max(), shape
        assert np.abs(got - orc.softmax_axis(x, 1)).max() <= 8 * tol * truth.max(), shape
        assert np.array_equal(got, ctx.softmax_axis(ctx.upload(x), 1).numpy())  # reproducible
    x = rng.standard_normal((40, 60)).astype(dtype)  # whole-tensor softmax = one row of 2400
    got = ctx.softmax_axis(ctx.upload(x.reshape(1, -1)), 1).numpy().reshape(x.shape)
    assert np.abs(got - orc.softmax_all(x)).max() <= 8 * tol * got.max()


POOL_CASES = [  # N, C, H, W, (kh, kw), (sh, sw), (ph, pw)
    (1, 1, 4, 4, (2, 2), (2, 2), (0, 0)), (2, 3, 8, 8, (2, 2), (2, 2), (0, 0)), (1, 2, 7, 9, (3, 3), (2, 2), (1, 1)),
    (2, 1, 6, 5, (3, 3), (1, 1), (1, 1)), (3, 4, 32, 32, (2, 2), (2, 2), (0, 0)), (2, 2, 9, 9, (3, 3), (3, 3), (1, 1)),
    (2, 3, 1, 11, (1, 2), (1, 2), (0, 0)), (2, 3, 1, 10, (1, 3), (1, 1), (0, 1)), (1, 1, 5, 7, (3, 2), (2, 1), (1, 0)),
    (1, 1, 3, 3, (3, 3), (1, 1), (2, 2)),
]


@pytest.mark.parametrize("dtype", DTYPES)
def test_pooling_and_unpooling_bit_exact(ctx, orc, dtype):
    rng = np.random.default_rng(84)
    for (N, Cc, H, W, k, s, p) in POOL_CASES:
        case = (N, Cc, H, W, k, s, p)
        x = rng.standard_normal((N, Cc, H, W)).astype(dtype)
        x[0, 0, 0, :2] = 1.5  # a tie inside a window: every tied position receives the gradient
        dx = ctx.upload(x)
        for is_max in (True, False):
            want = orc.pool2d(x, k, s, p, is_max)
            got = ctx.pool2d(dx, k, s, p, is_max)
            assert np.array_equal(got.numpy(), want), (case, is_max)
            g = rng.standard_normal(want.shape).astype(dtype)
            gi = ctx.unpool2d(ctx.upload(g), dx, got, k, s, p, is_max).numpy()
            assert np.array_equal(gi, orc.unpool2d(g, x, want, k, s, p, is_max)), (case, is_max)


def test_pooling_reference_vectors(ctx, golden):
    for key, is_max, shape, k in (("maxpool1d", True, (1, 1, 1, 6), (1, 2)), ("avgpool1d", False, (1, 1, 1, 6), (1, 2)),
                                  ("maxpool2d", True, (1, 1, 4, 4), (2, 2)), ("avgpool2d", False, (1, 1, 4, 4), (2, 2))):
        x, want = (np.array(v, np.float32) for v in golden[key]["arrays"])
        got = ctx.pool2d(ctx.upload(x.reshape(shape)), k, k, (0, 0), is_max).numpy()
        assert np.array_equal(got.ravel(), want), key


def test_device_to_device_copy_moves_every_bit_pattern(ctx):
    """fx_d2d: small blocks run as a copy kernel, large / odd ones through the runtime; random 32-bit patterns (NaN payloads,
    denormals, both zeros) must arrive unchanged at every size and alignment."""
    import ctypes as C
    from ferrox_amd.capi import check, lib
    rng = np.random.default_rng(77)
    n = (40 << 20) // 4 + 3
    bits = rng.integers(0, 2 ** 32, n, dtype=np.uint32)
    bits[:4] = [0x7FC00001, 0x7F800001, 0x80000000, 0x00000001]   # quiet NaN with payload, signalling NaN, -0, denormal
    src = ctx.upload(bits.view(np.float32))
    dst = ctx.fill((n + 8,), 0.0, np.float32)
    for off_src, off_dst, nbytes in [(0, 0, 4), (0, 0, 16), (4, 8, 4 * 1027), (0, 4, 1 << 20), (12, 0, (1 << 20) + 4), (0, 0, 3),
                                     (1, 2, 1001), (0, 0, 32 << 20), (0, 0, (32 << 20) + 4), (4, 4, 40 << 20), (0, 0, 0)]:
        check(lib.fx_fill_f32(ctx.h, dst.ptr, C.c_float(0.0), n + 8))
        check(lib.fx_d2d(ctx.h, dst.ptr + off_dst, src.ptr + off_src, nbytes))
        got = dst.numpy().view(np.uint8)
        want = np.zeros((n + 8) * 4, np.uint8)
        want[off_dst:off_dst + nbytes] = bits.view(np.uint8)[off_src:off_src + nbytes]
        assert np.array_equal(got, want), (off_src, off_dst, nbytes)
