"""GPU parity tests: every kernel family of libferrox_hip.so, called through the C ABI, against the CPU oracle
on the same seeded inputs.  Bit-exact where the arithmetic order is defined (data movement, elementwise
compositions, max/argmax); rel 1e-5 (f32) / 1e-12 (f64) against a float64/longdouble ground truth elsewhere."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import parity
from parity import TOL

DTYPES = [np.float32, np.float64]


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


def rel_err(got, ref):
    ref = np.asarray(ref, dtype=np.float64)
    return np.abs(np.asarray(got, dtype=np.float64) - ref).max() / max(1e-30, np.abs(ref).max())


# ------------------------------------------------------------------------------------------ elementwise
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [1, 3, 4, 1023, 1024, 4099, 1 << 20])
def test_binary_ops_bit_exact(ctx, orc, dtype, n):
    rng = np.random.default_rng(n)
    a = rng.uniform(-4, 4, n).astype(dtype)
    b = rng.uniform(-4, 4, n).astype(dtype)
    b[::7] = a[::7]  # exercise equality
    da, db = ctx.upload(a), ctx.upload(b)
    for op in ("add", "sub", "mul", "div", "equal", "greater", "greater_equal", "less", "less_equal", "min", "max"):
        got = ctx.binary(op, da, db).numpy()
        assert np.array_equal(got, orc.binary(op, a, b)), op


@pytest.mark.parametrize("dtype", DTYPES)
def test_division_by_zero_follows_ieee_like_cpu(ctx, orc, dtype):
    a = np.array([1.0, -1.0, 0.0, 2.0], dtype)
    b = np.array([0.0, 0.0, 0.0, 4.0], dtype)
    got = ctx.binary("div", ctx.upload(a), ctx.upload(b)).numpy()
    with np.errstate(all="ignore"):
        ref = orc.binary("div", a, b)
    assert np.array_equal(got, ref, equal_nan=True)


@pytest.mark.parametrize("dtype", DTYPES)
def test_scalar_and_clamp_bit_exact(ctx, orc, dtype):
    rng = np.random.default_rng(11)
    a = rng.uniform(-4, 4, 70001).astype(dtype)
    da = ctx.upload(a)
    for op, s in (("add_scalar", 1.5), ("sub_scalar", 1.0), ("mul_scalar", 0.01), ("div_scalar", 3.0), ("greater_scalar", 0.0),
                  ("greater_equal_scalar", 1e-8), ("less_equal_scalar", 0.5), ("less_scalar", 0.0)):
        assert np.array_equal(ctx.scalar(op, da, s).numpy(), orc.scalar(op, a, dtype(s))), op
    lo, hi = dtype(1e-8), dtype(1.0 - 1e-8)
    assert np.array_equal(ctx.clamp(da, lo, hi).numpy(), orc.clamp(a, lo, hi))


@pytest.mark.parametrize("dtype", DTYPES)
def test_unary_ops(ctx, orc, dtype):
    rng = np.random.default_rng(12)
    a = rng.uniform(-4, 4, 100003).astype(dtype)
    a[:6] = [0.0, -0.0, 25.0, -25.0, 1000.0, -1000.0]
    da = ctx.upload(a)
    pos = ctx.upload(np.abs(a) + dtype(1e-3))
    for op in ("neg", "relu", "abs"):  # exact ops
        assert np.array_equal(ctx.unary(op, da).numpy(), orc.unary(op, a)), op
    for op in ("exp", "sigmoid", "tanh"):  # libm vs device math: elementwise relative tolerance
        with np.errstate(over="ignore"):
            ref = orc.unary(op, a.astype(np.float64)).astype(dtype)  # overflow to inf exactly where T overflows
        # tanh's exp-based formula (cpu.rs:1120-1146) cancels near 0 in T on CPU and GPU alike: allow a few ulp of 1.0
        atol = 4 * np.finfo(dtype).eps if op == "tanh" else 0
        np.testing.assert_allclose(ctx.unary(op, da).numpy(), ref, rtol=TOL[np.dtype(dtype)], atol=atol, err_msg=op)
    for op in ("sqrt", "log", "reciprocal"):
        ref = orc.unary(op, (np.abs(a) + dtype(1e-3)).astype(np.float64))
        parity.check("unary " + op, ctx.unary(op, pos).numpy(), ref)
    # saturation like the CPU backend (tensor.rs:2667-2729): exactly +-1 beyond |x| > 20, sigmoid -> 0 / 1
    t = ctx.unary("tanh", da).numpy()
    assert t[2] == 1.0 and t[3] == -1.0 and t[4] == 1.0 and t[5] == -1.0
    s = ctx.unary("sigmoid", da).numpy()
    assert s[4] == 1.0 and s[5] == 0.0


def test_reference_activation_vectors(ctx, golden):
    for key, op in (("relu", "relu"), ("sigmoid", "sigmoid"), ("tanh", "tanh"), ("neg", "neg")):
        x, y = (np.array(v, np.float32) for v in golden[key]["arrays"])
        got = ctx.unary(op, ctx.upload(x)).numpy()
        np.testing.assert_allclose(got, y, atol=1e-4, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_activation_backward_bit_exact_vs_composed_cpu(ctx, orc, dtype):
    rng = np.random.default_rng(13)
    n = 300007
    g = rng.uniform(-4, 4, n).astype(dtype)
    x = rng.uniform(-4, 4, n).astype(dtype)
    x[:3] = [0.0, -0.0, 1e-30]
    dg, dx = ctx.upload(g), ctx.upload(x)
    assert np.array_equal(ctx.relu_bwd(dg, dx).numpy(), orc.relu_bwd(g, x))
    s = orc.unary("sigmoid", x)
    t = orc.unary("tanh", x)
    ds, dt = ctx.upload(s), ctx.upload(t)
    for lit in (0, 1):
        assert np.array_equal(ctx.sigmoid_bwd(dg, ds, lit).numpy(), orc.sigmoid_bwd(g, s, lit))
    assert np.array_equal(ctx.tanh_bwd(dg, dt).numpy(), orc.tanh_bwd(g, t))
    # the fused kernels equal the reference's op-by-op composition run on the GPU (src/ops/unary.rs:358-375)
    mask = ctx.scalar("greater_scalar", dx, 0.0)
    assert np.array_equal(ctx.binary("mul", dg, mask).numpy(), ctx.relu_bwd(dg, dx).numpy())
    # correct-mode sigmoid gradient against the closed form in float64
    ref = g.astype(np.float64) * s.astype(np.float64) * (1 - s.astype(np.float64))
    assert rel_err(ctx.sigmoid_bwd(dg, ds, 0).numpy(), ref) <= TOL[np.dtype(dtype)]


@pytest.mark.parametrize("dtype", DTYPES)
def test_fill_and_materialize(ctx, orc, dtype):
    assert np.array_equal(ctx.fill((3, 5, 7), 2.5, dtype).numpy(), np.full((3, 5, 7), 2.5, dtype))
    rng = np.random.default_rng(14)
    bias = rng.standard_normal(32).astype(dtype)
    # bias [C] -> [1,C,1,1] -> broadcast [B,C,H,W]  (src/nn/layers/utils.rs:6-42)
    got = ctx.materialize(ctx.upload(bias), (4, 32, 5, 6), (0, 1, 0, 0)).numpy()
    assert np.array_equal(got, np.broadcast_to(bias.reshape(1, 32, 1, 1), (4, 32, 5, 6)))
    assert np.array_equal(got, orc.materialize(bias, (4, 32, 5, 6), (0, 1, 0, 0)))
    m = rng.standard_normal((37, 53)).astype(dtype)
    got = ctx.materialize(ctx.upload(m), (53, 37), (1, 53)).numpy()  # transpose
    assert np.array_equal(got, m.T)


@pytest.mark.parametrize("dtype", DTYPES)
def test_materialize_views_bit_exact(ctx, dtype):
    """Broadcasts, permutations, slices-with-step and 5..8-dim views against numpy's as_strided (element strides):
    covers the vector kernel (contiguous or broadcast inner dim, aligned and misaligned source), the 32-bit
    one-element kernel and the collapse of mergeable dims."""
    from numpy.lib.stride_tricks import as_strided
    rng = np.random.default_rng(15)
    base = rng.standard_normal(40000).astype(dtype)
    dbase = ctx.upload(base)
    item = base.itemsize
    views = [
        ((256, 32, 8, 8), (0, 1, 0, 0)),          # bias broadcast, inner dims merge to one broadcast dim
        ((64, 128), (0, 1)), ((128, 64), (1, 0)),  # row / column broadcast
        ((100, 64), (1, 100)), ((37, 53), (53, 1)), ((53, 37), (1, 53)),  # transposes and identity
        ((6, 5, 4, 8), (160, 8, 40, 1)),           # permute with contiguous inner dim
        ((3, 4, 5, 6), (1, 3, 12, 60)),            # full reversal of a [6,5,4,3] tensor
        ((7, 12), (24, 2)), ((5, 9, 4), (0, 4, 1)), ((2, 3, 1, 4, 1, 5), (60, 20, 0, 5, 0, 1)),
        ((2, 2, 2, 2, 2, 2, 2, 4), (512, 1024, 64, 128, 16, 32, 4, 1)), ((1,), (0,)), ((9,), (3,)), ((16,), (0,)),
        # the LDS-tiled transpose: ragged tiles, a batch of transposes, a padded leading dimension, a broadcast batch
        ((130, 67), (1, 130)), ((5, 70, 33), (2310, 1, 70)), ((40, 50), (1, 64)), ((4, 30, 20), (0, 1, 30)), ((16, 16), (1, 16)),
        ((15, 64), (1, 15)), ((3, 17, 19), (400, 1, 21)),
    ]
    for shape, strides in views:
        want = np.ascontiguousarray(as_strided(base, shape, tuple(s_ * item for s_ in strides)))
        got = ctx.materialize(dbase, shape, strides).numpy()
        assert np.array_equal(got, want), (shape, strides)
    # a source that is only element-aligned (view starting one element into the buffer)
    from ferrox_amd import capi
    shape, strides = (32, 64), (64, 1)
    out = ctx.empty(shape, dtype)
    sh, st = (capi._i64 * 2)(*shape), (capi._i64 * 2)(*strides)
    capi.check(ctx._fn("materialize", np.dtype(dtype))(ctx.h, dbase.ptr + item, out.ptr, sh, st, 2, 32 * 64))
    assert np.array_equal(out.numpy(), base[1:1 + 2048].reshape(shape))


# ------------------------------------------------------------------------------------------ im2col / col2im
GEOMS = [  # B, C, H, W, k, s, p
    (1, 1, 5, 5, 3, 1, 1), (2, 3, 8, 7, 3, 1, 1), (3, 2, 9, 9, 3, 2, 1), (2, 2, 6, 6, 2, 2, 0), (2, 3, 7, 5, 1, 1, 0),
    (32, 1, 28, 28, 3, 1, 1), (4, 3, 32, 32, 3, 1, 1), (4, 32, 32, 32, 3, 2, 1),
]


@pytest.mark.parametrize("dtype", DTYPES)
def test_im2col_col2im_bit_exact(ctx, orc, dtype):
    rng = np.random.default_rng(20)
    for (B, Cc, H, W, k, s, p) in GEOMS:
        x = rng.uniform(-1, 1, (B, Cc, H, W)).astype(dtype)
        col = ctx.im2col(ctx.upload(x), (k, k), (s, s), (p, p))
        ref = orc.im2col(x, (k, k), (s, s), (p, p))
        assert np.array_equal(col.numpy(), ref), (B, Cc, H, W, k, s, p)
        c2 = rng.standard_normal(ref.shape).astype(dtype)
        dc2 = ctx.upload(c2)
        for layout in (0, 1):
            got = ctx.col2im(dc2, x.shape, (k, k), (s, s), (p, p), layout).numpy()
            assert np.array_equal(got, orc.col2im(c2, x.shape, (k, k), (s, s), (p, p), layout)), (layout, B, Cc, H, W, k, s, p)


def test_im2col_rectangular(ctx, orc):
    rng = np.random.default_rng(21)
    x = rng.uniform(-1, 1, (2, 2, 9, 6)).astype(np.float32)
    for k, s, p in [((3, 2), (2, 1), (1, 0)), ((1, 3), (1, 2), (0, 1)), ((2, 2), (1, 1), (2, 2))]:
        assert np.array_equal(ctx.im2col(ctx.upload(x), k, s, p).numpy(), orc.im2col(x, k, s, p))


# ------------------------------------------------------------------------------------------ reductions
RED_SHAPES = [(2, 2), (7, 13), (256, 10), (64, 1000), (3, 5, 7), (16, 32, 8, 8), (1, 70001), (5000, 33), (300, 4100), (2049, 515),
              # short last axes that are whole 16-byte vectors (one vector per lane, several rows per thread): 1 to 64 vectors per row,
              # row counts that end inside a block's pass, more rows than one grid dimension holds
              (37, 4), (1029, 12), (8, 32, 32), (515, 36), (100, 64), (77, 100), (33, 128), (9, 256), (70001, 8), (3, 2)]


@pytest.mark.parametrize("dtype", DTYPES)
def test_reduce_every_axis(ctx, orc, dtype):
    rng = np.random.default_rng(30)
    for shape in RED_SHAPES:
        x = rng.standard_normal(shape).astype(dtype)
        dx = ctx.upload(x)
        for axis in range(len(shape)):
            truth = x.astype(np.longdouble).sum(axis=axis)
            terms = np.abs(x).astype(np.float64).sum(axis=axis).max()
            got = ctx.reduce("sum", dx, axis).numpy()
            # the GPU's summation order and the oracle's CPU order, each against the long double sum
            parity.check("reduce sum", got, truth, oracle=orc.reduce_axis("sum", x, axis), case=(shape, axis), terms=terms)
            got = ctx.reduce("mean", dx, axis).numpy()
            parity.check("reduce mean", got, truth / shape[axis], oracle=orc.reduce_axis("mean", x, axis), case=(shape, axis),
                         terms=terms / shape[axis])
            v, i = ctx.reduce("max", dx, axis, want_idx=True)
            rv, ri = orc.reduce_axis("max", x, axis, want_idx=True)
            assert np.array_equal(v.numpy(), rv), ("max", shape, axis)
            assert np.array_equal(i, ri) and np.array_equal(i, np.argmax(x, axis=axis)), ("argmax", shape, axis)
            # without the positions (the value-only accumulator): the same values, and the minimum likewise
            assert np.array_equal(ctx.reduce("max", dx, axis).numpy(), rv), ("max, no index", shape, axis)
            mv, mi = ctx.reduce("min", dx, axis, want_idx=True)
            assert np.array_equal(mv.numpy(), x.min(axis=axis)) and np.array_equal(mi, np.argmin(x, axis=axis)), ("min", shape, axis)
            assert np.array_equal(ctx.reduce("min", dx, axis).numpy(), x.min(axis=axis)), ("min, no index", shape, axis)


@pytest.mark.parametrize("dtype", DTYPES)
def test_reduce_all_and_ties(ctx, orc, dtype):
    rng = np.random.default_rng(31)
    x = rng.integers(-3, 4, (1 << 21) + 5).astype(dtype)  # many ties: first occurrence must win
    dx = ctx.upload(x)
    v, i = ctx.reduce("max", dx, 0, want_idx=True)
    assert v.numpy().item() == x.max() and i.item() == int(np.argmax(x))
    assert ctx.reduce("sum", dx, 0).numpy().item() == x.astype(np.float64).sum()  # small integers: exact in any order
    y = rng.integers(-2, 3, (513, 1031)).astype(dtype)
    dy = ctx.upload(y)
    for axis in (0, 1):
        v, i = ctx.reduce("max", dy, axis, want_idx=True)
        assert np.array_equal(i, np.argmax(y, axis=axis)) and np.array_equal(v.numpy(), y.max(axis=axis))
        assert np.array_equal(ctx.reduce("sum", dy, axis).numpy(), y.sum(axis=axis))


def test_reduce_max_identity_and_nan(ctx, orc):
    lowest = np.finfo(np.float32).min
    x = np.array([[-np.inf, -np.inf, -np.inf], [np.nan, 1.0, 2.0], [lowest, lowest, -np.inf]], np.float32)
    v, i = ctx.reduce("max", ctx.upload(x), 1, want_idx=True)
    rv, ri = orc.reduce_axis("max", x, 1, want_idx=True)
    assert np.array_equal(v.numpy(), rv) and np.array_equal(i, ri)
    assert v.numpy()[0] == lowest and i[0] == 0 and i[1] == 2
    assert np.array_equal(ctx.reduce("max", ctx.upload(x), 1).numpy(), rv)  # value-only accumulator: same identity, NaN never taken


def test_reference_reduction_vectors(ctx, golden):
    up = lambda k: ctx.upload(np.array(golden[k]["arrays"][0], np.float32).reshape(2, 2))  # noqa: E731
    flat = lambda d: d.reshape(4)  # noqa: E731
    assert ctx.reduce("sum", flat(up("sum_all")), 0).numpy().item() == golden["sum_all"]["arrays"][1][0]
    assert ctx.reduce("sum", up("sum_axis0"), 0).numpy().tolist() == golden["sum_axis0"]["arrays"][1]
    assert ctx.reduce("mean", flat(up("mean_all")), 0).numpy().item() == golden["mean_all"]["arrays"][1][0]
    assert ctx.reduce("mean", up("mean_axis1"), 1).numpy().tolist() == golden["mean_axis1"]["arrays"][1]
    assert ctx.reduce("max", flat(up("max_all")), 0).numpy().item() == golden["max_all"]["arrays"][1][0]
    assert ctx.reduce("max", up("max_axis0"), 0).numpy().tolist() == golden["max_axis0"]["arrays"][1]


@pytest.mark.parametrize("dtype", DTYPES)
def test_softmax_axis(ctx, orc, golden, dtype):
    rng = np.random.default_rng(32)
    for shape, axis in (((256, 10), 1), ((4, 7, 5), 1), ((6, 9), 0)):
        x = (rng.standard_normal(shape) * 3).astype(dtype)
        got = ctx.softmax_axis(ctx.upload(x), axis).numpy()
        parity.check("softmax_axis", got, orc.softmax_axis(x.astype(np.float64), axis), oracle=orc.softmax_axis(x, axis), case=(shape, axis))
    for key, shape, axis in (("softmax_axis1", (2, 3), 1), ("softmax_axis0", (2, 2), 0)):
        x, y = (np.array(v, dtype) for v in golden[key]["arrays"])
        got = ctx.softmax_axis(ctx.upload(x.reshape(shape)), axis).numpy().ravel()
        np.testing.assert_allclose(got, y, atol=1e-3, rtol=0)


# ------------------------------------------------------------------------------------------ GEMM
GEMM_SHAPES = [(2, 2, 2), (1, 1, 1), (5, 7, 3), (64, 64, 64), (128, 128, 16), (130, 257, 75), (256, 256, 784), (256, 10, 128),
               (256, 10, 16384), (16384, 10, 256), (256, 16384, 10), (300, 200, 1000)]


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_all_transposes(ctx, orc, golden, dtype):
    rng = np.random.default_rng(40)
    for (M, N, K) in GEMM_SHAPES:
        a = rng.standard_normal((M, K)).astype(dtype)
        b = rng.standard_normal((K, N)).astype(dtype)
        truth = a.astype(np.float64) @ b.astype(np.float64)
        scale = (np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64)).max()
        for ta in (False, True):
            for tb in (False, True):
                da = ctx.upload(a.T if ta else a)
                db = ctx.upload(b.T if tb else b)
                got = ctx.gemm(da, db, ta, tb).numpy()
                parity.check("gemm", got, truth, case=(M, N, K, ta, tb), terms=scale)
    a, b, c = (np.array(v, dtype).reshape(2, 2) for v in golden["matmul"]["arrays"])
    assert np.array_equal(ctx.gemm(ctx.upload(a), ctx.upload(b)).numpy(), c)
    got = ctx.gemm(ctx.upload(rng.standard_normal((64, 64)).astype(dtype)), ctx.upload(np.eye(64, dtype=dtype))).numpy()
    assert got.shape == (64, 64)


# Products large enough for the LDS-slab f32 kernel on a 256-CU device (at least 384 tiles of 128 x 128, K % 64 == 0):
# exact tiles, ragged M and N (rows / columns past the matrix are re-read, never stored), N below one tile.
GEMM_LDS_SHAPES = [(2560, 2560, 128), (2500, 2436, 192), (4096, 3200, 64 * 3), (49152, 100, 128), (128 * 50, 1024 + 4, 256),
                   # too few 128-row tiles to fill the chip: 64 x 64 and 64 x 128 tiles (exact, ragged rows and columns, M below 128)
                   (1024, 1024, 1024), (1000, 1100, 192), (1280, 832, 128), (2048, 512, 256), (100, 16384, 128), (1988, 724, 320),
                   # K that is no multiple of the 64-deep stage (served for A . B^T with both operands k-contiguous; the other forms take
                   # the general tiles): a tail of 4, 40 and 60 values
                   (2560, 2560, 132), (2048, 1536, 1000), (1024, 1024, 252),
                   # about one 64-row tile per CU (ragged rows and columns too)
                   (1000, 1000, 384), (640, 1100, 512), (1024, 960, 256)]


def test_gemm_lds_kernel_shapes_all_transposes_and_bias(ctx):
    from ferrox_amd import capi
    rng = np.random.default_rng(41)
    for (M, N, K) in GEMM_LDS_SHAPES:
        a = rng.standard_normal((M, K)).astype(np.float32)
        b = rng.standard_normal((K, N)).astype(np.float32)
        truth = a.astype(np.float64) @ b.astype(np.float64)
        scale = (np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64)).max()
        bias = rng.standard_normal(N).astype(np.float32)
        dbias = ctx.upload(bias)
        for ta in (False, True):
            for tb in (False, True):
                da = ctx.upload(np.ascontiguousarray(a.T) if ta else a)
                db = ctx.upload(np.ascontiguousarray(b.T) if tb else b)
                got = ctx.gemm(da, db, ta, tb)
                parity.check("gemm lds", got.numpy(), truth, case=(M, N, K, ta, tb), terms=scale)
                # same bits run to run, and the bias (+ReLU) epilogue equals the two-call sequence
                assert np.array_equal(ctx.gemm(da, db, ta, tb).numpy(), got.numpy()), (M, N, K, ta, tb)
                fused = ctx.empty((M, N), np.float32)
                capi.check(capi.lib.fx_gemm_bias_act_f32(ctx.h, int(ta), int(tb), M, N, K, da.ptr, db.ptr, dbias.ptr, fused.ptr, 1))
                ctx.bias_act(got, dbias, M, N, 1, act=1)
                assert np.array_equal(fused.numpy(), got.numpy()), (M, N, K, ta, tb)


# products with one dimension of at most 16 (a classifier head and its two gradients, in the layouts the Linear layer
# produces): (kind, M, N, K) with kind naming the thin dimension -- n: A [M,K], B stored [N,K]; k: both plain; m: A
# stored [K,M].  They run as ragged MFMA tiles split along K, with the bias added after the ordered sum.
GEMM_THIN_SHAPES = [
    ("n", 256, 10, 16384), ("n", 37, 1, 1024), ("n", 130, 16, 2052), ("n", 2050, 7, 1536), ("n", 16, 13, 4096),
    ("k", 256, 16384, 10), ("k", 19, 1028, 1), ("k", 300, 4096, 16), ("k", 17, 2052, 7),
    ("m", 10, 16384, 256), ("m", 1, 1024, 16), ("m", 16, 1028, 1000), ("m", 7, 2052, 33), ("m", 13, 65536, 40),
    # wide enough for the one-launch thin kernel (f32): ragged N, odd K, K past one round of loads, all 32 rows
    ("m", 32, 9000, 100), ("m", 7, 8200, 131), ("m", 1, 8192, 33), ("m", 10, 8192, 1000),
]


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_with_one_thin_dimension(ctx, dtype):
    from ferrox_amd import capi
    rng = np.random.default_rng(43)
    sfx = "f32" if dtype == np.float32 else "f64"
    for (kind, M, N, K) in GEMM_THIN_SHAPES:
        ta, tb = kind == "m", kind == "n"
        a = rng.standard_normal((M, K)).astype(dtype)
        b = rng.standard_normal((K, N)).astype(dtype)
        truth = a.astype(np.float64) @ b.astype(np.float64)
        scale = (np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64)).max()
        da = ctx.upload(np.ascontiguousarray(a.T) if ta else a)
        db = ctx.upload(np.ascontiguousarray(b.T) if tb else b)
        got = ctx.gemm(da, db, ta, tb)
        parity.check("gemm thin", got.numpy(), truth, case=(kind, M, N, K), terms=scale)
        assert np.array_equal(ctx.gemm(da, db, ta, tb).numpy(), got.numpy()), (kind, M, N, K)
        bias = rng.standard_normal(N).astype(dtype)
        dbias = ctx.upload(bias)
        fused = ctx.empty((M, N), dtype)
        capi.check(getattr(capi.lib, "fx_gemm_bias_act_" + sfx)(ctx.h, int(ta), int(tb), M, N, K, da.ptr, db.ptr, dbias.ptr,
                                                                 fused.ptr, 1))
        ctx.bias_act(got, dbias, M, N, 1, act=1)
        assert np.array_equal(fused.numpy(), got.numpy()), (kind, M, N, K)


# small products take a one-launch kernel (32 x 32 tile per block, K split over the block's waves): every layout, ragged
# tile edges, K with half a group of eight left over, the longest K it takes, and K not a multiple of 4 for each layout (only the
# row/column-contiguous loads take that; the others fall back to the general tiles)
GEMM_SMALL_SHAPES = [(33, 65, 36), (256, 512, 784), (100, 31, 1024), (1, 1, 32), (64, 64, 44), (32, 96, 250), (70, 200, 127),
                     # short and odd reductions: a k-contiguous A read element by element (K = 10: a classifier head's data gradient)
                     (256, 128, 10), (40, 70, 1), (65, 33, 31), (256, 256, 45)]


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_small_products_all_layouts(ctx, dtype):
    from ferrox_amd import capi
    rng = np.random.default_rng(47)
    sfx = "f32" if dtype == np.float32 else "f64"
    for (M, N, K) in GEMM_SMALL_SHAPES:
        a = rng.standard_normal((M, K)).astype(dtype)
        b = rng.standard_normal((K, N)).astype(dtype)
        truth = a.astype(np.float64) @ b.astype(np.float64)
        scale = (np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64)).max()
        bias = rng.standard_normal(N).astype(dtype)
        dbias = ctx.upload(bias)
        for ta in (False, True):
            for tb in (False, True):
                da = ctx.upload(np.ascontiguousarray(a.T) if ta else a)
                db = ctx.upload(np.ascontiguousarray(b.T) if tb else b)
                got = ctx.gemm(da, db, ta, tb)
                case = (M, N, K, ta, tb)
                parity.check("gemm small", got.numpy(), truth, case=case, terms=scale)
                assert np.array_equal(ctx.gemm(da, db, ta, tb).numpy(), got.numpy()), case
                fused = ctx.empty((M, N), dtype)
                capi.check(getattr(capi.lib, "fx_gemm_bias_act_" + sfx)(ctx.h, int(ta), int(tb), M, N, K, da.ptr, db.ptr, dbias.ptr, fused.ptr, 1))
                ctx.bias_act(got, dbias, M, N, 1, act=1)
                assert np.array_equal(fused.numpy(), got.numpy()), case
    # an infinity in the last row of K must not leak into other outputs through the clamped re-reads past K
    M, N, K = 40, 40, 36
    a = rng.standard_normal((M, K)).astype(dtype)
    b = rng.standard_normal((K, N)).astype(dtype)
    b[K - 1, 3] = np.inf
    a[5, K - 1] = 0.0
    got = ctx.gemm(ctx.upload(np.ascontiguousarray(a.T)), ctx.upload(b), True, False).numpy()
    with np.errstate(invalid="ignore"):
        ref = a.astype(np.float64) @ b.astype(np.float64)
    assert np.isnan(got[5, 3]) and np.isnan(ref[5, 3])
    assert np.array_equal(np.isinf(got), np.isinf(ref)) and np.array_equal(np.isnan(got), np.isnan(ref))


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_tn_with_column_sums(ctx, dtype):
    """Linear's weight + bias gradient in one call: the product and the column sums of dY to rounding, the same bits run to run
    (one-launch small and thin products, a K that is split over blocks, the general tiles with the sums in a second launch)."""
    rng = np.random.default_rng(57)
    # K (batch), M (out), N (in)
    for (K, M, N) in [(256, 10, 128), (256, 10, 16384), (256, 128, 256), (256, 256, 784), (64, 3, 40), (100, 33, 70), (37, 5, 9),
                      (2048, 10, 64), (512, 600, 520), (256, 40, 16384)]:
        a = rng.standard_normal((K, M)).astype(dtype)
        b = rng.standard_normal((K, N)).astype(dtype)
        da, db = ctx.upload(a), ctx.upload(b)
        c, s = ctx.gemm_tn_colsum(da, db)
        scale = (np.abs(a.T).astype(np.float64) @ np.abs(b).astype(np.float64)).max()
        parity.check("gemm tn + colsum: product", c.numpy(), a.T.astype(np.float64) @ b.astype(np.float64), case=(K, M, N), terms=scale)
        parity.check("gemm tn + colsum: sums", s.numpy(), a.astype(np.longdouble).sum(axis=0), case=(K, M, N),
                     terms=np.abs(a).astype(np.float64).sum(axis=0).max())
        c2, s2 = ctx.gemm_tn_colsum(da, db)  # the same bits on a second run
        assert np.array_equal(c2.numpy(), c.numpy()) and np.array_equal(s2.numpy(), s.numpy()), (K, M, N)


@pytest.mark.parametrize("dtype", DTYPES)
def test_linear_backward_products_in_one_call(ctx, dtype):
    """fx_linear_bwd: dW and db with the bits of fx_gemm_tn_colsum, dX the product to rounding, whether the two products share a launch
    (both small) or one of them is a thin / large / split product and they run one after the other; with and without the bias gradient;
    the ReLU gradient of the layer below applied to dX bit for bit."""
    rng = np.random.default_rng(56)
    # B, in, out
    for (Bn, I, O) in [(256, 256, 128), (256, 784, 256), (256, 128, 10), (256, 16384, 10), (64, 40, 33), (37, 9, 50), (512, 512, 512),
                       (256, 64, 96), (2048, 100, 64), (256, 128, 7), (100, 60, 3)]:
        dy = rng.standard_normal((Bn, O)).astype(dtype)
        w = rng.standard_normal((O, I)).astype(dtype)
        x = rng.standard_normal((Bn, I)).astype(dtype)
        ddy, dw_, dx_ = ctx.upload(dy), ctx.upload(w), ctx.upload(x)
        gx, gw, gb = ctx.linear_bwd(ddy, dw_, dx_)
        # dX: the product (the separate call may run another tile shape, i.e. another summation order)
        scale = (np.abs(dy).astype(np.float64) @ np.abs(w).astype(np.float64)).max()
        parity.check("linear bwd dX", gx.numpy(), dy.astype(np.float64) @ w.astype(np.float64), case=(Bn, I, O), terms=scale)
        rw, rb = ctx.gemm_tn_colsum(ddy, dx_)
        assert np.array_equal(gw.numpy(), rw.numpy()) and np.array_equal(gb.numpy(), rb.numpy()), ("dW, db", Bn, I, O)
        gx2, gw2, _ = ctx.linear_bwd(ddy, dw_, dx_, want_db=False)
        assert np.array_equal(gx2.numpy(), gx.numpy()) and np.array_equal(gw2.numpy(), gw.numpy()), ("no db", Bn, I, O)
        # x as the output of a ReLU (zeros where it clipped): dX times the ReLU's mask, the bits of fx_relu_bwd on the product
        xr = np.maximum(x, 0)
        dxr = ctx.upload(xr)
        gx3, gw3, gb3 = ctx.linear_bwd(ddy, dw_, dxr, relu_below=True)
        assert np.array_equal(gx3.numpy(), ctx.relu_bwd(gx, dxr).numpy()), ("masked dX", Bn, I, O)
        rw3, rb3 = ctx.gemm_tn_colsum(ddy, dxr)
        assert np.array_equal(gw3.numpy(), rw3.numpy()) and np.array_equal(gb3.numpy(), rb3.numpy()), ("dW, db with relu below", Bn, I, O)


def test_gemm_shape_mismatch_message(ctx):
    from ferrox_amd.capi import FerroxHipError
    a = ctx.upload(np.zeros((2, 3), np.float32))
    b = ctx.upload(np.zeros((4, 5), np.float32))
    with pytest.raises(FerroxHipError, match=r"Matrix multiplication shape mismatch: \(2, 3\) @ \(4, 5\)"):
        ctx.gemm(a, b)


# ------------------------------------------------------------------------------------------ convolution
CONV_CASES = [  # B, Cin, H, W, Cout, k, s, p
    (1, 1, 5, 5, 1, 3, 1, 1), (1, 3, 5, 5, 4, 3, 1, 1), (2, 3, 8, 8, 4, 3, 1, 1), (3, 2, 9, 7, 5, 3, 2, 1), (2, 4, 6, 6, 3, 1, 1, 0),
    (32, 1, 28, 28, 8, 3, 1, 1), (8, 3, 32, 32, 32, 3, 1, 1), (8, 32, 32, 32, 64, 3, 2, 1), (2, 64, 56, 56, 128, 3, 1, 1),
    (2, 70, 13, 11, 130, 3, 1, 1), (2, 3, 7, 7, 2, 2, 2, 0),
]


@pytest.mark.parametrize("dtype", DTYPES)
def test_conv2d_fwd_dgrad_wgrad_vs_oracle(ctx, orc, dtype):
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(50)
    for (B, Cin, H, W, Cout, k, s, p) in CONV_CASES:
        x = rng.uniform(-1, 1, (B, Cin, H, W)).astype(dtype)
        w = (rng.standard_normal((Cout, Cin, k, k)) * np.sqrt(2.0 / (Cin * k * k))).astype(dtype)
        oh, ow = orc.out_hw(H, W, k, k, s, s, p, p)
        g = rng.standard_normal((B, Cout, oh, ow)).astype(dtype)
        dx_, dw_, dg_ = ctx.upload(x), ctx.upload(w), ctx.upload(g)
        y = ctx.conv2d_fwd(dx_, dw_, (s, s), (p, p)).numpy()
        dxg = ctx.conv2d_dgrad(dg_, dw_, x.shape, (s, s), (p, p), 0).numpy()
        dwg = ctx.conv2d_wgrad(dx_, dg_, w.shape, (s, s), (p, p), 0).numpy()
        # float64 ground truth from torch (the textbook routine) with |.|-scaled bounds
        tx = torch.from_numpy(x).double().requires_grad_(True)
        tw = torch.from_numpy(w).double().requires_grad_(True)
        ty = F.conv2d(tx, tw, stride=s, padding=p)
        ty.backward(torch.from_numpy(g).double())
        ay = F.conv2d(tx.detach().abs(), tw.detach().abs(), stride=s, padding=p).max().item()
        case = (B, Cin, H, W, Cout, k, s, p)
        # the GPU result and the CPU oracle's (restated reference algorithm) on the same inputs, each within the stated
        # tolerance of the float64 truth
        parity.check("conv fwd", y, ty.detach().numpy(), oracle=orc.conv2d_fwd(x, w, (s, s), (p, p)), case=case, terms=ay)
        parity.check("conv dgrad", dxg, tx.grad.numpy(), oracle=orc.conv2d_dgrad(g, w, x.shape, (s, s), (p, p), 0), case=case)
        parity.check("conv wgrad", dwg, tw.grad.numpy(), oracle=orc.conv2d_wgrad(x, g, w.shape, (s, s), (p, p), 0), case=case)
        # the CPU backend's literal gradients at every shape: truth = the oracle's literal arithmetic carried out in float64
        # (for f64 results the f64 oracle itself: two f64 summation orders differ by ~1e-15, far inside 1e-12)
        lit_dx = ctx.conv2d_dgrad(dg_, dw_, x.shape, (s, s), (p, p), 1).numpy()
        lit_dw = ctx.conv2d_wgrad(dx_, dg_, w.shape, (s, s), (p, p), 1).numpy()
        x64, w64, g64 = x.astype(np.float64), w.astype(np.float64), g.astype(np.float64)
        parity.check("conv dgrad literal", lit_dx, orc.conv2d_dgrad(g64, w64, x.shape, (s, s), (p, p), 1),
                     oracle=orc.conv2d_dgrad(g, w, x.shape, (s, s), (p, p), 1), case=case)
        parity.check("conv wgrad literal", lit_dw, orc.conv2d_wgrad(x64, g64, w.shape, (s, s), (p, p), 1),
                     oracle=orc.conv2d_wgrad(x, g, w.shape, (s, s), (p, p), 1), case=case)


# 3x3 weight gradients around the LDS-patch kernel (taken when Cin % 32 == 0, Cout > 32, W % 4 == 0, W <= 64, even
# output width; up to 64 output channels the waves also split the input channels (Cin % 64 == 0) or the pixel rows
# (output width % 4 == 0)): ragged Cout, one and two output rows per stage, strides, asymmetric padding, the widest
# row, and neighbours that fall back to the implicit GEMM (Cout <= 32, W % 4 != 0).  B, Cin, H, W, Cout, (sh, sw), (ph, pw)
WGRAD_PATCH_CASES = [
    (3, 32, 12, 10, 40, (1, 1), (1, 1)), (2, 64, 9, 14, 72, (1, 1), (0, 0)), (5, 32, 15, 18, 33, (1, 1), (1, 1)),
    (2, 32, 17, 16, 64, (2, 1), (1, 1)), (2, 96, 16, 16, 160, (2, 2), (1, 1)), (3, 32, 11, 12, 48, (1, 2), (2, 0)),
    (1, 32, 8, 6, 32, (1, 1), (1, 2)), (37, 32, 6, 8, 32, (1, 1), (1, 1)), (2, 32, 7, 62, 130, (3, 1), (1, 1)),
    (21, 32, 29, 56, 32, (1, 1), (1, 1)), (2, 32, 10, 56, 100, (1, 1), (1, 1)), (3, 64, 28, 28, 96, (1, 1), (1, 1)),
    (2, 32, 16, 16, 128, (1, 1), (1, 1)), (2, 32, 9, 64, 128, (1, 1), (0, 1)), (40, 64, 14, 14, 200, (1, 1), (1, 1)),
    (3, 32, 12, 20, 96, (1, 2), (2, 0)), (2, 32, 8, 24, 65, (2, 2), (0, 0)),
    (2, 64, 12, 56, 64, (1, 1), (1, 1)), (3, 64, 10, 32, 64, (1, 1), (1, 1)), (4, 128, 8, 16, 48, (1, 1), (1, 1)),
    (2, 32, 12, 32, 64, (1, 1), (1, 1)), (2, 32, 16, 32, 64, (2, 2), (1, 1)), (3, 64, 9, 24, 40, (1, 2), (1, 1)),
    (5, 32, 6, 64, 33, (1, 1), (1, 1)), (2, 96, 8, 8, 64, (1, 1), (1, 1)), (2, 64, 7, 12, 56, (1, 1), (0, 0)),
    # ragged output-channel counts in the last image: the 16-row staging passes past the last channel must not be read
    (1, 32, 6, 24, 40, (1, 1), (1, 1)), (2, 64, 6, 28, 49, (1, 1), (1, 1)), (1, 32, 4, 32, 97, (1, 1), (1, 1)),
    (3, 32, 8, 12, 72, (1, 1), (1, 1)), (2, 32, 8, 16, 150, (1, 1), (1, 1)), (1, 64, 5, 56, 36, (1, 1), (1, 1)),
    # at most 32 output channels: wave layouts 1 x 2 x 2 and 1 x 1 x 4, ragged counts
    (2, 64, 8, 32, 32, (1, 1), (1, 1)), (3, 32, 8, 32, 32, (1, 1), (1, 1)), (2, 64, 6, 28, 20, (1, 1), (1, 1)), (2, 32, 10, 24, 7, (1, 1), (1, 1)),
    (2, 96, 12, 16, 17, (1, 1), (1, 1)), (33, 32, 16, 16, 32, (1, 1), (1, 1)), (2, 128, 16, 16, 32, (1, 1), (1, 1)),
    (3, 128, 16, 16, 64, (1, 1), (1, 1)),
    # input channels that do not fill the last block of 32 (their LDS planes stay zero)
    (2, 16, 8, 32, 32, (1, 1), (1, 1)), (3, 48, 8, 32, 30, (1, 1), (1, 1)), (2, 24, 12, 24, 20, (1, 1), (1, 1)), (2, 40, 6, 16, 13, (1, 1), (1, 1)),
    (1, 33, 8, 24, 16, (1, 1), (1, 1)), (2, 17, 6, 32, 32, (1, 1), (1, 1)), (3, 48, 8, 32, 64, (1, 1), (1, 1)),
    # 64-wide rows with 64 x 64 channels (the 64-plane layout exceeds the LDS budget)
    (2, 64, 8, 64, 64, (1, 1), (1, 1)), (2, 64, 8, 64, 32, (1, 1), (1, 1)),
    # stride 2, padding 1 over maps 32 and 64 wide: the double-buffered stride-2 kernel in its three wave layouts, a top row
    # without padding, an odd height (the last patch row is below the image), many splits
    (3, 32, 32, 32, 64, (2, 2), (1, 1)), (2, 64, 8, 32, 128, (2, 2), (1, 1)), (5, 32, 16, 32, 32, (2, 2), (1, 1)), (2, 32, 8, 64, 64, (2, 2), (1, 1)),
    (2, 64, 4, 64, 128, (2, 2), (1, 1)), (3, 32, 12, 64, 96, (2, 2), (1, 1)), (2, 32, 9, 32, 64, (2, 2), (0, 1)), (2, 32, 15, 32, 64, (2, 2), (1, 1)),
    (40, 32, 8, 32, 64, (2, 2), (1, 1)),
    # the same kernel over maps 56 wide (rows of 28 pixels: two and one row segments) and 16 wide (a whole 8 x 8 output per stage:
    # one, two and four row segments) and 28 wide (two of 14 output rows per stage, 128 output channels per block), a top row without
    # padding, an odd height, many splits
    (2, 32, 56, 56, 64, (2, 2), (1, 1)), (2, 64, 8, 56, 128, (2, 2), (1, 1)), (3, 32, 12, 56, 192, (2, 2), (1, 1)), (2, 32, 9, 56, 64, (2, 2), (0, 1)),
    (3, 32, 16, 16, 32, (2, 2), (1, 1)), (5, 64, 16, 16, 64, (2, 2), (1, 1)), (2, 32, 16, 16, 128, (2, 2), (1, 1)), (2, 32, 15, 16, 64, (2, 2), (1, 1)),
    (2, 32, 17, 16, 96, (2, 2), (0, 1)), (70, 32, 16, 16, 64, (2, 2), (1, 1)), (33, 32, 4, 56, 128, (2, 2), (1, 1)),
    (3, 32, 28, 28, 128, (2, 2), (1, 1)), (2, 64, 12, 28, 256, (2, 2), (1, 1)), (2, 32, 27, 28, 128, (2, 2), (1, 1)),
    # narrow maps: one whole image per stage, (channel, row) pair staging
    (3, 64, 8, 8, 128, (1, 1), (1, 1)), (2, 32, 8, 8, 64, (1, 1), (1, 1)), (2, 96, 8, 8, 20, (1, 1), (1, 1)), (2, 32, 6, 8, 100, (1, 1), (1, 1)),
    (3, 64, 4, 16, 72, (1, 1), (1, 1)), (2, 48, 8, 8, 24, (1, 1), (1, 1)), (70, 128, 8, 8, 128, (1, 1), (1, 1)),
    # strided layers (implicit GEMM)
    (3, 32, 32, 32, 64, (2, 2), (1, 1)), (2, 64, 56, 56, 128, (2, 2), (1, 1)), (2, 32, 16, 24, 70, (2, 1), (1, 1)),
    (2, 32, 13, 32, 48, (2, 2), (0, 1)),
    # rows of more than 64 floats, walked in segments of 24 to 56 pixels with halo columns from the neighbouring segments: every
    # wave layout, unrolled and plain pixel loops, two to seven segments per row, ragged channel counts, a row stride
    (2, 32, 6, 112, 128, (1, 1), (1, 1)), (1, 64, 5, 128, 64, (1, 1), (1, 1)), (1, 32, 4, 224, 40, (1, 1), (1, 1)),
    (2, 64, 3, 96, 32, (1, 1), (1, 1)), (1, 32, 4, 80, 20, (1, 1), (1, 1)), (1, 32, 3, 72, 130, (1, 1), (1, 1)),
    (1, 16, 4, 112, 32, (1, 1), (1, 1)), (1, 64, 7, 128, 200, (2, 1), (1, 1)), (1, 128, 2, 256, 64, (1, 1), (1, 1)),
]


def test_conv2d_wgrad_patch_kernel_shapes(ctx, orc):
    import torch
    from ferrox_amd import capi
    import torch.nn.functional as F
    rng = np.random.default_rng(57)
    for (B, Cin, H, W, Cout, st, pd) in WGRAD_PATCH_CASES:
        x = rng.uniform(-1, 1, (B, Cin, H, W)).astype(np.float32)
        oh, ow = orc.out_hw(H, W, 3, 3, st[0], st[1], pd[0], pd[1])
        g = rng.standard_normal((B, Cout, oh, ow)).astype(np.float32)
        dx_, dg_ = ctx.upload(x), ctx.upload(g)
        dw = ctx.conv2d_wgrad(dx_, dg_, (Cout, Cin, 3, 3), st, pd, 0).numpy()
        tw = torch.zeros((Cout, Cin, 3, 3), dtype=torch.float64, requires_grad=True)
        F.conv2d(torch.from_numpy(x).double(), tw, stride=st, padding=pd).backward(torch.from_numpy(g).double())
        case = (B, Cin, H, W, Cout, st, pd)
        parity.check("wgrad patch kernels", dw, tw.grad.numpy(), oracle=orc.conv2d_wgrad(x, g, (Cout, Cin, 3, 3), st, pd, 0), case=case)
        # same bits on a second run and with a caller-provided workspace of exactly the advertised size
        assert np.array_equal(dw, ctx.conv2d_wgrad(dx_, dg_, (Cout, Cin, 3, 3), st, pd, 0).numpy()), case
        need = capi.lib.fx_conv2d_workspace_bytes(capi.CONV_WGRAD, capi.FX_F32, 0, B, Cin, H, W, Cout, 3, 3, st[0], st[1], pd[0], pd[1])
        assert need >= 0
        ws = ctx.empty((max(need, 4) // 4,), np.float32)
        out = ctx.empty((Cout, Cin, 3, 3), np.float32)
        capi.check(capi.lib.fx_conv2d_wgrad_f32(ctx.h, dx_.ptr, dg_.ptr, out.ptr, B, Cin, H, W, Cout, 3, 3, st[0], st[1],
                                                pd[0], pd[1], 0, ws.ptr, need))
        assert np.array_equal(dw, out.numpy()), case
        if need > 0:
            assert capi.lib.fx_conv2d_wgrad_f32(ctx.h, dx_.ptr, dg_.ptr, out.ptr, B, Cin, H, W, Cout, 3, 3, st[0], st[1],
                                                pd[0], pd[1], 0, ws.ptr, need - 4) != 0


# 3x3 forward / stride-1 data-gradient shapes that take the LDS-patch kernel (channels % 8 == 0, W % 4 == 0,
# W <= 64): 64- and 128-row tiles, ragged channel counts, ragged last pixel tile, paddings 0..2 (the data gradient
# then runs with padding 2..0), a strided forward, the widest supported row.  B, Cin, H, W, Cout, (sh, sw), (ph, pw)
CONV_PATCH_CASES = [
    (2, 8, 6, 12, 16, (1, 1), (1, 1)), (3, 16, 8, 36, 100, (1, 1), (0, 0)), (2, 24, 4, 8, 136, (1, 1), (2, 2)),
    (2, 64, 28, 28, 64, (1, 1), (1, 1)), (1, 8, 64, 64, 32, (1, 1), (1, 1)), (2, 16, 6, 16, 40, (2, 2), (1, 1)),
    (2, 8, 5, 12, 24, (1, 1), (0, 1)), (5, 72, 6, 40, 200, (1, 1), (1, 1)), (2, 128, 6, 8, 72, (1, 1), (1, 0)),
    (2, 8, 12, 12, 16, (1, 1), (1, 1)),
    # ragged output-channel counts, one per tile shape
    # of the forward kernel on a 256-CU device: 2x2, 2x3, 2x4, 4x4, 4x5, 4x6, 4x7, 4x8
    (2, 8, 6, 12, 60, (1, 1), (1, 1)), (3, 16, 8, 36, 120, (1, 1), (0, 0)), (2, 24, 6, 8, 104, (1, 1), (2, 2)),
    (1, 8, 64, 64, 52, (1, 1), (1, 1)), (2, 16, 15, 18, 60, (2, 2), (1, 1)), (2, 128, 6, 8, 120, (1, 1), (1, 0)),
    (2, 8, 9, 64, 128, (2, 1), (1, 1)), (128, 8, 8, 40, 120, (1, 1), (1, 1)), (32, 8, 56, 56, 64, (1, 1), (1, 1)),
    (16, 8, 56, 56, 120, (1, 1), (1, 1)), (128, 8, 8, 40, 250, (1, 1), (1, 1)), (96, 8, 12, 48, 384, (1, 1), (1, 1)),
    (32, 8, 56, 56, 120, (1, 1), (1, 1)), (128, 8, 16, 64, 120, (1, 1), (1, 1)),
    # strided layers: up to 20 patch rows under a tile
    (8, 32, 32, 32, 64, (2, 2), (1, 1)), (4, 64, 56, 56, 128, (2, 2), (1, 1)), (2, 16, 30, 40, 60, (2, 1), (1, 1)),
    (2, 8, 16, 34, 128, (3, 3), (1, 1)), (64, 16, 28, 28, 128, (2, 2), (1, 1)),
    # 21 to 40 patch rows of at most 32 floats (four rows per staging pass): stride 2 over 28- and 14-wide maps (one tile of two
    # images at 14 x 14, odd batch), no padding, a row length that is no multiple of four floats, 64- and 128-row tiles; stacked
    # images of 5 x 5 and 6 x 6 maps at stride 1 (4 x 4 maps stay on the implicit GEMM)
    (4, 16, 28, 28, 128, (2, 2), (1, 1)), (3, 8, 28, 28, 64, (2, 2), (1, 1)), (5, 16, 14, 14, 128, (2, 2), (1, 1)), (6, 8, 14, 14, 64, (2, 2), (1, 1)),
    (2, 8, 30, 30, 40, (2, 2), (0, 0)), (2, 8, 27, 31, 64, (2, 2), (1, 1)), (9, 16, 5, 5, 64, (1, 1), (1, 1)), (13, 8, 4, 4, 128, (1, 1), (1, 1)),
    (3, 8, 20, 24, 200, (3, 2), (1, 1)),
    # 32 channels out (forward) or in (data gradient): one block of channels, four waves along the pixels (1x2, 1x3, 1x4)
    (64, 64, 32, 32, 32, (1, 1), (1, 1)), (3, 16, 9, 20, 30, (1, 1), (1, 1)), (64, 8, 16, 32, 32, (2, 1), (1, 1)),
    (2, 8, 18, 10, 27, (1, 1), (0, 0)), (64, 32, 32, 32, 64, (1, 1), (1, 1)), (40, 32, 16, 16, 24, (1, 1), (1, 1)),
    # up to half of a tile's channel rows are padding
    (3, 16, 8, 32, 16, (1, 1), (1, 1)), (2, 8, 12, 28, 40, (1, 1), (1, 1)), (16, 8, 56, 56, 72, (1, 1), (1, 1)), (3, 24, 12, 12, 17, (1, 1), (1, 1)),
    (4, 48, 16, 16, 64, (1, 1), (1, 1)),
    # row lengths that are not multiples of four floats (the last vector of a row is moved back to end with the row)
    (3, 8, 14, 14, 64, (1, 1), (1, 1)), (2, 16, 10, 7, 32, (1, 1), (1, 1)), (2, 8, 9, 30, 128, (1, 1), (0, 0)), (2, 8, 15, 18, 40, (2, 2), (1, 1)),
    (2, 8, 6, 63, 64, (1, 1), (1, 1)), (64, 64, 14, 14, 128, (1, 1), (1, 1)),
    # maps of at most 64 pixels: whole images stacked in one tile (odd batches: the last tile holds one image)
    (5, 16, 8, 8, 128, (1, 1), (1, 1)), (3, 8, 7, 7, 64, (1, 1), (1, 1)), (7, 8, 6, 6, 40, (1, 1), (1, 1)), (4, 8, 6, 10, 200, (1, 1), (0, 1)),
    (33, 64, 8, 8, 64, (1, 1), (1, 1)), (9, 16, 8, 8, 100, (1, 1), (0, 0)),
    # stride 2 over maps 32 and 64 wide (fwd_patch_s2.hpp): 32 or 64 output channels per block, one to five chunks of 8 input
    # channels, one to four tiles of 256 pixels per image
    (2, 8, 32, 32, 32, (2, 2), (1, 1)), (2, 16, 64, 64, 64, (2, 2), (1, 1)), (2, 24, 16, 64, 32, (2, 2), (1, 1)),
    (3, 40, 64, 32, 32, (2, 2), (1, 1)), (5, 8, 32, 32, 64, (2, 2), (1, 1)), (1, 8, 128, 64, 32, (2, 2), (1, 1)),
    # rows of 65 to 128 floats (one patch row per staging pass): tiles 4x4, 2x4, 2x3, ragged channels and pixels, a row length that
    # is not a multiple of four floats, no padding, two row strides
    (2, 8, 10, 112, 128, (1, 1), (1, 1)), (1, 16, 6, 128, 64, (1, 1), (1, 1)), (2, 8, 7, 100, 40, (1, 1), (1, 1)), (1, 8, 9, 127, 72, (1, 1), (0, 0)),
    (2, 24, 5, 66, 200, (1, 1), (1, 1)), (1, 8, 12, 96, 64, (2, 1), (1, 1)), (3, 8, 4, 128, 120, (1, 1), (1, 2)), (1, 16, 33, 80, 32, (1, 1), (1, 1)),
    # rows of 129 to 256 floats (two staging passes per patch row)
    (1, 8, 5, 224, 64, (1, 1), (1, 1)), (1, 16, 4, 256, 128, (1, 1), (1, 1)), (2, 8, 6, 160, 40, (1, 1), (1, 1)), (1, 8, 7, 130, 72, (1, 1), (0, 0)),
    (1, 24, 3, 255, 200, (1, 1), (1, 1)),
]


def test_conv2d_patch_kernel_shapes(ctx, orc):
    import torch
    import torch.nn.functional as F
    from ferrox_amd import capi
    rng = np.random.default_rng(58)
    for (B, Cin, H, W, Cout, st, pd) in CONV_PATCH_CASES:
        case = (B, Cin, H, W, Cout, st, pd)
        x = rng.uniform(-1, 1, (B, Cin, H, W)).astype(np.float32)
        w = (rng.standard_normal((Cout, Cin, 3, 3)) * np.sqrt(2.0 / (Cin * 9))).astype(np.float32)
        oh, ow = orc.out_hw(H, W, 3, 3, st[0], st[1], pd[0], pd[1])
        g = rng.standard_normal((B, Cout, oh, ow)).astype(np.float32)
        dx_, dw_, dg_ = ctx.upload(x), ctx.upload(w), ctx.upload(g)
        y = ctx.conv2d_fwd(dx_, dw_, st, pd).numpy()
        dxg = ctx.conv2d_dgrad(dg_, dw_, x.shape, st, pd, 0).numpy()
        tx = torch.from_numpy(x).double().requires_grad_(True)
        tw = torch.from_numpy(w).double()
        ty = F.conv2d(tx, tw, stride=st, padding=pd)
        ty.backward(torch.from_numpy(g).double())
        ay = F.conv2d(tx.detach().abs(), tw.abs(), stride=st, padding=pd).max().item()
        parity.check("patch kernels fwd", y, ty.detach().numpy(), oracle=orc.conv2d_fwd(x, w, st, pd), case=case, terms=ay)
        parity.check("patch kernels dgrad", dxg, tx.grad.numpy(), oracle=orc.conv2d_dgrad(g, w, x.shape, st, pd, 0), case=case)
        dims = (B, Cin, H, W, Cout, 3, 3, st[0], st[1], pd[0], pd[1])
        # bias + ReLU in the store of the kernel = the forward pass followed by fx_bias_act, bit for bit
        db_ = ctx.upload(rng.standard_normal(Cout).astype(np.float32))
        fused = ctx.empty(y.shape, np.float32)
        capi.check(capi.lib.fx_conv2d_fwd_bias_act_f32(ctx.h, dx_.ptr, dw_.ptr, db_.ptr, fused.ptr, *dims, 1, None, 0))
        two = ctx.conv2d_fwd(dx_, dw_, st, pd)
        ctx.bias_act(two, db_, B, Cout, oh * ow, act=1)
        assert np.array_equal(fused.numpy(), two.numpy()), ("bias+relu", case)
        # caller-provided workspaces of exactly the advertised size give the same bits
        for kind, fn, a, b_, ref, shape in (
                (capi.CONV_FWD, capi.lib.fx_conv2d_fwd_f32, dx_, dw_, y, y.shape),
                (capi.CONV_DGRAD, capi.lib.fx_conv2d_dgrad_f32, dg_, dw_, dxg, x.shape)):
            need = capi.lib.fx_conv2d_workspace_bytes(kind, capi.FX_F32, 0, *dims)
            assert need >= 0, case
            ws = ctx.empty((max(need, 4) // 4,), np.float32)
            out = ctx.empty(shape, np.float32)
            extra = () if kind == capi.CONV_FWD else (0,)
            capi.check(fn(ctx.h, a.ptr, b_.ptr, out.ptr, *dims, *extra, ws.ptr, need))
            assert np.array_equal(out.numpy(), ref), (kind, case)


# f64 on the 16x16x4 MFMA patch kernel (conv_patch_f64.hpp: 3x3, channels % 8 == 0, even rows of up to 64 doubles, at most 8 patch
# rows under a tile, at least 32 output channels and 64 pixels): every tile width, two channel tiles, ragged channel counts,
# tiles that end inside a row, paddings 0 / 1 / 2, a strided forward pass, bias + ReLU in the store.
CONV_F64_PATCH_CASES = [  # B, Cin, H, W, Cout, (sh, sw), (ph, pw)
    (2, 64, 56, 56, 128, (1, 1), (1, 1)), (3, 8, 6, 12, 60, (1, 1), (1, 1)), (3, 16, 8, 36, 120, (1, 1), (0, 0)), (2, 24, 10, 16, 104, (1, 1), (2, 2)),
    (1, 8, 64, 64, 52, (1, 1), (1, 1)), (2, 16, 9, 62, 64, (2, 1), (1, 1)), (5, 32, 32, 32, 64, (1, 1), (1, 1)), (3, 8, 14, 28, 72, (1, 1), (1, 1)),
    (2, 8, 9, 30, 128, (1, 1), (0, 0)), (2, 32, 28, 28, 33, (1, 1), (1, 1)),
    # stride 2 over maps 32 and 64 wide (fwd_patch_s2_f64.hpp; the data gradient runs dgrad_patch_s2_f64.hpp where Cin % 32 == 0): 32 and
    # 64 output channels per block, one to eight chunks of 4 input channels, one to four tiles per image
    (3, 32, 32, 32, 64, (2, 2), (1, 1)), (2, 4, 32, 32, 32, (2, 2), (1, 1)), (2, 16, 64, 64, 64, (2, 2), (1, 1)), (2, 12, 16, 64, 32, (2, 2), (1, 1)),
    (1, 8, 128, 64, 64, (2, 2), (1, 1)),
]


def test_conv2d_f64_patch_kernel_shapes(ctx, orc):
    import torch
    import torch.nn.functional as F
    from ferrox_amd import capi
    rng = np.random.default_rng(61)
    for (B, Cin, H, W, Cout, st, pd) in CONV_F64_PATCH_CASES:
        case = (B, Cin, H, W, Cout, st, pd)
        x = rng.uniform(-1, 1, (B, Cin, H, W))
        w = rng.standard_normal((Cout, Cin, 3, 3)) * np.sqrt(2.0 / (Cin * 9))
        bias = rng.standard_normal(Cout)
        oh, ow = orc.out_hw(H, W, 3, 3, st[0], st[1], pd[0], pd[1])
        g = rng.standard_normal((B, Cout, oh, ow))
        dx_, dw_, dg_, db_ = ctx.upload(x), ctx.upload(w), ctx.upload(g), ctx.upload(bias)
        y = ctx.conv2d_fwd(dx_, dw_, st, pd).numpy()
        dxg = ctx.conv2d_dgrad(dg_, dw_, x.shape, st, pd, 0).numpy()
        tx = torch.from_numpy(x).to(torch.float64).requires_grad_(True)
        tw = torch.from_numpy(w).to(torch.float64)
        ty = F.conv2d(tx, tw, stride=st, padding=pd)
        ty.backward(torch.from_numpy(g))
        ay = F.conv2d(tx.detach().abs(), tw.abs(), stride=st, padding=pd).max().item()
        parity.check("patch kernels fwd", y, ty.detach().numpy(), oracle=orc.conv2d_fwd(x, w, st, pd), case=case, terms=ay)
        parity.check("patch kernels dgrad", dxg, tx.grad.numpy(), oracle=orc.conv2d_dgrad(g, w, x.shape, st, pd, 0), case=case)
        # bias + ReLU in the store of the kernel = the forward pass followed by fx_bias_act, bit for bit
        dims = (B, Cin, H, W, Cout, 3, 3, st[0], st[1], pd[0], pd[1])
        fused = ctx.empty(y.shape, np.float64)
        capi.check(capi.lib.fx_conv2d_fwd_bias_act_f64(ctx.h, dx_.ptr, dw_.ptr, db_.ptr, fused.ptr, *dims, 1, None, 0))
        two = ctx.conv2d_fwd(dx_, dw_, st, pd)
        capi.check(capi.lib.fx_bias_act_f64(ctx.h, two.ptr, db_.ptr, B, Cout, oh * ow, 1))
        assert np.array_equal(fused.numpy(), two.numpy()), ("bias + relu", case)
        # caller-provided workspaces of exactly the advertised size give the same bits
        for kind, fn, a, b_, ref, shape in (
                (capi.CONV_FWD, capi.lib.fx_conv2d_fwd_f64, dx_, dw_, y, y.shape),
                (capi.CONV_DGRAD, capi.lib.fx_conv2d_dgrad_f64, dg_, dw_, dxg, x.shape)):
            need = capi.lib.fx_conv2d_workspace_bytes(kind, capi.FX_F64, 0, *dims)
            assert need >= 0, case
            ws = ctx.empty((max(need, 8) // 8,), np.float64)
            out = ctx.empty(shape, np.float64)
            extra = () if kind == capi.CONV_FWD else (0,)
            capi.check(fn(ctx.h, a.ptr, b_.ptr, out.ptr, *dims, *extra, ws.ptr, need))
            assert np.array_equal(out.numpy(), ref), (kind, case)


# f64 weight gradient on the 16x16x4 MFMA patch kernel (wgrad_patch_f64.hpp: 3x3, unit column stride, rows of 24 / 32 / 56 / 64
# pixels, Cin % 16 == 0, Cout % 64 == 0): every row length, several channel tiles, paddings 0 / 1 / 2, a row stride of 2, a batch
# that does not fill the splits evenly.
CONV_F64_WGRAD_CASES = [  # B, Cin, H, W, Cout, sh, (ph, pw)
    (2, 64, 56, 56, 128, 1, (1, 1)), (3, 16, 32, 32, 64, 1, (1, 1)), (2, 32, 26, 26, 64, 1, (0, 0)), (2, 16, 24, 62, 128, 1, (2, 2)),
    (2, 48, 47, 24, 64, 2, (1, 1)), (5, 16, 8, 64, 64, 1, (1, 1)), (37, 16, 9, 32, 64, 1, (1, 1)),
    # stride 2 in both directions over maps 32 and 64 wide (wgrad_patch_s2_f64.hpp): one and several tiles, an odd height, a top
    # row without padding, stage ranges that do not divide evenly
    (3, 32, 32, 32, 64, (2, 2), (1, 1)), (2, 64, 16, 64, 128, (2, 2), (1, 1)), (5, 32, 31, 32, 64, (2, 2), (1, 1)),
    (2, 32, 33, 32, 64, (2, 2), (0, 1)), (70, 32, 32, 32, 64, (2, 2), (1, 1)), (3, 64, 6, 64, 192, (2, 2), (1, 1)),
    # ... and 16 wide (half of an 8 x 8 output per stage)
    (3, 32, 16, 16, 64, (2, 2), (1, 1)), (2, 64, 16, 16, 128, (2, 2), (1, 1)), (5, 32, 15, 16, 64, (2, 2), (1, 1)), (2, 32, 17, 16, 64, (2, 2), (0, 1)),
    (70, 32, 8, 16, 64, (2, 2), (1, 1)),
]


def test_conv2d_f64_wgrad_patch_kernel_shapes(ctx, orc):
    import torch
    import torch.nn.functional as F
    from ferrox_amd import capi
    rng = np.random.default_rng(62)
    for (B, Cin, H, W, Cout, sh, pd) in CONV_F64_WGRAD_CASES:
        case = (B, Cin, H, W, Cout, sh, pd)
        st = sh if isinstance(sh, tuple) else (sh, 1)
        x = rng.uniform(-1, 1, (B, Cin, H, W))
        oh, ow = orc.out_hw(H, W, 3, 3, st[0], st[1], pd[0], pd[1])
        g = rng.standard_normal((B, Cout, oh, ow))
        dx_, dg_ = ctx.upload(x), ctx.upload(g)
        dwg = ctx.conv2d_wgrad(dx_, dg_, (Cout, Cin, 3, 3), st, pd, 0).numpy()
        tw = torch.zeros((Cout, Cin, 3, 3), dtype=torch.float64, requires_grad=True)
        F.conv2d(torch.from_numpy(x), tw, stride=st, padding=pd).backward(torch.from_numpy(g))
        orc_dw = orc.conv2d_wgrad(x, g, (Cout, Cin, 3, 3), st, pd, 0) if B * Cout * oh * ow <= 1 << 20 else None
        parity.check("wgrad patch kernels f64", dwg, tw.grad.numpy(), oracle=orc_dw, case=case)
        # a caller-provided workspace of exactly the advertised size gives the same bits
        dims = (B, Cin, H, W, Cout, 3, 3, st[0], st[1], pd[0], pd[1])
        need = capi.lib.fx_conv2d_workspace_bytes(capi.CONV_WGRAD, capi.FX_F64, 0, *dims)
        ws = ctx.empty((max(need, 8) // 8,), np.float64)
        out = ctx.empty((Cout, Cin, 3, 3), np.float64)
        capi.check(capi.lib.fx_conv2d_wgrad_f64(ctx.h, dx_.ptr, dg_.ptr, out.ptr, *dims, 0, ws.ptr, need))
        assert np.array_equal(out.numpy(), dwg), case


# Image layers (at most 4 input channels forward, 3 for the weight gradient; W % 4 == 0): the LDS-patch kernels for
# few channels.  Ragged Cout, tiles that end inside a row, strides, wide rows, padding 0 and 2, one-channel MNIST shape.
SMALLC_CASES = [  # B, Cin, H, W, Cout, (sh, sw), (ph, pw)
    (4, 3, 32, 32, 32, (1, 1), (1, 1)), (5, 1, 28, 28, 8, (1, 1), (1, 1)), (3, 3, 10, 12, 40, (1, 1), (0, 0)),
    (2, 2, 17, 20, 33, (2, 2), (1, 1)), (2, 3, 7, 8, 5, (3, 1), (1, 1)), (1, 3, 40, 36, 64, (1, 1), (1, 1)),
    (1, 3, 66, 64, 16, (2, 2), (1, 1)), (2, 1, 5, 4, 70, (1, 1), (2, 2)), (1, 3, 19, 60, 8, (1, 1), (1, 1)),
    (1, 3, 20, 224, 16, (2, 2), (1, 1)), (1, 4, 10, 64, 16, (1, 2), (2, 0)), (3, 3, 9, 12, 40, (1, 1), (0, 0)), (37, 3, 16, 16, 32, (1, 1), (1, 1)),
    # row lengths that are not multiples of four floats
    (2, 3, 14, 14, 32, (1, 1), (1, 1)), (2, 1, 9, 7, 16, (1, 1), (1, 1)), (2, 3, 12, 30, 8, (1, 1), (1, 1)), (3, 1, 8, 5, 8, (1, 1), (1, 1)),
    # rows of 128 floats (two per tile): the reference's own benchmark layer (kernels/benchmark.cu:856-860) and neighbours
    (1, 3, 128, 128, 32, (1, 1), (1, 1)), (2, 1, 6, 128, 40, (1, 1), (1, 1)), (1, 2, 7, 256, 8, (2, 2), (1, 1)), (2, 3, 5, 128, 16, (1, 1), (0, 0)),
    # row-band weight gradient: bands of 4 and 8 rows that do not divide the height, two blocks of 32 pixels per row, ragged Cout
    (130, 2, 33, 32, 40, (1, 1), (1, 1)), (300, 1, 30, 32, 32, (1, 1), (1, 1)), (70, 3, 30, 64, 8, (1, 1), (1, 1)),
]


def test_conv2d_image_layer_kernels(ctx, orc):
    import torch
    import torch.nn.functional as F
    from ferrox_amd import capi
    rng = np.random.default_rng(59)
    for (B, Cin, H, W, Cout, st, pd) in SMALLC_CASES:
        case = (B, Cin, H, W, Cout, st, pd)
        x = rng.uniform(-1, 1, (B, Cin, H, W)).astype(np.float32)
        w = (rng.standard_normal((Cout, Cin, 3, 3)) * np.sqrt(2.0 / (Cin * 9))).astype(np.float32)
        bias = rng.standard_normal(Cout).astype(np.float32)
        oh, ow = orc.out_hw(H, W, 3, 3, st[0], st[1], pd[0], pd[1])
        g = rng.standard_normal((B, Cout, oh, ow)).astype(np.float32)
        dx_, dw_, dg_, db_ = ctx.upload(x), ctx.upload(w), ctx.upload(g), ctx.upload(bias)
        y = ctx.conv2d_fwd(dx_, dw_, st, pd).numpy()
        gw = ctx.conv2d_wgrad(dx_, dg_, w.shape, st, pd, 0).numpy()
        gx = ctx.conv2d_dgrad(dg_, dw_, x.shape, st, pd, 0).numpy()
        tx = torch.from_numpy(x).double().requires_grad_(True)
        tw = torch.from_numpy(w).double().requires_grad_(True)
        ty = F.conv2d(tx, tw, stride=st, padding=pd)
        ty.backward(torch.from_numpy(g).double())
        ay = F.conv2d(tx.detach().abs(), tw.detach().abs(), stride=st, padding=pd).max().item()
        parity.check("image layers fwd", y, ty.detach().numpy(), oracle=orc.conv2d_fwd(x, w, st, pd), case=case, terms=ay)
        parity.check("image layers wgrad", gw, tw.grad.numpy(), oracle=orc.conv2d_wgrad(x, g, w.shape, st, pd, 0), case=case)
        # the data gradient of a layer of few input channels (a gather per input pixel, four pixels per thread at unit stride)
        parity.check("image layers dgrad", gx, tx.grad.numpy(), oracle=orc.conv2d_dgrad(g, w, x.shape, st, pd, 0), case=case)
        assert np.array_equal(ctx.conv2d_dgrad(dg_, dw_, x.shape, st, pd, 0).numpy(), gx), case
        # same bits on a second run; bias + ReLU in the store equals the separate pass
        assert np.array_equal(ctx.conv2d_fwd(dx_, dw_, st, pd).numpy(), y), case
        assert np.array_equal(ctx.conv2d_wgrad(dx_, dg_, w.shape, st, pd, 0).numpy(), gw), case
        dims = (B, Cin, H, W, Cout, 3, 3, st[0], st[1], pd[0], pd[1])
        fused = ctx.empty(y.shape, np.float32)
        capi.check(capi.lib.fx_conv2d_fwd_bias_act_f32(ctx.h, dx_.ptr, dw_.ptr, db_.ptr, fused.ptr, *dims, 1, None, 0))
        two = ctx.conv2d_fwd(dx_, dw_, st, pd)
        ctx.bias_act(two, db_, B, Cout, oh * ow, act=1)
        assert np.array_equal(fused.numpy(), two.numpy()), ("bias+relu", case)
        # a caller-provided workspace of exactly the advertised size
        need = capi.lib.fx_conv2d_workspace_bytes(capi.CONV_WGRAD, capi.FX_F32, 0, *dims)
        assert need >= 0
        ws = ctx.empty((max(need, 4) // 4,), np.float32)
        out = ctx.empty(w.shape, np.float32)
        capi.check(capi.lib.fx_conv2d_wgrad_f32(ctx.h, dx_.ptr, dg_.ptr, out.ptr, *dims, 0, ws.ptr, need))
        assert np.array_equal(out.numpy(), gw), case


# maps 32 wide, heights a multiple of 8, output channels a multiple of 32: the image-layer kernel of conv_image_f64.hpp (1 to 4
# channels, one to five tiles per image, one to three blocks of output channels)
IMAGE_F64_EXTRA = [
    (3, 1, 8, 32, 64, (1, 1), (1, 1)), (2, 4, 40, 32, 96, (1, 1), (1, 1)), (5, 2, 24, 32, 32, (1, 1), (1, 1)),
    (9, 3, 32, 32, 32, (1, 1), (1, 1)), (70, 3, 32, 32, 64, (1, 1), (1, 1)),
    # row-band weight gradient: heights that are not multiples of 8 or of the band, bands of 4 and 8 rows
    (9, 3, 33, 32, 32, (1, 1), (1, 1)), (140, 2, 30, 32, 32, (1, 1), (1, 1)), (300, 1, 30, 32, 64, (1, 1), (1, 1)),
]


def test_conv2d_f64_image_layer_forward(ctx, orc):
    """Image layers in f64 (1 to 4 input channels, K = Cin * 9 below two slabs of the implicit GEMM): forward, bias + ReLU in the store,
    weight gradient."""
    import torch
    import torch.nn.functional as F
    from ferrox_amd import capi
    rng = np.random.default_rng(63)
    for (B, Cin, H, W, Cout, st, pd) in SMALLC_CASES + IMAGE_F64_EXTRA:
        case = (B, Cin, H, W, Cout, st, pd)
        x = rng.uniform(-1, 1, (B, Cin, H, W))
        w = rng.standard_normal((Cout, Cin, 3, 3)) * np.sqrt(2.0 / (Cin * 9))
        bias = rng.standard_normal(Cout)
        oh, ow = orc.out_hw(H, W, 3, 3, st[0], st[1], pd[0], pd[1])
        dx_, dw_, db_ = ctx.upload(x), ctx.upload(w), ctx.upload(bias)
        y = ctx.conv2d_fwd(dx_, dw_, st, pd).numpy()
        ty = F.conv2d(torch.from_numpy(x), torch.from_numpy(w), stride=st, padding=pd).numpy()
        ay = F.conv2d(torch.from_numpy(np.abs(x)), torch.from_numpy(np.abs(w)), stride=st, padding=pd).max().item()
        parity.check("image layers fwd f64", y, ty, oracle=orc.conv2d_fwd(x, w, st, pd), case=case, terms=ay)
        assert np.array_equal(ctx.conv2d_fwd(dx_, dw_, st, pd).numpy(), y), case
        dims = (B, Cin, H, W, Cout, 3, 3, st[0], st[1], pd[0], pd[1])
        fused = ctx.empty(y.shape, np.float64)
        capi.check(capi.lib.fx_conv2d_fwd_bias_act_f64(ctx.h, dx_.ptr, dw_.ptr, db_.ptr, fused.ptr, *dims, 1, None, 0))
        two = ctx.conv2d_fwd(dx_, dw_, st, pd)
        capi.check(capi.lib.fx_bias_act_f64(ctx.h, two.ptr, db_.ptr, B, Cout, oh * ow, 1))
        assert np.array_equal(fused.numpy(), two.numpy()), ("bias+relu", case)
        # the weight gradient of the layer (conv_image_f64.hpp for 1 to 3 channels on maps 32 wide, the implicit GEMM otherwise)
        g = rng.standard_normal((B, Cout, oh, ow))
        dg_ = ctx.upload(g)
        gw = ctx.conv2d_wgrad(dx_, dg_, w.shape, st, pd, 0).numpy()
        tw = torch.from_numpy(w).requires_grad_(True)
        F.conv2d(torch.from_numpy(x), tw, stride=st, padding=pd).backward(torch.from_numpy(g))
        parity.check("image layers wgrad f64", gw, tw.grad.numpy(), oracle=orc.conv2d_wgrad(x, g, w.shape, st, pd, 0), case=case)
        assert np.array_equal(ctx.conv2d_wgrad(dx_, dg_, w.shape, st, pd, 0).numpy(), gw), case
        need = capi.lib.fx_conv2d_workspace_bytes(capi.CONV_WGRAD, capi.FX_F64, 0, *dims)
        assert need >= 0
        ws = ctx.empty((max(need, 8) // 8,), np.float64)
        out = ctx.empty(w.shape, np.float64)
        capi.check(capi.lib.fx_conv2d_wgrad_f64(ctx.h, dx_.ptr, dg_.ptr, out.ptr, *dims, 0, ws.ptr, need))
        assert np.array_equal(out.numpy(), gw), case


def test_conv2d_tune_up_front_and_ragged_batch(ctx, orc):
    """fx_conv2d_tune_f32 pays the tile timing for a layer before its first use; a ragged batch of the same size class and
    one of another class run afterwards, all against the oracle.  An output that overlaps an operand is not timed."""
    from ferrox_amd import capi
    rng = np.random.default_rng(61)
    Cin, H, W, Cout = 64, 16, 16, 64
    w = (rng.standard_normal((Cout, Cin, 3, 3)) * 0.05).astype(np.float32)
    dw = ctx.upload(w)
    for kind in (capi.CONV_FWD, capi.CONV_DGRAD, capi.CONV_WGRAD):
        ctx.conv2d_tune(kind, (40, Cin, H, W), w.shape, (1, 1), (1, 1))
    ctx.conv2d_tune(capi.CONV_FWD, (40, Cin, H, W), w.shape, (1, 1), (1, 1), with_bias=True, act=1)
    for B in (40, 37, 9):
        x = rng.uniform(-1, 1, (B, Cin, H, W)).astype(np.float32)
        g = rng.standard_normal((B, Cout, H, W)).astype(np.float32)
        y = ctx.conv2d_fwd(ctx.upload(x), dw, (1, 1), (1, 1)).numpy()
        d = ctx.conv2d_dgrad(ctx.upload(g), dw, x.shape, (1, 1), (1, 1), 0).numpy()
        assert rel_err(y, orc.conv2d_fwd(x, w, (1, 1), (1, 1))) <= 8e-5 / 8
        assert rel_err(d, orc.conv2d_dgrad(g, w, x.shape, (1, 1), (1, 1), 0)) <= 8e-5 / 8
    with pytest.raises(capi.FerroxHipError, match="unknown kind"):
        ctx.conv2d_tune(7, (4, Cin, H, W), w.shape, (1, 1), (1, 1))


def test_conv2d_tile_shape_timing_does_not_change_the_bits(ctx, tmp_path):
    """The forward / data-gradient patch kernel times its candidate tile shapes on the first call of a layer shape.  Every
    shape adds the terms of an output in the same order, so a process that keeps the modelled shape (FX_CONV_TUNE=0) must
    produce the same bits as this one, whatever shape won here."""
    import os
    import subprocess
    import sys
    cases = [(32, 64, 56, 56, 128), (64, 64, 32, 32, 64), (128, 32, 16, 16, 64)]
    script = tmp_path / "untuned.py"
    script.write_text(
        "import sys, numpy as np\n"
        "sys.path.insert(0, %r)\n"
        "from ferrox_amd import capi\n"
        "ctx = capi.Context(0)\n"
        "for i, (B, Cin, H, W, Cout) in enumerate(%r):\n"
        "    x = ctx.uniform((B, Cin, H, W), 71 + i, -1.0, 1.0)\n"
        "    w = ctx.normal((Cout, Cin, 3, 3), 81 + i, 0.0, 0.05)\n"
        "    g = ctx.normal((B, Cout, H, W), 91 + i, 0.0, 1.0)\n"
        "    np.save(%r + '/y%%d.npy' %% i, ctx.conv2d_fwd(x, w, (1, 1), (1, 1)).numpy())\n"
        "    np.save(%r + '/d%%d.npy' %% i, ctx.conv2d_dgrad(g, w, (B, Cin, H, W), (1, 1), (1, 1), 0).numpy())\n"
        "ctx.close()\n" % (os.path.dirname(os.path.dirname(os.path.abspath(__file__))), cases, str(tmp_path), str(tmp_path)))
    env = dict(os.environ, FX_CONV_TUNE="0")
    subprocess.run([sys.executable, str(script)], check=True, env=env, timeout=240)
    for i, (B, Cin, H, W, Cout) in enumerate(cases):
        x = ctx.uniform((B, Cin, H, W), 71 + i, -1.0, 1.0)
        w = ctx.normal((Cout, Cin, 3, 3), 81 + i, 0.0, 0.05)
        g = ctx.normal((B, Cout, H, W), 91 + i, 0.0, 1.0)
        y = ctx.conv2d_fwd(x, w, (1, 1), (1, 1)).numpy()
        d = ctx.conv2d_dgrad(g, w, (B, Cin, H, W), (1, 1), (1, 1), 0).numpy()
        assert np.array_equal(y, np.load(tmp_path / ("y%d.npy" % i))), ("fwd", cases[i])
        assert np.array_equal(d, np.load(tmp_path / ("d%d.npy" % i))), ("dgrad", cases[i])
        assert np.array_equal(y, ctx.conv2d_fwd(x, w, (1, 1), (1, 1)).numpy())


# Strided data gradients, computed per pixel class (Cout % 16 == 0, kernel >= stride) and by the all-taps gather
# otherwise: odd sizes, classes without pixels, kernel == stride, stride 3, 5x5, asymmetric stride and padding.
# B, Cin, H, W, Cout, (kh, kw), (sh, sw), (ph, pw)
STRIDED_DGRAD_CASES = [
    (3, 5, 9, 7, 16, (3, 3), (2, 2), (1, 1)), (2, 32, 32, 32, 64, (3, 3), (2, 2), (1, 1)), (2, 40, 11, 13, 32, (3, 3), (2, 1), (1, 0)),
    (2, 3, 8, 8, 16, (2, 2), (2, 2), (0, 0)), (2, 70, 10, 9, 48, (3, 3), (3, 3), (1, 1)), (1, 8, 12, 12, 16, (5, 5), (2, 2), (2, 2)),
    (2, 4, 1, 9, 16, (3, 3), (2, 2), (1, 1)), (2, 130, 7, 6, 32, (3, 3), (1, 2), (0, 1)), (2, 6, 9, 9, 24, (3, 3), (2, 2), (1, 1)),
    (1, 2, 5, 5, 16, (3, 3), (2, 2), (0, 0)),
    # stride 2, padding 1, maps 32 and 64 wide: the parity-class patch kernel (one and several tiles per image, channel tiles,
    # one to eight output-channel chunks)
    (3, 32, 32, 32, 64, (3, 3), (2, 2), (1, 1)), (2, 64, 32, 32, 128, (3, 3), (2, 2), (1, 1)), (2, 32, 64, 64, 32, (3, 3), (2, 2), (1, 1)),
    (2, 64, 16, 64, 64, (3, 3), (2, 2), (1, 1)), (2, 32, 32, 32, 48, (3, 3), (2, 2), (1, 1)), (1, 96, 64, 32, 16, (3, 3), (2, 2), (1, 1)),
    # output channels in chunks of 8 (the f64 kernel): one chunk, three chunks
    (1, 32, 32, 32, 8, (3, 3), (2, 2), (1, 1)), (2, 32, 32, 64, 24, (3, 3), (2, 2), (1, 1)),
]


@pytest.mark.parametrize("dtype", DTYPES)
def test_conv2d_strided_dgrad_vs_torch_and_oracle(ctx, orc, dtype):
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(60)
    for (B, Cin, H, W, Cout, k, st, pd) in STRIDED_DGRAD_CASES:
        case = (B, Cin, H, W, Cout, k, st, pd)
        oh, ow = orc.out_hw(H, W, k[0], k[1], st[0], st[1], pd[0], pd[1])
        w = (rng.standard_normal((Cout, Cin, k[0], k[1])) * np.sqrt(2.0 / (Cin * k[0] * k[1]))).astype(dtype)
        g = rng.standard_normal((B, Cout, oh, ow)).astype(dtype)
        dx = ctx.conv2d_dgrad(ctx.upload(g), ctx.upload(w), (B, Cin, H, W), st, pd, 0).numpy()
        tx = torch.zeros((B, Cin, H, W), dtype=torch.float64, requires_grad=True)
        F.conv2d(tx, torch.from_numpy(w).double(), stride=st, padding=pd).backward(torch.from_numpy(g).double())
        parity.check("strided dgrad", dx, tx.grad.numpy(), oracle=orc.conv2d_dgrad(g, w, (B, Cin, H, W), st, pd, 0), case=case)


# 1x1 filters at unit stride without padding: one launch of the batched LDS-slab product where the channel counts allow it
# (channels reduced in slabs of 64, at least 128 of them; rows of H*W floats a multiple of four), the implicit GEMM otherwise.
# B, Cin, H, W, Cout
POINTWISE_CASES = [(3, 128, 16, 16, 256), (4, 256, 8, 8, 128), (2, 192, 12, 20, 96), (70, 128, 8, 8, 64), (1, 512, 32, 32, 128),
                   (2, 64, 16, 16, 64), (3, 130, 8, 8, 70), (2, 128, 7, 9, 256), (5, 256, 16, 16, 256),
                   # maps whose pixel count is no multiple of 64 (the weight gradient's reduction length): 14 x 14, 28 x 28, 10 x 10
                   (64, 256, 14, 14, 256), (16, 128, 28, 28, 256), (96, 128, 10, 10, 128),
                   # about one 64-row tile per CU
                   (4, 512, 28, 28, 256), (2, 256, 32, 32, 512)]


def test_conv2d_pointwise_layers(ctx, orc):
    import torch
    import torch.nn.functional as F
    from ferrox_amd import capi
    rng = np.random.default_rng(64)
    for (B, Cin, H, W, Cout) in POINTWISE_CASES:
        case = (B, Cin, H, W, Cout)
        x = rng.uniform(-1, 1, (B, Cin, H, W)).astype(np.float32)
        w = (rng.standard_normal((Cout, Cin, 1, 1)) * np.sqrt(2.0 / Cin)).astype(np.float32)
        g = rng.standard_normal((B, Cout, H, W)).astype(np.float32)
        bias = rng.standard_normal(Cout).astype(np.float32)
        dx_, dw_, dg_, db_ = ctx.upload(x), ctx.upload(w), ctx.upload(g), ctx.upload(bias)
        y = ctx.conv2d_fwd(dx_, dw_, (1, 1), (0, 0)).numpy()
        gx = ctx.conv2d_dgrad(dg_, dw_, x.shape, (1, 1), (0, 0), 0).numpy()
        gw = ctx.conv2d_wgrad(dx_, dg_, w.shape, (1, 1), (0, 0), 0).numpy()
        tx = torch.from_numpy(x).double().requires_grad_(True)
        tw = torch.from_numpy(w).double().requires_grad_(True)
        ty = F.conv2d(tx, tw)
        ty.backward(torch.from_numpy(g).double())
        ay = F.conv2d(tx.detach().abs(), tw.detach().abs()).max().item()
        small = B * Cout * H * W * Cin <= 1 << 27  # the oracle's explicit column matrix stays small
        parity.check("pointwise fwd", y, ty.detach().numpy(), oracle=orc.conv2d_fwd(x, w, (1, 1), (0, 0)) if small else None, case=case, terms=ay)
        parity.check("pointwise dgrad", gx, tx.grad.numpy(), oracle=orc.conv2d_dgrad(g, w, x.shape, (1, 1), (0, 0), 0) if small else None, case=case)
        parity.check("pointwise wgrad", gw, tw.grad.numpy(), oracle=orc.conv2d_wgrad(x, g, w.shape, (1, 1), (0, 0), 0) if small else None, case=case)
        # same bits on a second run; bias + ReLU in the store equals the separate pass
        assert np.array_equal(ctx.conv2d_fwd(dx_, dw_, (1, 1), (0, 0)).numpy(), y), case
        assert np.array_equal(ctx.conv2d_wgrad(dx_, dg_, w.shape, (1, 1), (0, 0), 0).numpy(), gw), case
        dims = (B, Cin, H, W, Cout, 1, 1, 1, 1, 0, 0)
        fused = ctx.empty(y.shape, np.float32)
        capi.check(capi.lib.fx_conv2d_fwd_bias_act_f32(ctx.h, dx_.ptr, dw_.ptr, db_.ptr, fused.ptr, *dims, 1, None, 0))
        two = ctx.conv2d_fwd(dx_, dw_, (1, 1), (0, 0))
        capi.check(capi.lib.fx_bias_act_f32(ctx.h, two.ptr, db_.ptr, B, Cout, H * W, 1))
        assert np.array_equal(fused.numpy(), two.numpy()), ("bias+relu", case)
        # a caller workspace of exactly the advertised size for the weight gradient
        need = capi.lib.fx_conv2d_workspace_bytes(capi.CONV_WGRAD, capi.FX_F32, 0, *dims)
        ws = ctx.empty((max(need, 4) // 4,), np.float32)
        out = ctx.empty(w.shape, np.float32)
        capi.check(capi.lib.fx_conv2d_wgrad_f32(ctx.h, dx_.ptr, dg_.ptr, out.ptr, *dims, 0, ws.ptr, need))
        assert np.array_equal(out.numpy(), gw), case


EXPECTED_PATHS = [  # (B, Cin, H, W, Cout, k, stride, padding, dtype) -> kernel family of forward, data gradient, weight gradient
    ((8, 64, 56, 56, 128, 3, 1, 1, np.float32), ("LDS patch (cpk)", "LDS patch (cpk)", "LDS patch (wgp)")),                       # the roofline layer
    ((8, 64, 56, 56, 128, 3, 1, 1, np.float64), ("LDS patch (cpd)", "LDS patch (cpd)", "LDS patch (wgd)")),
    ((16, 3, 32, 32, 32, 3, 1, 1, np.float32), ("image layer, tiles (csc)", "direct gather, few input channels", "image layer, row bands (csc)")),
    ((16, 3, 32, 32, 32, 3, 1, 1, np.float64), ("image layer (cim)", "direct gather, few input channels", "image layer, row bands (cim)")),
    ((16, 32, 32, 32, 64, 3, 2, 1, np.float32), ("LDS patch (cpk)", "stride-2 patch (dg2)", "stride-2 patch (wg2)")),
    ((16, 32, 32, 32, 64, 3, 2, 1, np.float64), ("stride-2 patch (fwd2)", "stride-2 patch (dgd2)", "stride-2 patch (wgd2)")),
    ((16, 32, 16, 16, 64, 3, 2, 1, np.float64), ("implicit GEMM", "implicit GEMM by pixel classes", "stride-2 patch (wgd2)")),
    ((2, 64, 12, 112, 128, 3, 1, 1, np.float32), ("LDS patch (cpk)", "LDS patch (cpk)", "LDS patch, row segments (wgp)")),       # rows of 112 floats
    ((1, 64, 6, 224, 64, 3, 1, 1, np.float32), ("LDS patch (cpk)", "LDS patch (cpk)", "LDS patch, row segments (wgp)")),         # rows of 224 floats
    ((1, 3, 128, 128, 32, 3, 1, 1, np.float32), ("image layer, tiles (csc)", "direct gather, few input channels", "image layer, tiles (csc)")),  # the reference's benchmark layer
    ((64, 256, 32, 32, 256, 1, 1, 0, np.float32), ("1x1 as batched slab GEMM (glk)",) * 3),                                     # enough tiles to fill the chip
    ((4, 32, 20, 20, 64, 5, 1, 2, np.float32), ("implicit GEMM",) * 3),                                                          # no 5 x 5 kernels
    ((4, 64, 56, 56, 128, 3, 2, 1, np.float32), ("LDS patch (cpk)", "implicit GEMM by pixel classes", "stride-2 patch (wg2)")),   # stride 2 over a 56-wide map
    ((8, 64, 16, 16, 128, 3, 2, 1, np.float32), ("LDS patch (cpk)", "implicit GEMM by pixel classes", "stride-2 patch (wg2)")),   # ... and a 16-wide one
    ((8, 64, 28, 28, 128, 3, 2, 1, np.float32), ("LDS patch (cpk)", "implicit GEMM by pixel classes", "stride-2 patch (wg2)")),   # 23 patch rows under a tile
    ((8, 64, 14, 14, 128, 3, 2, 1, np.float32), ("LDS patch (cpk)", "implicit GEMM by pixel classes", "implicit GEMM")),          # two 7 x 7 outputs per tile
]


def test_layers_take_the_kernels_written_for_them(ctx):
    """A parity test passes on the implicit GEMM as well: this one asks the library which kernel family each call ran, for the
    baseline layers and for one layer per specialised path, so that a planner that silently starts refusing a shape fails here."""
    for (B, Cin, H, W, Cout, k, s, p, dtype), want in EXPECTED_PATHS:
        oh, ow = (H + 2 * p - k) // s + 1, (W + 2 * p - k) // s + 1
        x, w, g = ctx.uniform((B, Cin, H, W), 1, -1.0, 1.0, dtype), ctx.normal((Cout, Cin, k, k), 2, 0.0, 0.1, dtype), ctx.normal((B, Cout, oh, ow), 3, 0.0, 1.0, dtype)
        got = []
        ctx.conv2d_fwd(x, w, (s, s), (p, p)).free()
        got.append(ctx.conv2d_last_path())
        ctx.conv2d_dgrad(g, w, x.shape, (s, s), (p, p), 0).free()
        got.append(ctx.conv2d_last_path())
        ctx.conv2d_wgrad(x, g, w.shape, (s, s), (p, p), 0).free()
        got.append(ctx.conv2d_last_path())
        for a in (x, w, g):
            a.free()
        assert tuple(got) == want, ((B, Cin, H, W, Cout, k, s, p, np.dtype(dtype).name), got, want)


RANDOM_CONV_SEEDS = [(61, np.float32), (62, np.float32), (63, np.float32), (64, np.float32), (65, np.float64), (66, np.float64),
                     (67, np.float32), (68, np.float32), (69, np.float64), (70, np.float32), (71, np.float64)]


def random_conv_shapes(seed):
    """Seeded random 3x3 / 1x1 / 5x5 layer shapes biased towards the dispatch boundaries of the conv kernels (channel counts around
    multiples of 8 / 16 / 32 / 64, widths around 64 and multiples of 4, strides 1-3, paddings 0-2); seeds from 67 on draw rows of
    72 to 256 floats (the wide-row paths of the patch kernels).  Also walked on the CPU before they run on a GPU."""
    rng = np.random.default_rng(seed)
    chans = [1, 3, 4, 8, 16, 24, 32, 40, 64, 65, 72, 96, 128, 136]
    widths = [4, 6, 8, 12, 14, 16, 20, 28, 30, 32, 36, 56, 60, 64, 66, 68] if seed < 67 else [72, 80, 96, 100, 112, 126, 128, 130, 160, 192, 224, 256]
    heights = [1, 2, 3, 5, 8, 9, 14, 28] if seed < 67 else [1, 2, 3, 4, 5, 7]
    out = []
    for it in range(70 if seed < 67 else 40):
        Cin, Cout = int(rng.choice(chans)), int(rng.choice(chans))
        k = int(rng.choice([3, 3, 3, 3, 1, 5]))
        sh, sw = int(rng.choice([1, 1, 1, 2, 3])), int(rng.choice([1, 1, 1, 2, 3]))
        ph, pw = int(rng.integers(0, 3)), int(rng.integers(0, 3))
        W = int(rng.choice(widths))
        H = int(rng.choice(heights)) if seed >= 67 or rng.random() < 0.7 else W
        B = int(rng.choice([1, 2, 3, 5]))
        if H + 2 * ph < k or W + 2 * pw < k or B * Cin * H * W > 1_500_000 or B * Cout * H * W > 3_000_000:
            continue
        out.append((it, B, Cin, H, W, Cout, k, (sh, sw), (ph, pw)))
    return out


@pytest.mark.parametrize("seed,dtype", RANDOM_CONV_SEEDS)
def test_conv2d_random_shapes_all_paths_vs_torch(ctx, seed, dtype):
    """Forward, data gradient and weight gradient of random_conv_shapes(seed) against torch in float64."""
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(seed + 1000)
    for case in random_conv_shapes(seed):
        it, B, Cin, H, W, Cout, k, (sh, sw), (ph, pw) = case
        x = rng.uniform(-1, 1, (B, Cin, H, W)).astype(dtype)
        w = (rng.standard_normal((Cout, Cin, k, k)) * np.sqrt(2.0 / (Cin * k * k))).astype(dtype)
        tx = torch.from_numpy(x).double().requires_grad_(True)
        tw = torch.from_numpy(w).double().requires_grad_(True)
        ty = F.conv2d(tx, tw, stride=(sh, sw), padding=(ph, pw))
        g = rng.standard_normal(tuple(ty.shape)).astype(dtype)
        ty.backward(torch.from_numpy(g).double())
        dx_, dw_, dg_ = ctx.upload(x), ctx.upload(w), ctx.upload(g)
        y = ctx.conv2d_fwd(dx_, dw_, (sh, sw), (ph, pw)).numpy()
        ay = F.conv2d(tx.detach().abs(), tw.detach().abs(), stride=(sh, sw), padding=(ph, pw)).max().item()
        parity.check("random shapes fwd", y, ty.detach().numpy(), case=case, terms=max(ay, 1e-30))
        parity.check("random shapes dgrad", ctx.conv2d_dgrad(dg_, dw_, x.shape, (sh, sw), (ph, pw), 0).numpy(), tx.grad.numpy(), case=case)
        parity.check("random shapes wgrad", ctx.conv2d_wgrad(dx_, dg_, w.shape, (sh, sw), (ph, pw), 0).numpy(), tw.grad.numpy(), case=case)


def test_conv2d_misaligned_tensors_match_aligned(ctx):
    """Tensors that are only 4-byte aligned (a view into a larger buffer) cannot use the 16-byte loads of the
    patch kernels; the library must fall back and give the implicit-GEMM result, not fault or misread."""
    from ferrox_amd import capi
    rng = np.random.default_rng(59)
    B, Cin, H, W, Cout = 2, 32, 10, 56, 100
    x = rng.uniform(-1, 1, (B, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, Cin, 3, 3)) * 0.06).astype(np.float32)
    g = rng.standard_normal((B, Cout, H, W)).astype(np.float32)
    dims = (B, Cin, H, W, Cout, 3, 3, 1, 1, 1, 1)

    def shifted(a):  # device copy of `a` that starts 4 bytes into its allocation
        buf = ctx.upload(np.concatenate([np.zeros(1, np.float32), a.ravel()]))
        return buf, buf.ptr + 4

    (xb, xp), (gb, gp) = shifted(x), shifted(g)
    dw_, dx_al, dg_al = ctx.upload(w), ctx.upload(x), ctx.upload(g)
    y, dx, dwt = ctx.empty(g.shape, np.float32), ctx.empty(x.shape, np.float32), ctx.empty(w.shape, np.float32)
    capi.check(capi.lib.fx_conv2d_fwd_f32(ctx.h, xp, dw_.ptr, y.ptr, *dims, None, 0))
    capi.check(capi.lib.fx_conv2d_dgrad_f32(ctx.h, gp, dw_.ptr, dx.ptr, *dims, 0, None, 0))
    capi.check(capi.lib.fx_conv2d_wgrad_f32(ctx.h, xp, gp, dwt.ptr, *dims, 0, None, 0))
    import torch
    import torch.nn.functional as F
    tx = torch.from_numpy(x).double().requires_grad_(True)
    tw = torch.from_numpy(w).double().requires_grad_(True)
    ty = F.conv2d(tx, tw, stride=1, padding=1)
    ty.backward(torch.from_numpy(g).double())
    # the fallback kernels (misaligned) and the aligned ones, each against the float64 truth
    parity.check("misaligned fwd", y.numpy(), ty.detach().numpy(), oracle=ctx.conv2d_fwd(dx_al, dw_, (1, 1), (1, 1)).numpy())
    parity.check("misaligned dgrad", dx.numpy(), tx.grad.numpy(), oracle=ctx.conv2d_dgrad(dg_al, dw_, x.shape, (1, 1), (1, 1), 0).numpy())
    parity.check("misaligned wgrad", dwt.numpy(), tw.grad.numpy(), oracle=ctx.conv2d_wgrad(dx_al, dg_al, w.shape, (1, 1), (1, 1), 0).numpy())
    del xb, gb


def test_conv2d_reference_vectors(ctx, golden):
    for key in ("conv2d_test", "conv2d_simple_forward", "conv2d_edge_cases"):
        gv = golden[key]
        x = np.array(gv["x"], np.float32).reshape(gv["x_shape"])
        w = np.array(gv["w"], np.float32).reshape(gv["w_shape"])
        y = ctx.conv2d_fwd(ctx.upload(x), ctx.upload(w), tuple(gv["stride"]), tuple(gv["padding"])).numpy()
        assert list(y.shape) == gv["y_shape"]
        np.testing.assert_allclose(y.ravel(), np.array(gv["y"], np.float32), atol=gv["tol"], rtol=0)


def test_conv2d_run_to_run_determinism(ctx):
    rng = np.random.default_rng(51)
    x = ctx.upload(rng.uniform(-1, 1, (4, 16, 20, 20)).astype(np.float32))
    w = ctx.upload(rng.standard_normal((24, 16, 3, 3)).astype(np.float32))
    g = ctx.upload(rng.standard_normal((4, 24, 20, 20)).astype(np.float32))
    a = [ctx.conv2d_dgrad(g, w, x.shape, (1, 1), (1, 1)).numpy(), ctx.conv2d_wgrad(x, g, w.shape, (1, 1), (1, 1)).numpy()]
    b = [ctx.conv2d_dgrad(g, w, x.shape, (1, 1), (1, 1)).numpy(), ctx.conv2d_wgrad(x, g, w.shape, (1, 1), (1, 1)).numpy()]
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
