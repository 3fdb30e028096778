"""The benchmark configurations at their full sizes, checked through properties that do not need a CPU run of the
whole problem: sampled outputs against float64 arithmetic on the host, the adjoint identity that ties the three
convolution passes together, linearity, and exact / order-independent facts about the reductions.
  C3  conv N=128 Cin=64 56x56 -> Cout=128 3x3 s1 p1 f32          C4  reductions on 8192 x 8192, elementwise on 2^28 f32
(the MLP / CNN training configurations run at full size against the oracle in test_gpu_train.py)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from ferrox_amd import capi
    c = capi.Context(0)
    yield c
    c.close()


def dot64(a, b):
    """sum(a*b) in float64, in slabs (keeps the temporaries small)."""
    a, b = a.reshape(-1), b.reshape(-1)
    s, sa, step = 0.0, 0.0, 1 << 24
    for i in range(0, a.size, step):
        p = a[i:i + step].astype(np.float64) * b[i:i + step]
        s += p.sum()
        sa += np.abs(p).sum()
    return s, sa


def test_c3_convolution_full_size(ctx):
    B, Cin, H, W, Cout = 128, 64, 56, 56, 128
    st, pd = (1, 1), (1, 1)
    dx = ctx.uniform((B, Cin, H, W), 3, -1.0, 1.0)
    dw = ctx.normal((Cout, Cin, 3, 3), 4, 0.0, float(np.sqrt(2.0 / 576)))
    dg = ctx.normal((B, Cout, H, W), 5, 0.0, 1.0)
    x, w, g = dx.numpy(), dw.numpy(), dg.numpy()
    y = ctx.conv2d_fwd(dx, dw, st, pd).numpy()
    gx = ctx.conv2d_dgrad(dg, dw, x.shape, st, pd, 0).numpy()
    gw = ctx.conv2d_wgrad(dx, dg, w.shape, st, pd, 0).numpy()
    rng = np.random.default_rng(0)
    xp = np.zeros((B, Cin, H + 2, W + 2), np.float32)
    xp[:, :, 1:-1, 1:-1] = x
    gp = np.zeros((B, Cout, H + 2, W + 2), np.float32)
    gp[:, :, 1:-1, 1:-1] = g
    w64 = w.astype(np.float64)
    # sampled entries of each pass, corners and edges included, against float64 sums; tolerance 1e-5 of sum |terms|
    pts = [(0, 0, 0, 0), (B - 1, Cout - 1, H - 1, W - 1), (5, 7, 0, W - 1), (9, 3, H - 1, 0)]
    pts += [tuple(int(v) for v in (rng.integers(B), rng.integers(Cout), rng.integers(H), rng.integers(W))) for _ in range(600)]
    import parity
    got_s, ref_s = [], []
    for (b, oc, oy, ox) in pts:
        patch = xp[b, :, oy:oy + 3, ox:ox + 3].astype(np.float64)
        ref, mag = (patch * w64[oc]).sum(), np.abs(patch * w64[oc]).sum()
        assert abs(y[b, oc, oy, ox] - ref) <= 1e-5 * mag, ("fwd", b, oc, oy, ox)
        got_s.append(y[b, oc, oy, ox]); ref_s.append(ref)
    # and the contract's own form on the sample: max |got - truth| within 1e-5 of max |truth|
    parity.check("C3 full size fwd (604 sampled outputs)", np.array(got_s), np.array(ref_s), np.float32, case=(B, Cin, H, W, Cout))
    got_s, ref_s = [], []
    for _ in range(600):
        b, c, yy, xx = (int(v) for v in (rng.integers(B), rng.integers(Cin), rng.integers(H), rng.integers(W)))
        # dx[b,c,y,x] = sum_{oc,ky,kx} g[b,oc,y+1-ky,x+1-kx] * w[oc,c,ky,kx]
        patch = gp[b, :, yy:yy + 3, xx:xx + 3][:, ::-1, ::-1].astype(np.float64)
        terms = patch * w64[:, c]
        assert abs(gx[b, c, yy, xx] - terms.sum()) <= 1e-5 * np.abs(terms).sum(), ("dgrad", b, c, yy, xx)
        got_s.append(gx[b, c, yy, xx]); ref_s.append(terms.sum())
    parity.check("C3 full size dgrad (600 sampled outputs)", np.array(got_s), np.array(ref_s), np.float32, case=(B, Cin, H, W, Cout))
    got_s, ref_s = [], []
    for _ in range(40):
        oc, c, ky, kx = (int(v) for v in (rng.integers(Cout), rng.integers(Cin), rng.integers(3), rng.integers(3)))
        terms = g[:, oc].astype(np.float64) * xp[:, c, ky:ky + H, kx:kx + W]
        assert abs(gw[oc, c, ky, kx] - terms.sum()) <= 1e-5 * np.abs(terms).sum(), ("wgrad", oc, c, ky, kx)
        got_s.append(gw[oc, c, ky, kx]); ref_s.append(terms.sum())
    parity.check("C3 full size wgrad (40 sampled outputs)", np.array(got_s), np.array(ref_s), np.float32, case=(B, Cin, H, W, Cout))
    # adjoint identity: <conv(x, w), g> = <x, dgrad(g, w)> = <w, wgrad(x, g)>
    a, mag = dot64(y, g)
    b_, _ = dot64(x, gx)
    c_, _ = dot64(w, gw)
    assert abs(a - b_) <= 1e-6 * mag and abs(a - c_) <= 1e-6 * mag, (a, b_, c_, mag)
    # linearity in the filter
    dw2 = ctx.normal((Cout, Cin, 3, 3), 6, 0.0, 0.05)
    y2 = ctx.conv2d_fwd(dx, dw2, st, pd)
    ysum = ctx.conv2d_fwd(dx, ctx.binary("add", dw, dw2), st, pd).numpy()
    ref = y.astype(np.float64) + y2.numpy()
    assert np.abs(ysum - ref).max() <= 2e-5 * np.abs(ref).max()
    # same bits run to run
    assert np.array_equal(ctx.conv2d_wgrad(dx, dg, w.shape, st, pd, 0).numpy(), gw)
    assert np.array_equal(ctx.conv2d_fwd(dx, dw, st, pd).numpy(), y)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_c4_reductions_full_size(ctx, dtype):
    n = 8192
    da = ctx.normal((n, n), 4, 0.0, 1.0, dtype)
    a = da.numpy()
    a64 = a.astype(np.float64)
    tol = 1e-5 if dtype == np.float32 else 1e-12
    for axis in (0, 1):
        s = ctx.reduce("sum", da, axis).numpy()
        ref, mag = a64.sum(axis=axis), np.abs(a64).sum(axis=axis)
        assert np.all(np.abs(s - ref) <= tol * mag), axis
        m = ctx.reduce("mean", da, axis).numpy()
        assert np.all(np.abs(m - ref / n) <= tol * mag / n), axis
        v, idx = ctx.reduce("max", da, axis, want_idx=True)
        assert np.array_equal(v.numpy(), a.max(axis=axis)) and np.array_equal(idx, a.argmax(axis=axis)), axis
        v, idx = ctx.reduce("min", da, axis, want_idx=True)
        assert np.array_equal(v.numpy(), a.min(axis=axis)) and np.array_equal(idx, a.argmin(axis=axis)), axis
    flat = da.reshape(n * n)
    total = ctx.reduce("sum", flat, 0).numpy().item()
    assert abs(total - a64.sum()) <= tol * np.abs(a64).sum()
    v, idx = ctx.reduce("max", flat, 0, want_idx=True)
    assert v.numpy().item() == a.max() and int(np.asarray(idx).reshape(-1)[0]) == int(a.argmax())
    # a sum of the column sums is the sum of everything (to rounding)
    cols = ctx.reduce("sum", da, 0)
    assert abs(ctx.reduce("sum", cols, 0).numpy().item() - total) <= 4 * tol * np.abs(a64).sum()


def test_c4_elementwise_full_size(ctx):
    import oracle as orc
    n = 1 << 28
    dg = ctx.uniform((n,), 7, -4.0, 4.0)
    dx = ctx.uniform((n,), 8, -4.0, 4.0)
    g, x = dg.numpy(), dx.numpy()
    assert np.array_equal(ctx.binary("add", dg, dx).numpy(), g + x)
    assert np.array_equal(ctx.binary("mul", dg, dx).numpy(), g * x)
    assert np.array_equal(ctx.relu_bwd(dg, dx).numpy(), g * (x > 0))
    ds, dt = ctx.unary("sigmoid", dx), ctx.unary("tanh", dx)
    s, t = ds.numpy(), dt.numpy()
    sb, tb = ctx.sigmoid_bwd(dg, ds, 0).numpy(), ctx.tanh_bwd(dg, dt).numpy()
    # the composed expressions of the reference's operators, rounded step by step like the kernels: g*(s*(1-s)) and
    # g*(-(t*t-1)) (ops/unary.rs:254-328), over the whole array in numpy float32 ...
    one = np.float32(1)
    assert np.array_equal(tb, g * (-(t * t - one)))
    assert np.array_equal(sb, g * (s * (one - s)))
    # ... and the oracle's own kernels on slices from the start, the middle and the ragged end
    for lo in (0, n // 2 - 12345, n - (1 << 20) - 3):
        sl = slice(lo, lo + (1 << 20) + 3)
        assert np.array_equal(sb[sl], orc.sigmoid_bwd(g[sl], s[sl], 0))
        assert np.array_equal(tb[sl], orc.tanh_bwd(g[sl], t[sl]))
        assert np.abs(s[sl] - orc.unary("sigmoid", x[sl])).max() <= 1.2e-7   # expf differs from libm by an ulp at most


def test_convolution_over_tensors_beyond_2_gib(ctx):
    """Tensors of 2 GiB or more run as slices of the batch: forward and data gradient are checked on the images either
    side of the slice boundary, the weight gradient against the ordered sum of two halves that each fit one launch."""
    import torch
    import torch.nn.functional as F
    B, Cin, H, W, Cout = 2300, 16, 128, 128, 16           # 2.41 GB per activation tensor; one launch takes 2047 images
    st, pd = (1, 1), (1, 1)
    per_image = Cin * H * W * 4
    cut = (2 ** 31 - 1) // per_image
    assert cut < B
    dx = ctx.uniform((B, Cin, H, W), 11, -1.0, 1.0)
    dw = ctx.normal((Cout, Cin, 3, 3), 12, 0.0, float(np.sqrt(2.0 / (Cin * 9))))
    dg = ctx.normal((B, Cout, H, W), 13, 0.0, 1.0)
    y = ctx.conv2d_fwd(dx, dw, st, pd)
    gx = ctx.conv2d_dgrad(dg, dw, (B, Cin, H, W), st, pd, 0)
    w = torch.from_numpy(dw.numpy()).double()
    for b in (0, cut - 1, cut, B - 1):
        xb = torch.from_numpy(dx.rows(b, b + 1).numpy()).double().requires_grad_(True)
        gb = torch.from_numpy(dg.rows(b, b + 1).numpy()).double()
        ref = F.conv2d(xb, w, stride=st, padding=pd)
        ref.backward(gb)
        mag = F.conv2d(xb.detach().abs(), w.abs(), stride=st, padding=pd).max().item()
        assert np.abs(y.rows(b, b + 1).numpy() - ref.detach().numpy()).max() <= 1e-5 * mag, ("fwd", b)
        gmag = F.conv_transpose2d(gb.abs(), w.abs(), stride=st, padding=pd).max().item()
        assert np.abs(gx.rows(b, b + 1).numpy() - xb.grad.numpy()).max() <= 1e-5 * gmag, ("dgrad", b)
    gw = ctx.conv2d_wgrad(dx, dg, (Cout, Cin, 3, 3), st, pd, 0).numpy()
    half = B // 2
    parts = [ctx.conv2d_wgrad(dx.rows(lo, hi), dg.rows(lo, hi), (Cout, Cin, 3, 3), st, pd, 0).numpy().astype(np.float64)
             for lo, hi in ((0, half), (half, B))]
    ref = parts[0] + parts[1]
    # sums of 37.7 million products each: the two groupings differ by rounding only
    assert np.abs(gw - ref).max() <= 1e-5 * np.abs(ref).max() + 1e-3
    assert np.array_equal(gw, ctx.conv2d_wgrad(dx, dg, (Cout, Cin, 3, 3), st, pd, 0).numpy())
    # the CPU-literal gradient modes read the batch as one flat matrix and refuse such sizes
    from ferrox_amd.capi import FerroxHipError
    with pytest.raises(FerroxHipError, match="mode 1 does not support tensors of 2 GiB or more"):
        ctx.conv2d_wgrad(dx, dg, (Cout, Cin, 3, 3), st, pd, 1)


def test_pooling_over_tensors_beyond_2_pow_31_elements(ctx):
    """One launch numbers its elements with 32 bits; larger tensors run as ranges of (image, channel) planes.  Checked
    on the images around the range boundary (plane 32767 of 256 x 256 elements lies inside image 2047)."""
    import oracle as orc
    N, Cc, H, W = 2100, 16, 256, 256                      # 2.2e9 elements, 8.8 GB
    dx = ctx.uniform((N, Cc, H, W), 21, -1.0, 1.0)
    dg = ctx.normal((N, Cc, H // 2, W // 2), 22, 0.0, 1.0)
    pooled = ctx.pool2d(dx, (2, 2), (2, 2), (0, 0), True)
    gin = ctx.unpool2d(dg, dx, pooled, (2, 2), (2, 2), (0, 0), True)
    avg = ctx.pool2d(dx, (3, 3), (2, 2), (1, 1), False)
    for b in (0, 2047, 2048, N - 1):
        x = dx.rows(b, b + 1).numpy()
        g = dg.rows(b, b + 1).numpy()
        want = orc.pool2d(x, (2, 2), (2, 2), (0, 0), True)
        assert np.array_equal(pooled.rows(b, b + 1).numpy(), want), ("max", b)
        assert np.array_equal(gin.rows(b, b + 1).numpy(), orc.unpool2d(g, x, want, (2, 2), (2, 2), (0, 0), True)), ("unpool", b)
        assert np.array_equal(avg.rows(b, b + 1).numpy(), orc.pool2d(x, (3, 3), (2, 2), (1, 1), False)), ("avg", b)


def test_batchnorm_statistics_over_more_than_2_pow_24_samples_per_channel(ctx):
    """f32 sample counts above 2^24 are only weights of the pairwise merge; mean and variance stay at float accuracy."""
    outer, Cc, inner = 48, 3, 1 << 20                      # 50.3 million samples per channel
    dx = ctx.normal((outer, Cc, inner), 31, 3.0, 2.0)
    mean, var = ctx.batchnorm_stats(dx)
    x = dx.numpy().astype(np.float64)
    m, v = x.mean(axis=(0, 2)), x.var(axis=(0, 2))
    assert np.abs(mean.numpy() - m).max() <= 1e-5 * np.abs(m).max()
    assert np.abs(var.numpy() - v).max() <= 1e-5 * v.max()
    mean2, var2 = ctx.batchnorm_stats(dx)
    assert np.array_equal(mean.numpy(), mean2.numpy()) and np.array_equal(var.numpy(), var2.numpy())
