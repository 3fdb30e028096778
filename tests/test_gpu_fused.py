"""Fused entry points (bias add + ReLU, bias gradient, softmax cross-entropy, Adam / SGD step) against the same
sequences composed op by op from the CPU oracle's primitives.  Where no reduction is involved the fused kernel
performs the composed path's operations in the same order, so the comparison is bit-exact."""
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
def train():
    import oracle.train as t
    return t


def rel_err(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-300)


@pytest.mark.parametrize("dtype", DTYPES)
def test_bias_act_bit_exact(ctx, train, dtype):
    rng = np.random.default_rng(70)
    for shape in [(4, 10), (256, 10), (3, 7, 5, 6), (2, 32, 8, 8), (5, 3, 1, 9), (1, 1, 1, 1), (2, 5, 4, 4)]:
        y = rng.standard_normal(shape).astype(dtype)
        b = rng.standard_normal(shape[1]).astype(dtype)
        inner = int(np.prod(shape[2:], dtype=np.int64))
        for act in (0, 1):
            got = ctx.bias_act(ctx.upload(y), ctx.upload(b), shape[0], shape[1], inner, act).numpy()
            assert np.array_equal(got, train.bias_act(y, b, relu=bool(act))), (shape, act)


@pytest.mark.parametrize("dtype", DTYPES)
def test_bias_grad_vs_oracle_and_float64(ctx, train, dtype):
    rng = np.random.default_rng(71)
    tol = TOL[np.dtype(dtype)]
    for shape in [(256, 10), (7, 3), (256, 32, 32, 32), (64, 64, 16, 16), (3, 5, 7, 9), (1, 4, 2, 2), (1000, 1, 3, 3)]:
        g = rng.standard_normal(shape).astype(dtype)
        inner = int(np.prod(shape[2:], dtype=np.int64))
        got = ctx.bias_grad(ctx.upload(g), shape[0], shape[1], inner).numpy()
        axes = (0,) if g.ndim == 2 else (0, 2, 3)
        truth = g.astype(np.float64).sum(axis=axes)
        scale = np.abs(g.astype(np.float64)).sum(axis=axes).max()
        assert np.abs(got - truth).max() <= tol * scale, shape
        assert np.abs(got - train.bias_grad(g)).max() <= 2 * tol * scale, shape
        # same bits on a second run
        assert np.array_equal(got, ctx.bias_grad(ctx.upload(g), shape[0], shape[1], inner).numpy())


@pytest.mark.parametrize("dtype", DTYPES)
def test_softmax_ce_fwd_bwd_vs_oracle(ctx, train, dtype):
    import torch
    rng = np.random.default_rng(72)
    tol = TOL[np.dtype(dtype)]
    for (B, C) in [(256, 10), (1, 1), (3, 2), (300, 17), (5, 1000), (1024, 16), (1500, 7), (700, 100)]:  # one- and two-kernel forward
        x = (rng.standard_normal((B, C)) * 3).astype(dtype)
        if B >= 3:
            x[0, 0] = 60.0   # saturates: the other classes' probabilities fall under the 1e-8 clamp
            x[1] = 0.0       # uniform row
        y = np.eye(C, dtype=dtype)[rng.integers(0, C, B)]
        if B >= 3:
            y[0] = 0
            y[0, C - 1] = 1  # target on a clamped class: the gradient must vanish there (f64) like the composed path
        probs, loss = ctx.softmax_ce_fwd(ctx.upload(x), ctx.upload(y))
        ol, os_ = train.softmax_ce_forward(x, y)
        # same operations in the same order as the library's softmax kernel; exp differs from the CPU libm by rounding
        assert np.array_equal(probs.numpy(), ctx.softmax_axis(ctx.upload(x), 1).numpy()), (B, C)
        assert np.abs(probs.numpy() - os_).max() <= 4 * tol, (B, C)
        assert abs(loss.numpy()[0] - ol.item()) <= 4 * tol * max(1.0, abs(ol.item())), (B, C)
        gl = np.array([0.75], dtype)
        d = ctx.softmax_ce_bwd(probs, ctx.upload(y), ctx.upload(gl)).numpy()
        od = train.softmax_ce_backward(probs.numpy(), y, gl[0])
        assert np.abs(d - od).max() <= 8 * tol * max(np.abs(od).max(), 1e-30), (B, C)
        # forward + gradient for a unit upstream gradient in one call: the bits of the two calls
        p1, l1, d1 = ctx.softmax_ce_fwd_unit_grad(ctx.upload(x), ctx.upload(y))
        assert np.array_equal(p1.numpy(), probs.numpy()) and np.array_equal(l1.numpy(), loss.numpy()), (B, C)
        assert np.array_equal(d1.numpy(), ctx.softmax_ce_bwd(probs, ctx.upload(y), ctx.upload(np.array([1.0], dtype))).numpy()), (B, C)
        # textbook check where the clamp is inactive: torch log_softmax in float64
        if C > 1 and B < 3:
            tx = torch.from_numpy(x.astype(np.float64)).requires_grad_(True)
            tl = -(torch.from_numpy(y.astype(np.float64)) * torch.log_softmax(tx, 1)).sum(1).mean()
            tl.backward()
            assert abs(loss.numpy()[0] - tl.item()) <= 1e-4 * max(1, abs(tl.item()))
            assert np.abs(d - 0.75 * tx.grad.numpy()).max() <= 1e-4


@pytest.mark.parametrize("dtype", DTYPES)
def test_adam_and_sgd_step_bit_exact(ctx, train, dtype):
    rng = np.random.default_rng(73)
    dt = np.dtype(dtype).type
    for n in (1, 10, 864, 18432, 163840):
        for wd in (0.0, 0.01):
            w = rng.standard_normal(n).astype(dtype)
            m = (rng.standard_normal(n) * 0.1).astype(dtype)
            v = (rng.random(n) * 0.01).astype(dtype)
            dw, dm, dv = ctx.upload(w), ctx.upload(m), ctx.upload(v)
            for t in (1, 2, 3):
                g = rng.standard_normal(n).astype(dtype)
                b1, b2 = dt(0.9), dt(0.999)
                bc1 = dt(1) - max(dt(np.power(b1, dt(t))), dt(1e-8))
                bc2 = dt(1) - max(dt(np.power(b2, dt(t))), dt(1e-8))
                w, m, v, _ = train.adam_update(w, g, m, v, dt(1e-3), b1, b2, dt(1e-8), dt(wd), bc1, bc2)
                ctx.adam_step(dw, ctx.upload(g), dm, dv, 1e-3, 0.9, 0.999, 1e-8, wd, float(bc1), float(bc2))
                assert np.array_equal(dw.numpy(), w) and np.array_equal(dm.numpy(), m) and np.array_equal(dv.numpy(), v), (n, wd, t)
    import oracle as orc
    w = rng.standard_normal(1000).astype(dtype)
    g = rng.standard_normal(1000).astype(dtype)
    dw = ctx.upload(w)
    ctx.sgd_step(dw, ctx.upload(g), 0.01)
    assert np.array_equal(dw.numpy(), orc.binary("sub", w, orc.scalar("mul_scalar", g, dt(0.01))))


@pytest.mark.parametrize("dtype", DTYPES)
def test_sgd_momentum_and_adam_amsgrad_steps_bit_exact(ctx, train, dtype):
    """fx_sgd_momentum_step (L2 weight decay, momentum, Nesterov) and fx_adam_amsgrad_step against the oracle's op-by-op
    optimizers, several steps in a row so the buffers carry over; and the buffer / momentum pairing is enforced."""
    from ferrox_amd.capi import FerroxHipError

    class One:  # the oracle optimizers update `model.params`
        def __init__(self, w):
            self.params, self.dtype = [w], np.dtype(dtype)

    rng = np.random.default_rng(77)
    dt = np.dtype(dtype).type
    for n in (1, 257, 18432):
        for mom, wd, nes in ((0.9, 0.0, False), (0.9, 5e-4, True), (0.0, 1e-2, False), (0.5, 0.1, False)):
            w = rng.standard_normal(n).astype(dtype)
            model, opt = One(w.copy()), train.SGD(0.05, mom, wd, nes)
            dw = ctx.upload(w)
            dbuf = ctx.fill((n,), 0.0, dtype) if mom != 0 else None
            for t in range(3):
                g = rng.standard_normal(n).astype(dtype)
                opt.step(model, [g])
                ctx.sgd_momentum_step(dw, ctx.upload(g), dbuf, 0.05, mom, wd, nes)
                assert np.array_equal(dw.numpy(), model.params[0]), (n, mom, wd, nes, t)
                if mom != 0:
                    assert np.array_equal(dbuf.numpy(), opt.buf[0]), (n, mom, wd, nes, t)
        for wd in (0.0, 0.01):
            w = rng.standard_normal(n).astype(dtype)
            model, opt = One(w.copy()), train.Adam(1e-3, 0.9, 0.999, 1e-8, wd, amsgrad=True)
            dw, dm, dv, dx = ctx.upload(w), ctx.fill((n,), 0.0, dtype), ctx.fill((n,), 0.0, dtype), ctx.fill((n,), 0.0, dtype)
            for t, scale in enumerate((3.0, 0.1, 1.0, 0.01), start=1):
                g = (rng.standard_normal(n) * scale).astype(dtype)
                opt.step(model, [g])
                bc1 = dt(1) - max(dt(np.power(dt(0.9), dt(t))), dt(1e-8))
                bc2 = dt(1) - max(dt(np.power(dt(0.999), dt(t))), dt(1e-8))
                ctx.adam_amsgrad_step(dw, ctx.upload(g), dm, dv, dx, 1e-3, 0.9, 0.999, 1e-8, wd, float(bc1), float(bc2))
                assert np.array_equal(dw.numpy(), model.params[0]), (n, wd, t)
                assert np.array_equal(dx.numpy(), opt.vmax[0]) and np.array_equal(dv.numpy(), opt.v[0]), (n, wd, t)
            assert np.any(opt.vmax[0] > opt.v[0])
    w = ctx.fill((8,), 1.0, dtype)
    with pytest.raises(FerroxHipError, match="momentum buffer"):
        ctx.sgd_momentum_step(w, w, None, 0.1, 0.9, 0.0, False)
    with pytest.raises(FerroxHipError, match="momentum buffer"):
        ctx.sgd_momentum_step(w, w, w, 0.1, 0.0, 0.0, False)


@pytest.mark.parametrize("dtype", DTYPES)
def test_relu_gradient_with_bias_gradient_in_one_pass(ctx, train, dtype):
    """fx_relu_bwd_bias_grad: the masked gradient has the bits of fx_relu_bwd, the channel sums agree with the oracle's
    three-axis sum and with fx_bias_grad of the masked gradient to tolerance."""
    import oracle as orc
    rng = np.random.default_rng(76)
    tol = TOL[np.dtype(dtype)]
    for shape in [(4, 3, 5, 5), (8, 32, 16, 16), (256, 10), (7, 5, 1, 3), (64, 64, 8, 8), (3, 6, 4, 4), (130, 257)]:
        g = rng.standard_normal(shape).astype(dtype)
        y = np.maximum(rng.standard_normal(shape), 0).astype(dtype)       # an activation output: zeros where it was clipped
        outer, C = shape[0], shape[1]
        inner = int(np.prod(shape[2:])) if len(shape) > 2 else 1
        dg, dy = ctx.upload(g), ctx.upload(y)
        gm, db = ctx.relu_bwd_bias_grad(dg, dy, outer, C, inner)
        want_gm = orc.binary("mul", g, orc.scalar("greater_scalar", y, dtype(0)))
        assert np.array_equal(gm.numpy(), want_gm), shape
        assert np.array_equal(gm.numpy(), ctx.relu_bwd(dg, dy).numpy()), shape
        want_db = train.bias_grad(want_gm.reshape(shape if len(shape) == 4 else shape))
        mag = np.abs(want_gm.astype(np.float64)).reshape(outer, C, inner).sum(axis=(0, 2)).max()
        assert np.abs(db.numpy() - want_db).max() <= tol * max(mag, 1e-30), shape
        assert np.abs(db.numpy() - ctx.bias_grad(gm, outer, C, inner).numpy()).max() <= tol * max(mag, 1e-30), shape


@pytest.mark.parametrize("dtype", DTYPES)
def test_multi_tensor_adam_and_sgd_equal_the_per_tensor_calls(ctx, dtype):
    """fx_adam_step_multi / fx_sgd_step_multi: one launch for a parameter list, bits of the per-tensor entry points;
    30 tensors exceed one launch's table (24), sizes include 1 and a non-multiple of the block."""
    rng = np.random.default_rng(75)
    sizes = [1, 10, 864, 32, 18432, 64, 163840, 10, 255, 256, 257] + [int(v) for v in rng.integers(1, 3000, 19)]
    arrs = lambda scale: [(rng.standard_normal(n) * scale).astype(dtype) for n in sizes]  # noqa: E731
    w, g, m = arrs(1.0), arrs(1.0), arrs(0.1)
    v = [np.abs(a) * 0.01 for a in arrs(1.0)]
    for wd in (0.0, 0.01):
        single = [[ctx.upload(a) for a in grp] for grp in (w, m, v)]
        multi = [[ctx.upload(a) for a in grp] for grp in (w, m, v)]
        dg = [ctx.upload(a) for a in g]
        for t in (1, 2):
            bc1, bc2 = 1 - 0.9 ** t, 1 - 0.999 ** t
            for i in range(len(sizes)):
                ctx.adam_step(single[0][i], dg[i], single[1][i], single[2][i], 1e-3, 0.9, 0.999, 1e-8, wd, bc1, bc2)
            ctx.adam_step_multi(multi[0], dg, multi[1], multi[2], 1e-3, 0.9, 0.999, 1e-8, wd, bc1, bc2)
            for grp_s, grp_m in zip(single, multi):
                for a, b in zip(grp_s, grp_m):
                    assert np.array_equal(a.numpy(), b.numpy()), (wd, t, a.size)
    sw, mw = [ctx.upload(a) for a in w], [ctx.upload(a) for a in w]
    dg = [ctx.upload(a) for a in g]
    for i in range(len(sizes)):
        ctx.sgd_step(sw[i], dg[i], 0.05)
    ctx.sgd_step_multi(mw, dg, 0.05)
    for a, b in zip(sw, mw):
        assert np.array_equal(a.numpy(), b.numpy()), a.size
    ctx.adam_step_multi([], [], [], [], 1e-3, 0.9, 0.999, 1e-8, 0.0, 0.1, 0.001)   # empty list: nothing to do
    ctx.sgd_step_multi([], [], 0.05)


@pytest.mark.parametrize("dtype", DTYPES)
def test_conv_and_gemm_with_bias_epilogue_equal_two_call_sequence(ctx, dtype):
    """fx_conv2d_fwd_bias_act / fx_gemm_bias_act must give the bits of fx_conv2d_fwd / fx_gemm followed by fx_bias_act,
    on every conv path (LDS-patch, implicit GEMM, strided) and on plain and split-K GEMMs."""
    from ferrox_amd import capi
    rng = np.random.default_rng(74)
    sfx = capi.dtype_code(dtype)[1]
    for (B, Cin, H, W, Cout, k, s, p) in [(2, 32, 8, 56, 96, 3, 1, 1), (2, 16, 6, 16, 40, 3, 1, 1), (3, 3, 9, 9, 8, 3, 1, 1),
                                          (2, 64, 14, 14, 130, 3, 2, 1), (2, 8, 7, 7, 5, 1, 1, 0)]:
        x = ctx.upload(rng.uniform(-1, 1, (B, Cin, H, W)).astype(dtype))
        w = ctx.upload((rng.standard_normal((Cout, Cin, k, k)) * 0.1).astype(dtype))
        b = ctx.upload(rng.standard_normal(Cout).astype(dtype))
        dims = (B, Cin, H, W, Cout, k, k, s, s, p, p)
        for act in (0, 1):
            y2 = ctx.conv2d_fwd(x, w, (s, s), (p, p))
            ctx.bias_act(y2, b, B, Cout, y2.shape[2] * y2.shape[3], act)
            y1 = ctx.empty(y2.shape, dtype)
            capi.check(getattr(capi.lib, f"fx_conv2d_fwd_bias_act_{sfx}")(ctx.h, x.ptr, w.ptr, b.ptr, y1.ptr, *dims, act, None, 0))
            assert np.array_equal(y1.numpy(), y2.numpy()), (dims, act)
    for (M, N, K, ta, tb) in [(256, 256, 784, 0, 1), (256, 10, 16384, 0, 1), (130, 70, 33, 0, 0), (512, 384, 256, 1, 0), (5, 3, 2, 0, 0)]:
        a = ctx.upload(rng.standard_normal((K, M) if ta else (M, K)).astype(dtype))
        bm = ctx.upload(rng.standard_normal((N, K) if tb else (K, N)).astype(dtype))
        bias = ctx.upload(rng.standard_normal(N).astype(dtype))
        for act in (0, 1):
            c2 = ctx.gemm(a, bm, bool(ta), bool(tb))
            ctx.bias_act(c2, bias, M, N, 1, act)
            c1 = ctx.empty((M, N), dtype)
            capi.check(getattr(capi.lib, f"fx_gemm_bias_act_{sfx}")(ctx.h, ta, tb, M, N, K, a.ptr, bm.ptr, bias.ptr, c1.ptr, act))
            assert np.array_equal(c1.numpy(), c2.numpy()), (M, N, K, ta, tb, act)


# layers whose backward has the fused kernels: (B, Cin, H, W, Cout, stride, padding); the first group are image layers (weight
# gradient only, as for a network's first layer), the second the stride-2 pair (weight and data gradient)
CONV_BWD_RELU_CASES = {
    np.float32: [
        (256, 3, 32, 32, 32, (1, 1), (1, 1)), (5, 1, 28, 28, 8, (1, 1), (1, 1)), (3, 3, 12, 16, 40, (1, 1), (1, 1)), (2, 2, 20, 8, 33, (2, 2), (1, 1)),
        (256, 32, 32, 32, 64, (2, 2), (1, 1)), (3, 32, 32, 32, 32, (2, 2), (1, 1)), (2, 64, 64, 64, 128, (2, 2), (1, 1)), (2, 32, 16, 32, 96, (2, 2), (1, 1)),
        (1, 96, 64, 64, 64, (2, 2), (1, 1)),
        # weight gradient only: the stride-2 kernel over maps 56, 28 and 16 wide
        (2, 32, 56, 56, 64, (2, 2), (1, 1)), (3, 64, 12, 56, 128, (2, 2), (1, 1)), (3, 32, 28, 28, 128, (2, 2), (1, 1)),
        (5, 32, 16, 16, 32, (2, 2), (1, 1)), (3, 64, 16, 16, 64, (2, 2), (1, 1)), (70, 32, 16, 16, 128, (2, 2), (1, 1))],
    np.float64: [
        (256, 3, 32, 32, 32, (1, 1), (1, 1)), (5, 1, 8, 32, 64, (1, 1), (1, 1)), (3, 2, 24, 32, 96, (1, 1), (1, 1)),
        (256, 32, 32, 32, 64, (2, 2), (1, 1)), (3, 32, 32, 32, 64, (2, 2), (1, 1)), (2, 64, 64, 64, 128, (2, 2), (1, 1)), (2, 32, 16, 32, 64, (2, 2), (1, 1)),
        (1, 96, 64, 64, 64, (2, 2), (1, 1)),
        (5, 32, 16, 16, 64, (2, 2), (1, 1)), (70, 64, 16, 16, 128, (2, 2), (1, 1))],
}


@pytest.mark.parametrize("dtype", DTYPES)
def test_conv_backward_from_the_unmasked_gradient(ctx, dtype):
    """fx_conv2d_wgrad_relu_bias / fx_conv2d_dgrad_relu: the ReLU mask applied while the kernels stage g.  dw and dx have the
    bits of fx_relu_bwd followed by fx_conv2d_wgrad / fx_conv2d_dgrad; db agrees with the long double sums of the masked gradient
    to the stated tolerance; a second run gives the same bits; shapes without a fused kernel are refused."""
    import parity
    from ferrox_amd import capi
    rng = np.random.default_rng(91)
    served = 0
    for (B, Cin, H, W, Cout, st, pd) in CONV_BWD_RELU_CASES[dtype]:
        case = (B, Cin, H, W, Cout, st, pd)
        oh, ow = (H + 2 * pd[0] - 3) // st[0] + 1, (W + 2 * pd[1] - 3) // st[1] + 1
        x = rng.uniform(-1, 1, (B, Cin, H, W)).astype(dtype)
        w = (rng.standard_normal((Cout, Cin, 3, 3)) * np.sqrt(2.0 / (Cin * 9))).astype(dtype)
        g = rng.standard_normal((B, Cout, oh, ow)).astype(dtype)
        act = np.maximum(rng.standard_normal((B, Cout, oh, ow)), 0).astype(dtype)
        dx_, dw_, dg_, da_ = ctx.upload(x), ctx.upload(w), ctx.upload(g), ctx.upload(act)
        assert ctx.conv2d_bwd_relu_supported(capi.CONV_WGRAD, dtype, x.shape, w.shape, st, pd), case
        gm = ctx.relu_bwd(dg_, da_)
        want_dw = ctx.conv2d_wgrad(dx_, gm, w.shape, st, pd).numpy()
        dw, db = ctx.conv2d_wgrad_relu_bias(dx_, dg_, da_, w.shape, st, pd)
        assert np.array_equal(dw.numpy(), want_dw), ("dw", case)
        masked = g.astype(np.longdouble) * (act > 0)
        parity.check("conv bwd from unmasked g: bias grad", db.numpy(), masked.sum(axis=(0, 2, 3)), case=case,
                     oracle=ctx.bias_grad(gm, B, Cout, oh * ow).numpy(), terms=float(np.abs(masked).sum(axis=(0, 2, 3)).max()))
        dw2, db2 = ctx.conv2d_wgrad_relu_bias(dx_, dg_, da_, w.shape, st, pd)
        assert np.array_equal(dw2.numpy(), dw.numpy()) and np.array_equal(db2.numpy(), db.numpy()), ("rerun", case)
        if ctx.conv2d_bwd_relu_supported(capi.CONV_DGRAD, dtype, x.shape, w.shape, st, pd):
            served += 1
            want_dx = ctx.conv2d_dgrad(gm, dw_, x.shape, st, pd).numpy()
            got_dx = ctx.conv2d_dgrad_relu(dg_, da_, dw_, x.shape, st, pd).numpy()
            assert np.array_equal(got_dx, want_dx), ("dx", case)
    assert served >= 4
    # no fused kernel: a stride-1 layer over many channels
    x_shape, w_shape = (2, 64, 16, 16), (64, 64, 3, 3)
    assert not ctx.conv2d_bwd_relu_supported(capi.CONV_WGRAD, dtype, x_shape, w_shape, (1, 1), (1, 1))
    assert not ctx.conv2d_bwd_relu_supported(capi.CONV_DGRAD, dtype, x_shape, w_shape, (1, 1), (1, 1))
    z = ctx.fill(x_shape, 0.0, dtype)
    with pytest.raises(capi.FerroxHipError) as e:
        ctx.conv2d_wgrad_relu_bias(z, z, z, w_shape, (1, 1), (1, 1))
    assert e.value.code == 4
    with pytest.raises(capi.FerroxHipError) as e:
        ctx.conv2d_dgrad_relu(z, z, ctx.fill(w_shape, 0.0, dtype), x_shape, (1, 1), (1, 1))
    assert e.value.code == 4
