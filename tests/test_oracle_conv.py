"""Pins the CPU oracle's convolution path: reference-held vectors, closed forms, brute force, and
torch's CPU conv2d/autograd as the independent textbook routine.  No GPU needed."""
import itertools

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle as orc


def brute_im2col(x, k, s, p):
    """Independent definition: col[(c,ky,kx),(b,oy,ox)] = xpad[b,c,oy*s+ky,ox*s+kx]."""
    B, C, H, W = x.shape
    (kh, kw), (sh, sw), (ph, pw) = k, s, p
    xp = np.zeros((B, C, H + 2 * ph, W + 2 * pw), x.dtype)
    xp[:, :, ph:ph + H, pw:pw + W] = x
    oh, ow = orc.out_hw(H, W, kh, kw, sh, sw, ph, pw)
    col = np.zeros((C, kh, kw, B, oh, ow), x.dtype)
    for ky in range(kh):
        for kx in range(kw):
            col[:, ky, kx] = xp[:, :, ky:ky + sh * oh:sh, kx:kx + sw * ow:sw].transpose(1, 0, 2, 3)
    return col.reshape(C * kh * kw, B * oh * ow)


SHAPES = [(B, C, H, W, k, s, p) for B in (1, 2, 3) for C in (1, 3) for (H, W) in ((4, 4), (5, 6), (6, 3))
          for k in (1, 2, 3) for s in (1, 2) for p in (0, 1) if H + 2 * p >= k and W + 2 * p >= k]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_im2col_brute_force(dtype):
    rng = np.random.default_rng(0)
    for (B, C, H, W, k, s, p) in SHAPES:
        x = rng.uniform(-1, 1, (B, C, H, W)).astype(dtype)
        got = orc.im2col(x, (k, k), (s, s), (p, p))
        assert np.array_equal(got, brute_im2col(x, (k, k), (s, s), (p, p))), (B, C, H, W, k, s, p)


def test_im2col_rect_kernel_and_stride():
    rng = np.random.default_rng(1)
    x = rng.uniform(-1, 1, (2, 2, 7, 5)).astype(np.float32)
    for k, s, p in [((3, 2), (2, 1), (1, 0)), ((1, 3), (1, 2), (0, 1)), ((2, 2), (1, 1), (2, 2))]:
        assert np.array_equal(orc.im2col(x, k, s, p), brute_im2col(x, k, s, p))


def test_im2col_sum_identity():
    """sum(col) == sum over windows of x: each pixel counted once per window covering it (integers -> exact)."""
    rng = np.random.default_rng(2)
    x = rng.integers(-5, 6, (2, 3, 6, 6)).astype(np.float64)
    col = orc.im2col(x, (3, 3), (1, 1), (1, 1))
    cover = orc.col2im(np.ones_like(col), x.shape, (3, 3), (1, 1), (1, 1), 0)
    assert col.sum() == (x * cover).sum()


@pytest.mark.parametrize("layout", [0, 1])
def test_col2im_of_im2col_counts_windows_batch1(layout):
    """For batch 1 both column layouts coincide and col2im(im2col(x)) = x * (#windows covering the pixel)."""
    rng = np.random.default_rng(3)
    x = rng.integers(-4, 5, (1, 2, 5, 5)).astype(np.float32)
    for k, s, p in [(3, 1, 1), (2, 2, 0), (3, 2, 1)]:
        col = orc.im2col(x, (k, k), (s, s), (p, p))
        back = orc.col2im(col, x.shape, (k, k), (s, s), (p, p), layout)
        ones = torch.ones(1, 1, 5, 5, dtype=torch.float64)
        cnt = F.fold(F.unfold(ones, k, padding=p, stride=s), (5, 5), k, padding=p, stride=s)[0, 0].numpy()
        assert np.array_equal(back, x * cnt.astype(np.float32))


def test_col2im_layout0_matches_torch_fold():
    rng = np.random.default_rng(4)
    B, C, H, W, k, s, p = 3, 2, 6, 5, 3, 1, 1
    oh, ow = orc.out_hw(H, W, k, k, s, s, p, p)
    col = rng.integers(-3, 4, (C * k * k, B * oh * ow)).astype(np.float64)
    got = orc.col2im(col, (B, C, H, W), (k, k), (s, s), (p, p), 0)
    t = torch.from_numpy(col.reshape(C * k * k, B, oh * ow).transpose(1, 0, 2).copy())
    ref = F.fold(t, (H, W), k, padding=p, stride=s).numpy()
    assert np.array_equal(got, ref)


def test_col2im_literal_is_batch_major_read():
    """layout 1 on a [CKK, B*L] buffer equals layout 0 on the same buffer reinterpreted as [B, CKK, L]."""
    rng = np.random.default_rng(5)
    B, C, H, W, k, s, p = 2, 2, 4, 4, 3, 1, 1
    L = 16
    flat = rng.integers(-3, 4, (C * k * k * B * L,)).astype(np.float32)
    lit = orc.col2im(flat, (B, C, H, W), (k, k), (s, s), (p, p), 1)
    as_rowmajor = flat.reshape(B, C * k * k, L).transpose(1, 0, 2).reshape(C * k * k, B * L)
    assert np.array_equal(lit, orc.col2im(as_rowmajor, (B, C, H, W), (k, k), (s, s), (p, p), 0))


def test_conv2d_reference_vectors(golden):
    for key in ("conv2d_test", "conv2d_simple_forward", "conv2d_edge_cases"):
        g = golden[key]
        x = np.array(g["x"], np.float32).reshape(g["x_shape"])
        w = np.array(g["w"], np.float32).reshape(g["w_shape"])
        y = orc.conv2d_fwd(x, w, tuple(g["stride"]), tuple(g["padding"]))
        assert list(y.shape) == g["y_shape"]
        np.testing.assert_allclose(y.ravel(), np.array(g["y"], np.float32), atol=g["tol"], rtol=0)


CONV_CASES = [  # B, Cin, H, W, Cout, k, s, p
    (1, 1, 5, 5, 1, 3, 1, 1), (2, 3, 8, 8, 4, 3, 1, 1), (3, 2, 9, 7, 5, 3, 2, 1), (2, 4, 6, 6, 3, 1, 1, 0),
    (4, 1, 28, 28, 8, 3, 1, 1), (2, 3, 7, 7, 2, 2, 2, 0),
]


@pytest.mark.parametrize("dtype,tol", [(np.float32, 1e-5), (np.float64, 1e-12)])
def test_conv2d_fwd_and_correct_grads_vs_torch(dtype, tol):
    rng = np.random.default_rng(6)
    for (B, Cin, H, W, Cout, k, s, p) in CONV_CASES:
        x = rng.uniform(-1, 1, (B, Cin, H, W)).astype(dtype)
        w = (rng.standard_normal((Cout, Cin, k, k)) * np.sqrt(2.0 / (Cin * k * k))).astype(dtype)
        tx = torch.from_numpy(x).double().requires_grad_(True)
        tw = torch.from_numpy(w).double().requires_grad_(True)
        ty = F.conv2d(tx, tw, stride=s, padding=p)
        g = rng.standard_normal(ty.shape).astype(dtype)
        ty.backward(torch.from_numpy(g).double())
        y = orc.conv2d_fwd(x, w, (s, s), (p, p))
        dx = orc.conv2d_dgrad(g, w, x.shape, (s, s), (p, p), 0)
        dw = orc.conv2d_wgrad(x, g, w.shape, (s, s), (p, p), 0)
        for got, ref in ((y, ty.detach()), (dx, tx.grad), (dw, tw.grad)):
            ref = ref.numpy()
            assert np.abs(got - ref).max() <= tol * max(1.0, np.abs(ref).max()), (B, Cin, H, W, Cout, k, s, p)


def test_literal_grads_equal_correct_for_batch1_and_differ_for_batch2():
    rng = np.random.default_rng(7)
    for B, expect_equal in ((1, True), (2, False)):
        x = rng.uniform(-1, 1, (B, 2, 5, 5))
        w = rng.standard_normal((3, 2, 3, 3))
        g = rng.standard_normal((B, 3, 5, 5))
        dx0, dx1 = (orc.conv2d_dgrad(g, w, x.shape, (1, 1), (1, 1), m) for m in (0, 1))
        dw0, dw1 = (orc.conv2d_wgrad(x, g, w.shape, (1, 1), (1, 1), m) for m in (0, 1))
        if expect_equal:
            np.testing.assert_allclose(dx1, dx0, rtol=0, atol=1e-13)
            np.testing.assert_allclose(dw1, dw0, rtol=0, atol=1e-13)
        else:
            assert np.abs(dx1 - dx0).max() > 1e-2 and np.abs(dw1 - dw0).max() > 1e-2


def test_conv1d_analogue_vector_from_dev_notes():
    """The 1-D PyTorch vector held in CUDA_DEVELOPMENT.md:236-262, expressed as a 1xW conv2d:
    x = [10,4,6,5,4], w = [1,0.5,-1] -> y = [6,2,4.5]; with loss = sum(y): dx = [1,1.5,.5,-.5,-1], dw = [20,15,15]."""
    x = np.array([10, 4, 6, 5, 4], np.float64).reshape(1, 1, 1, 5)
    w = np.array([1, 0.5, -1], np.float64).reshape(1, 1, 1, 3)
    g = np.ones((1, 1, 1, 3))
    assert orc.conv2d_fwd(x, w, (1, 1), (0, 0)).ravel().tolist() == [6.0, 2.0, 4.5]
    for mode in (0, 1):  # batch 1: literal and correct modes must agree
        assert orc.conv2d_wgrad(x, g, w.shape, (1, 1), (0, 0), mode).ravel().tolist() == [20.0, 15.0, 15.0]
        assert orc.conv2d_dgrad(g, w, x.shape, (1, 1), (0, 0), mode).ravel().tolist() == [1.0, 1.5, 0.5, -0.5, -1.0]


LITERAL_CASES = [  # B, Cin, H, W, Cout, k, s, p
    (2, 2, 5, 5, 3, 3, 1, 1), (3, 3, 8, 6, 4, 3, 1, 1), (2, 3, 9, 7, 5, 3, 2, 1), (3, 1, 7, 7, 2, 2, 2, 0),
    (2, 4, 6, 6, 3, 1, 1, 0), (4, 1, 28, 28, 8, 3, 1, 1),
]


@pytest.mark.parametrize("case", LITERAL_CASES)
def test_literal_grads_batch_gt1_vs_composed_torch_and_numpy(case):
    """The CPU backend's literal gradients for batch > 1, rebuilt from independent routines.

    Only the two flat reinterpretations are taken from the reference: grad_output [B, OC, oh, ow] is re-read as a
    row-major [OC, B*L] matrix (convolutions.rs:292-293, 323-326) and the column matrix [C*kh*kw, B*L] produced by the
    product is re-read by col2im with a batch-major flat index, i.e. as [B, C*kh*kw, L] (convolutions.rs:122-127).
    Everything else is numpy's float64 matmul and torch's unfold / fold.  A wrong stride, a transposed operand or a
    channel-major read of the column matrix fails this comparison (the last check below makes sure the literal result
    is NOT the mathematical gradient, so the test cannot pass by accident through the correct path)."""
    B, Cin, H, W, Cout, k, s, p = case
    rng = np.random.default_rng(100 + B * 7 + Cin)
    x = rng.uniform(-1, 1, (B, Cin, H, W))
    w = rng.standard_normal((Cout, Cin, k, k)) * np.sqrt(2.0 / (Cin * k * k))
    oh, ow = orc.out_hw(H, W, k, k, s, s, p, p)
    L = oh * ow
    g = rng.standard_normal((B, Cout, oh, ow))
    g2d = g.reshape(Cout, B * L)                      # the flat reinterpretation
    w2d = w.reshape(Cout, Cin * k * k)

    # weight gradient: g2d . im2col(x)^T, with torch.unfold as the independent im2col
    unf = F.unfold(torch.from_numpy(x), k, padding=p, stride=s).numpy()        # [B, CKK, L]
    col = unf.transpose(1, 0, 2).reshape(Cin * k * k, B * L)                    # [CKK, (b, l)]
    dw_ref = (g2d @ col.T).reshape(w.shape)
    dw = orc.conv2d_wgrad(x, g, w.shape, (s, s), (p, p), 1)
    np.testing.assert_allclose(dw, dw_ref, rtol=0, atol=1e-12 * max(1.0, np.abs(dw_ref).max()))

    # data gradient: fold of (w2d^T . g2d) re-read batch-major
    colm = (w2d.T @ g2d).reshape(-1)                                            # row-major [CKK, B*L], flattened
    dx_ref = F.fold(torch.from_numpy(colm.reshape(B, Cin * k * k, L).copy()), (H, W), k, padding=p, stride=s).numpy()
    dx = orc.conv2d_dgrad(g, w, x.shape, (s, s), (p, p), 1)
    np.testing.assert_allclose(dx, dx_ref, rtol=0, atol=1e-12 * max(1.0, np.abs(dx_ref).max()))

    # float32 follows the same path within its own rounding
    dw32 = orc.conv2d_wgrad(x.astype(np.float32), g.astype(np.float32), w.shape, (s, s), (p, p), 1)
    dx32 = orc.conv2d_dgrad(g.astype(np.float32), w.astype(np.float32), x.shape, (s, s), (p, p), 1)
    assert np.abs(dw32 - dw_ref).max() <= 1e-5 * max(1.0, np.abs(dw_ref).max())
    assert np.abs(dx32 - dx_ref).max() <= 1e-5 * max(1.0, np.abs(dx_ref).max())

    # and it is not the mathematical gradient (batch > 1), so the literal path really is a different function
    if Cout > 1:
        assert np.abs(dw - orc.conv2d_wgrad(x, g, w.shape, (s, s), (p, p), 0)).max() > 1e-3
    assert np.abs(dx - orc.conv2d_dgrad(g, w, x.shape, (s, s), (p, p), 0)).max() > 1e-3


def test_literal_wgrad_equals_correct_for_one_output_channel():
    """With Cout = 1 the flat [OC, B*L] re-read of grad_output is the identity, so the literal weight gradient is the
    mathematical one for any batch (torch.autograd as the independent value)."""
    rng = np.random.default_rng(9)
    x = rng.uniform(-1, 1, (3, 2, 6, 6))
    w = rng.standard_normal((1, 2, 3, 3))
    tx, tw = torch.from_numpy(x), torch.from_numpy(w).requires_grad_(True)
    ty = F.conv2d(tx, tw, stride=1, padding=1)
    g = rng.standard_normal(tuple(ty.shape))
    ty.backward(torch.from_numpy(g))
    dw = orc.conv2d_wgrad(x, g, w.shape, (1, 1), (1, 1), 1)
    np.testing.assert_allclose(dw, tw.grad.numpy(), rtol=0, atol=1e-12)
