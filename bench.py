#!/usr/bin/env python3
"""Benchmark of the Ferrox-on-MI355X hot path.  Prints ONE JSON line.

Primary workload (config C3 of BASELINE.json): a single Conv2d layer, f32, input N=128, C_in=64, 56x56, U(-1,1);
C_out=128, 3x3, stride 1, pad 1, Kaiming-normal weights; upstream gradient N(0,1).  One "step" is one forward +
one data-gradient + one weight-gradient pass.  `value` is the conv fwd+bwd throughput in TFLOP/s, counting the
algorithmic 2*Cout*(Cin*kh*kw)*(B*oh*ow) FLOP per pass, with all tensors resident in HBM before timing starts.

Also measured in the same run and reported under "also": the bandwidth kernels of config C4 (sum/mean/max over
axis 0, axis 1 and all elements of [8192,8192] f32 and f64; add/mul and ReLU/sigmoid/tanh backward on 2^28 f32).

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--skip-cpu] [--skip-also] [--skip-train]
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_F32_MFMA_TFLOPS = 157.3
PEAK_F64_MFMA_TFLOPS = 78.6
PEAK_HBM_GBS = 8000.0

C3 = dict(B=128, Cin=64, H=56, W=56, Cout=128, k=3, s=1, p=1)
PRIMING_STEPS = 20  # untimed steps before the `--warmup` steps of the headline measurement


def time_stream(ctx, fn, iters, warmup):
    """Average milliseconds per call of fn, measured with HIP events on the stream the kernels run on."""
    for _ in range(warmup):
        fn()
    ctx.sync()
    ctx.timer_start()
    for _ in range(iters):
        fn()
    return ctx.timer_stop() / iters


CONV_KERNELS = {"fwd": "cpk::conv_patch_persist_kernel (conv fwd pass)", "dgrad": "cpk::conv_patch_persist_kernel (conv dgrad pass)",
                "wgrad": "wgp::wgrad_patch_kernel + wgrad_patch_reduce_vec_kernel (conv wgrad pass)"}


def profile_traffic(path, row):
    """HBM-side bytes per launch of a kernel from a committed rocprofv3 counter summary under profiles/: the row that
    starts with `row`, column "total MB" (FETCH_SIZE + WRITE_SIZE per dispatch, each scaled by what the same counter reads
    for a streaming kernel of known size; the file states the commands and the factors).  Returns (bytes or None, source
    label with the file's content hash, so a line can be traced to the summary it was taken from)."""
    import hashlib
    full = os.path.join(ROOT, path)
    try:
        text = open(full).read()
    except OSError:
        return None, f"{path} (missing)"
    label = f"{path} sha1:{hashlib.sha1(text.encode()).hexdigest()[:12]}"
    header = None
    for line in text.splitlines():
        cells = [c.strip() for c in line.split("|")]
        if len(cells) < 3:
            continue
        if "total MB" in cells:
            header = cells
        elif header and cells[0] == row and len(cells) == len(header):
            try:
                return float(cells[header.index("total MB")]) * 1e6, label
            except ValueError:
                return None, label
    return None, label


CONV_C3_TRAFFIC_FILE = "profiles/conv_c3_f32_hbm_traffic.txt"
C4_TRAFFIC_FILE = "profiles/c4_bandwidth_kernels_hbm_traffic.txt"


def bench_conv(ctx, steps, warmup, dtype=np.float32, B=None):
    c = dict(C3)
    if B is not None:
        c["B"] = B
    B, Cin, H, W, Cout, k, s, p = (c[n] for n in ("B", "Cin", "H", "W", "Cout", "k", "s", "p"))
    x = ctx.uniform((B, Cin, H, W), 3, -1.0, 1.0, dtype)
    w = ctx.normal((Cout, Cin, k, k), 33, 0.0, (2.0 / (Cin * k * k)) ** 0.5, dtype)
    g = ctx.normal((B, Cout, H, W), 333, 0.0, 1.0, dtype)
    y = ctx.empty((B, Cout, H, W), dtype)
    dx = ctx.empty(x.shape, dtype)
    dw = ctx.empty(w.shape, dtype)
    flop = 2.0 * Cout * Cin * k * k * B * H * W
    passes = {
        "fwd": lambda: ctx.conv2d_fwd(x, w, (s, s), (p, p), out=y),
        "dgrad": lambda: ctx.conv2d_dgrad(g, w, x.shape, (s, s), (p, p), out=dx),
        "wgrad": lambda: ctx.conv2d_wgrad(x, g, w.shape, (s, s), (p, p), out=dw),
    }
    def step():
        for fn in passes.values():
            fn()

    # Clocks and caches settle over the first few tens of milliseconds of MFMA load; these priming steps are untimed
    # and come on top of the `warmup` steps of the contract (reported as "priming_steps" in the output line).
    for _ in range(PRIMING_STEPS):
        step()
    # the timed region of the headline number: exactly `steps` steps between two synchronisations
    for _ in range(warmup):
        step()
    ctx.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    ctx.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    # per-pass durations with HIP events on the library's stream (each pass = its main kernel + its small helper:
    # the weight-image build for fwd/dgrad, the ordered split-K sum for wgrad)
    per_pass = {}
    for name, fn in passes.items():
        ms = time_stream(ctx, fn, steps, warmup)
        per_pass[name] = {"ms": ms, "tflops": flop / ms / 1e9, "kernel_family": ctx.conv2d_last_path()}
    res = {"flop_per_pass": flop, "per_pass": per_pass, "ms_per_step": wall_ms, "tflops": 3 * flop / wall_ms / 1e9}
    if dtype == np.float32 and B == C3["B"]:
        # forward + bias + ReLU: in the conv kernel's store (one pass over y) vs conv, then an in-place bias/ReLU pass
        from ferrox_amd import capi
        bias = ctx.normal((Cout,), 34, 0.0, 0.1, dtype)
        dims = (B, Cin, H, W, Cout, k, k, s, s, p, p)
        fused = lambda: capi.check(capi.lib.fx_conv2d_fwd_bias_act_f32(ctx.h, x.ptr, w.ptr, bias.ptr, y.ptr, *dims, 1, None, 0))  # noqa: E731
        two = lambda: (ctx.conv2d_fwd(x, w, (s, s), (p, p), out=y), ctx.bias_act(y, bias, B, Cout, H * W, 1))  # noqa: E731
        res["fwd_bias_relu"] = {"epilogue_ms": time_stream(ctx, fused, steps, warmup), "two_call_ms": time_stream(ctx, two, steps, warmup)}
    return res


REDUCE_VIEWS = (("0", (1, 8192, 8192)), ("1", (8192, 8192, 1)), ("all", (1, 8192 * 8192, 1)))
ROTATE = 4  # distinct inputs a reduction cycles through: 4 x 256 MiB (f32) can not stay in the 256 MiB last-level cache


def c4_reduction_cases(ctx, dtype, rotate):
    """The nine reductions of config C4 on [8192, 8192] of one dtype: (name, algorithmic bytes, call) where call(j) reduces
    input j % rotate.  Algorithmic bytes = sizeof(T) * (8192^2 + outputs) + 8 * outputs for the int64 argmax indices."""
    import ctypes  # noqa: F401
    from ferrox_amd import capi
    sfx = capi.dtype_code(dtype)[1]
    ins = [ctx.normal((8192, 8192), 4 + j, 0.0, 1.0, dtype) for j in range(rotate)]
    res = ctx.empty((8192,), dtype)
    idx = ctx.empty((8192,), np.float64)  # int64 argmax indices (8 bytes each)
    cases = []
    for kind in ("sum", "mean", "max"):
        for axis, view in REDUCE_VIEWS:
            n_out = view[0] * view[2]
            if kind == "max":
                f = getattr(capi.lib, f"fx_reduce_max_{sfx}")
                call = lambda j, f=f, view=view: capi.check(f(ctx.h, ins[j % rotate].ptr, res.ptr, idx.ptr, *view))  # noqa: E731
                nbytes = ins[0].dtype.itemsize * (ins[0].size + n_out) + 8 * n_out
            else:
                f = getattr(capi.lib, f"fx_reduce_{kind}_{sfx}")
                call = lambda j, f=f, view=view: capi.check(f(ctx.h, ins[j % rotate].ptr, res.ptr, *view))  # noqa: E731
                nbytes = ins[0].dtype.itemsize * (ins[0].size + n_out)
            cases.append((f"{kind}_axis{axis}_{sfx}", nbytes, call))
    return cases, (ins, res, idx)


def c4_elementwise_cases(ctx):
    """add / mul and the fused ReLU / sigmoid / tanh gradients on 2^28 f32: 3 arrays of 1 GiB per call."""
    n = 1 << 28
    g = ctx.uniform((n,), 7, -4.0, 4.0)
    x = ctx.uniform((n,), 8, -4.0, 4.0)
    s = ctx.unary("sigmoid", x)
    t = ctx.unary("tanh", x)
    o = ctx.empty((n,))
    cases = [
        ("add_f32", 3 * 4 * n, lambda j: ctx.binary("add", g, x, out=o)),
        ("mul_f32", 3 * 4 * n, lambda j: ctx.binary("mul", g, x, out=o)),
        ("relu_bwd_f32", 3 * 4 * n, lambda j: ctx.relu_bwd(g, x, out=o)),
        ("sigmoid_bwd_f32", 3 * 4 * n, lambda j: ctx.sigmoid_bwd(g, s, 0, out=o)),
        ("tanh_bwd_f32", 3 * 4 * n, lambda j: ctx.tanh_bwd(g, t, out=o)),
    ]
    return cases, (g, x, s, t, o)


def time_cycling(ctx, call, iters, warmup, rotate=1):
    """Average ms per call; call(j) receives a running index so that consecutive calls may take different inputs."""
    k = [0]

    def fn():
        call(k[0])
        k[0] += 1
    return time_stream(ctx, fn, iters, warmup)


def bench_c4_profile(ctx, iters=4):
    """Profiler mode: every C4 kernel `iters` times on rotating inputs, cases separated by a one-element fill (a marker
    dispatch a counter trace can be split on).  Prints the order of the cases."""
    from ferrox_amd import capi
    marker = ctx.empty((1,))
    order = []

    def run_case(name, nbytes, call):
        capi.check(capi.lib.fx_fill_f32(ctx.h, marker.ptr, float(len(order)), 1))
        for j in range(iters):
            call(j)
        order.append({"case": name, "algorithmic_bytes": nbytes, "calls": iters})

    for dtype in (np.float32, np.float64):
        cases, keep = c4_reduction_cases(ctx, dtype, ROTATE)
        for c in cases:
            run_case(*c)
        ctx.sync()
        del cases, keep
    cases, keep = c4_elementwise_cases(ctx)
    for c in cases:
        run_case(*c)
    capi.check(capi.lib.fx_fill_f32(ctx.h, marker.ptr, -1.0, 1))
    ctx.sync()
    return order


def bench_bandwidth(ctx, iters=20, warmup=3):
    import ctypes
    from ferrox_amd import capi
    C_i64 = ctypes.c_int64
    out = {"reductions": {}, "elementwise": {}, "pooling": {}}
    # Reductions: `us_same_input` re-reads one buffer (an 8192^2 f32 matrix is exactly the size of the 256 MiB last-level
    # cache, so part of it is served from there); `us` cycles through ROTATE distinct inputs, which no cache can hold:
    # that is the figure quoted against the HBM peak.
    for dtype in (np.float32, np.float64):
        cases, keep = c4_reduction_cases(ctx, dtype, ROTATE)
        for name, nbytes, call in cases:
            same = time_cycling(ctx, lambda j: call(0), iters, warmup)
            ms = time_cycling(ctx, call, iters, warmup + ROTATE)
            out["reductions"][name] = {"us": ms * 1e3, "GBps": nbytes / ms / 1e6, "frac_hbm": nbytes / ms / 1e6 / PEAK_HBM_GBS,
                                       "us_same_input": same * 1e3, "GBps_same_input": nbytes / same / 1e6,
                                       "algorithmic_bytes": nbytes, "inputs_cycled": ROTATE}
        del cases, keep
    cases, keep = c4_elementwise_cases(ctx)
    for name, nbytes, call in cases:
        ms = time_cycling(ctx, call, 10, 2)
        out["elementwise"][name] = {"ms": ms, "GBps": nbytes / ms / 1e6, "frac_hbm": nbytes / ms / 1e6 / PEAK_HBM_GBS,
                                    "algorithmic_bytes": nbytes}
    del cases, keep
    n = 1 << 28
    # pooling and its gradient on [128, 64, 112, 112] f32, 2x2 stride 2: algorithmic bytes = input + output (forward),
    # grad_out + input + pooled + grad_in (max gradient), grad_out + grad_in (avg gradient)
    pshape, k2 = (128, 64, 112, 112), ((2, 2), (2, 2), (0, 0))
    px = ctx.uniform(pshape, 9, -1.0, 1.0)
    n_in, n_out = px.size, px.size // 4
    out["pooling"] = {}
    for name, is_max in (("maxpool2d", True), ("avgpool2d", False)):
        pooled = ctx.pool2d(px, *k2, is_max)
        pg = ctx.uniform(pooled.shape, 10, -1.0, 1.0)
        ms = time_stream(ctx, lambda: ctx.pool2d(px, *k2, is_max), 10, 2)
        nbytes = 4 * (n_in + n_out)
        out["pooling"][f"{name}_f32"] = {"ms": ms, "GBps": nbytes / ms / 1e6, "frac_hbm": nbytes / ms / 1e6 / PEAK_HBM_GBS}
        ms = time_stream(ctx, lambda: ctx.unpool2d(pg, px, pooled, *k2, is_max), 10, 2)
        nbytes = 4 * ((2 * n_in + 2 * n_out) if is_max else (n_in + n_out))
        out["pooling"][f"{name}_grad_f32"] = {"ms": ms, "GBps": nbytes / ms / 1e6, "frac_hbm": nbytes / ms / 1e6 / PEAK_HBM_GBS}
        del pooled, pg
    del px
    # BatchNorm on [256, 128, 56, 56] f32 (411 MB per array, larger than the last-level cache) and dropout on 2^28:
    # algorithmic bytes = x (statistics), x + y (forward), 2 reads of (dy, x) + dx (backward), x + mask + y (dropout)
    out["normalisation"] = {}
    bshape = (256, 128, 56, 56)
    bx = ctx.normal(bshape, 13, 0.5, 2.0)
    bg = ctx.normal(bshape, 14, 0.0, 1.0)
    gamma, beta = ctx.fill((128,), 1.0), ctx.fill((128,), 0.0)
    mean, var = ctx.batchnorm_stats(bx)
    by, bdx, dgm, dbt = ctx.empty(bshape), ctx.empty(bshape), ctx.empty((128,)), ctx.empty((128,))
    view = (256, 128, 56 * 56)
    bn_cases = {
        "batchnorm_stats": (1, lambda: capi.check(capi.lib.fx_batchnorm_stats_f32(ctx.h, bx.ptr, mean.ptr, var.ptr, None, None, 0.1, *view))),
        "batchnorm_fwd": (2, lambda: capi.check(capi.lib.fx_batchnorm_fwd_f32(ctx.h, bx.ptr, mean.ptr, var.ptr, gamma.ptr, beta.ptr,
                                                                            1e-5, by.ptr, *view, 0))),
        "batchnorm_bwd": (5, lambda: capi.check(capi.lib.fx_batchnorm_bwd_f32(ctx.h, bg.ptr, bx.ptr, None, mean.ptr, var.ptr, gamma.ptr, 1e-5,
                                                                            bdx.ptr, dgm.ptr, dbt.ptr, *view, 1))),
    }
    for name, (passes, fn) in bn_cases.items():
        ms = time_stream(ctx, fn, 10, 2)
        nbytes = passes * 4 * bx.size
        out["normalisation"][f"{name}_f32"] = {"ms": ms, "GBps": nbytes / ms / 1e6, "frac_hbm": nbytes / ms / 1e6 / PEAK_HBM_GBS}
    del bx, bg, by, bdx
    dxx = ctx.uniform((n,), 15, -1.0, 1.0)
    dm, dy_ = ctx.empty((n,)), ctx.empty((n,))
    ms = time_stream(ctx, lambda: capi.check(capi.lib.fx_dropout_f32(ctx.h, dxx.ptr, dm.ptr, dy_.ptr, n, 0.3, 99)), 10, 2)
    out["normalisation"]["dropout_f32"] = {"ms": ms, "GBps": 3 * 4 * n / ms / 1e6, "frac_hbm": 3 * 4 * n / ms / 1e6 / PEAK_HBM_GBS}
    del dxx, dm, dy_
    # explicit im2col / col2im (the reference's convolution path materialises the column matrix; here they exist for
    # parity and for callers that want the matrix) at the second conv layer of the CNN configuration, and the two
    # materialisations the layers issue most: a channel bias broadcast to [N,C,H,W] and a 2-D transpose.
    # Algorithmic bytes: column matrix + image (im2col, col2im); output (+ the small input) for the broadcast; 2 arrays.
    out["data_movement"] = {}
    ishape = (256, 32, 32, 32)
    ix = ctx.uniform(ishape, 16, -1.0, 1.0)
    col = ctx.im2col(ix, (3, 3), (2, 2), (1, 1))
    dims = (256, 32, 32, 32, 3, 3, 2, 2, 1, 1)
    back = ctx.empty(ishape)
    dm_cases = {
        "im2col_c5_conv2": (4 * (col.size + ix.size), lambda: capi.check(capi.lib.fx_im2col_f32(ctx.h, ix.ptr, col.ptr, *dims))),
        "col2im_c5_conv2": (4 * (col.size + ix.size), lambda: capi.check(capi.lib.fx_col2im_f32(ctx.h, col.ptr, back.ptr, *dims, 0))),
    }
    bias = ctx.uniform((128,), 17, -1.0, 1.0)
    bshape2 = (256, 128, 56, 56)
    bout = ctx.empty(bshape2)
    sh4, st4 = (C_i64 * 4)(*bshape2), (C_i64 * 4)(0, 1, 0, 0)
    dm_cases["broadcast_bias_to_nchw"] = (4 * bout.size, lambda: capi.check(capi.lib.fx_materialize_f32(ctx.h, bias.ptr, bout.ptr, sh4, st4, 4, bout.size)))
    tin = ctx.uniform((8192, 8192), 18, -1.0, 1.0)
    tout = ctx.empty((8192, 8192))
    sh2, st2 = (C_i64 * 2)(8192, 8192), (C_i64 * 2)(1, 8192)
    dm_cases["transpose_8192x8192"] = (2 * 4 * tin.size, lambda: capi.check(capi.lib.fx_materialize_f32(ctx.h, tin.ptr, tout.ptr, sh2, st2, 2, tin.size)))
    for name, (nbytes, fn) in dm_cases.items():
        ms = time_stream(ctx, fn, 10, 2)
        out["data_movement"][f"{name}_f32"] = {"ms": ms, "GBps": nbytes / ms / 1e6, "frac_hbm": nbytes / ms / 1e6 / PEAK_HBM_GBS}
    del ix, col, back, bias, bout, tin, tout
    # GEMMs of the MLP / CNN configurations (forward and the two backward products) and one large square product
    out["gemm"] = {}
    for name, (M, N, K, ta, tb) in {"c2_fc1_fwd": (256, 256, 784, 0, 1), "c2_fc1_dx": (256, 784, 256, 0, 0), "c2_fc1_dw": (256, 784, 256, 1, 0),
                                    "c5_fc_fwd": (256, 10, 16384, 0, 1), "c5_fc_dw": (10, 16384, 256, 1, 0),
                                    "square_4096": (4096, 4096, 4096, 0, 0)}.items():
        for dtype in (np.float32, np.float64):
            sfx = capi.dtype_code(dtype)[1]
            a = ctx.uniform((K, M) if ta else (M, K), 19, -1.0, 1.0, dtype)
            b = ctx.uniform((N, K) if tb else (K, N), 20, -1.0, 1.0, dtype)
            c = ctx.empty((M, N), dtype)
            fn = lambda: capi.check(getattr(capi.lib, f"fx_gemm_{sfx}")(ctx.h, ta, tb, M, N, K, a.ptr, b.ptr, c.ptr))  # noqa: E731
            ms = time_stream(ctx, fn, 20, 3)
            peak = PEAK_F32_MFMA_TFLOPS if dtype == np.float32 else PEAK_F64_MFMA_TFLOPS
            out["gemm"][f"{name}_{sfx}"] = {"us": ms * 1e3, "tflops": 2.0 * M * N * K / ms / 1e9, "frac_mfma": 2.0 * M * N * K / ms / 1e9 / peak}
            del a, b, c
    g = ctx.uniform((n,), 7, -4.0, 4.0)
    x = ctx.uniform((n,), 8, -4.0, 4.0)
    s = ctx.unary("sigmoid", x)
    t = ctx.unary("tanh", x)
    o = ctx.empty((n,))
    # the same gradients composed op by op as the reference's operators do (ops/unary.rs:254-375): more array passes
    # over HBM for the same algorithmic 3 arrays; GB/s below is still algorithmic bytes / time
    t1, t2 = ctx.empty((n,)), ctx.empty((n,))
    composed = {
        "relu_bwd": lambda: (ctx.scalar("greater_scalar", x, 0.0, out=t1), ctx.binary("mul", g, t1, out=o)),
        "sigmoid_bwd": lambda: (ctx.scalar("sub_scalar", s, 1.0, out=t1), ctx.binary("mul", s, t1, out=t2), ctx.binary("mul", g, t2, out=o)),
        "tanh_bwd": lambda: (ctx.binary("mul", t, t, out=t1), ctx.scalar("sub_scalar", t1, 1.0, out=t2), ctx.unary("neg", t2, out=t1),
                             ctx.binary("mul", g, t1, out=o)),
    }
    for name, fn in composed.items():
        ms = time_stream(ctx, fn, 5, 1)
        nbytes = 3 * 4 * n
        out["elementwise"][f"{name}_composed_f32"] = {"ms": ms, "GBps_algorithmic": nbytes / ms / 1e6}
    return out


TRAIN_CONFIGS = {
    "C5_cnn": dict(spec="conv 3 32 3 1 1; relu; conv 32 64 3 2 1; relu; flatten; linear 16384 10", in_shape=(256, 3, 32, 32),
                   classes=10, opt="adam 0.001 0.9 0.999 1e-08 0", seed=5),
    "C2_mlp": dict(spec="linear 784 256; relu; linear 256 128; relu; linear 128 10", in_shape=(256, 784), classes=10,
                   opt="sgd 0.01", seed=2),
    # CNNClassifier of the reference's examples (examples/common/models.rs:200-318) for 32x32 RGB images
    "cnn_classifier": dict(spec="conv 3 32 3 1 1; bn 32 0.001 0.1; relu; conv 32 64 3 1 1; bn 64 0.001 0.1; relu; gap; flatten; "
                                "linear 64 64; relu; dropout 0.3 23; linear 64 10", in_shape=(256, 3, 32, 32), classes=10,
                           opt="adam 0.001 0.9 0.999 1e-08 0", seed=6),
}


def make_train_problem(cfg, dtype):
    """Kaiming-uniform weights U(+-sqrt(6/fan_in)), zero biases, N(0,1) inputs, uniform one-hot labels."""
    rng = np.random.default_rng(cfg["seed"])
    params = []
    for tok in [t.strip() for t in cfg["spec"].split(";") if t.strip()]:
        p = tok.split()
        if p[0] == "linear":
            i, o = int(p[1]), int(p[2])
            params += [rng.uniform(-1, 1, (o, i)).astype(dtype) * dtype(np.sqrt(6.0 / i)), np.zeros(o, dtype)]
        elif p[0] == "conv":
            ci, co, k = int(p[1]), int(p[2]), int(p[3])
            params += [rng.uniform(-1, 1, (co, ci, k, k)).astype(dtype) * dtype(np.sqrt(6.0 / (ci * k * k))), np.zeros(co, dtype)]
        elif p[0] == "bn":  # weight ones, bias zeros (nn/layers/norm.rs:62-100)
            params += [np.ones(int(p[1]), dtype), np.zeros(int(p[1]), dtype)]
    x = rng.standard_normal(cfg["in_shape"]).astype(dtype)
    y = np.eye(cfg["classes"], dtype=dtype)[rng.integers(0, cfg["classes"], cfg["in_shape"][0])]
    return params, x, y


def c5_step_flop(batch=256):
    """Algorithmic FLOP of one C5 training step: 2*M*N*K per product; conv1 3->32 on 32x32 (forward + weight gradient: its
    input needs no gradient), conv2 32->64 stride 2 -> 16x16 and the 16384->10 classifier (forward + both gradients)."""
    conv1 = 2.0 * 32 * 27 * batch * 32 * 32
    conv2 = 2.0 * 64 * 288 * batch * 16 * 16
    fc = 2.0 * batch * 10 * 16384
    return 2 * conv1 + 3 * conv2 + 3 * fc


def train_step_roofline(name, batch, itemsize):
    """Per-kernel algorithmic work of the fused training step of config C5 (the CNN) or C2 (the perceptron): (label, FLOP, HBM
    bytes) for every launch group, each tensor counted once per kernel that must read or write it.  The time the step would take
    with every kernel at its own roofline is the sum over kernels of max(FLOP / MFMA peak, bytes / HBM peak)."""
    e = itemsize
    if name == "C5_cnn":
        a1 = batch * 32 * 32 * 32 * e      # conv1 activation [B,32,32,32]
        a2 = batch * 64 * 16 * 16 * e      # conv2 activation [B,64,16,16]
        x0 = batch * 3 * 32 * 32 * e
        w1, w2, w3 = 32 * 27 * e, 64 * 288 * e, 10 * 16384 * e
        f1, f2, f3 = 2.0 * 32 * 27 * batch * 1024, 2.0 * 64 * 288 * batch * 256, 2.0 * batch * 10 * 16384
        nparam = 32 * 27 + 32 + 64 * 288 + 64 + 10 * 16384 + 10
        return [
            ("conv1 fwd + bias + relu", f1, x0 + w1 + a1),
            ("conv2 fwd + bias + relu (stride 2)", f2, a1 + w2 + a2),
            ("head fwd + bias", f3, a2 + w3),
            ("softmax-CE loss + gradient", 0.0, 4 * batch * 10 * e),
            ("head dX", f3, w3 + a2),
            ("head dW + db", f3, a2 + w3),
            ("conv2 dgrad, relu mask in staging", f2, 2 * a2 + w2 + a1),
            ("conv2 wgrad + bias grad, relu mask in staging", f2, a1 + 2 * a2 + w2),
            ("conv1 wgrad + bias grad, relu mask in staging", f1, 2 * a1 + x0 + w1),
            ("Adam, all parameters in one launch", 0.0, 7 * nparam * e),
        ]
    if name == "C2_mlp":
        dims = [(784, 256), (256, 128), (128, 10)]
        rows = []
        for li, (i, o) in enumerate(dims):
            rows.append((f"fc{li + 1} fwd", 2.0 * batch * i * o, (batch * i + i * o + batch * o) * e))
        rows.append(("softmax-CE loss + gradient", 0.0, 4 * batch * 10 * e))
        for li, (i, o) in reversed(list(enumerate(dims))):
            if li > 0:
                rows.append((f"fc{li + 1} dX", 2.0 * batch * i * o, (batch * o + i * o + batch * i) * e))
            rows.append((f"fc{li + 1} dW + db", 2.0 * batch * i * o, (batch * o + batch * i + i * o) * e))
        nparam = sum(i * o + o for i, o in dims)
        rows.append(("SGD, all parameters in one launch", 0.0, 3 * nparam * e))
        return rows
    return None


def train_step_roofline_summary(name, dtype_name, step_ms, batch=256):
    itemsize = 8 if dtype_name == "float64" else 4
    rows = train_step_roofline(name, batch, itemsize)
    if not rows:
        return None
    peak = (PEAK_F64_MFMA_TFLOPS if itemsize == 8 else PEAK_F32_MFMA_TFLOPS) * 1e12
    t = [max(f / peak, b / (PEAK_HBM_GBS * 1e9)) for _, f, b in rows]
    total = sum(t)
    return {"bound": "mixed (per kernel: mfma or hbm, whichever is slower)", "time_at_roofline_ms": total * 1e3,
            "measured_ms": step_ms, "frac": total * 1e3 / step_ms,
            "algorithmic_flop": sum(f for _, f, _ in rows), "algorithmic_bytes": sum(b for _, _, b in rows),
            "kernels": [{"kernel": lab, "flop": f, "bytes": b, "us_at_roofline": ti * 1e6, "bound": "mfma" if f / peak >= b / (PEAK_HBM_GBS * 1e9) else "hbm"}
                        for (lab, f, b), ti in zip(rows, t)]}


def bench_reference_microbench(ctx):
    """The shapes of the reference's own kernel benchmark (kernels/benchmark.cu:21-25, 820-870): elementwise and activations on
    2^26 elements, reductions over 2^20 elements (all, and the [1000, 1024, 1] axis view), a 1024^3 product and the
    1 x 3 x 128 x 128 -> 32 convolution (forward, data gradient, weight gradient), f32 and f64."""
    from ferrox_amd import capi
    out = {}
    n = 1 << 26
    for dtype in (np.float32, np.float64):
        sfx = capi.dtype_code(dtype)[1]
        e = np.dtype(dtype).itemsize
        a = ctx.uniform((n,), 41, -4.0, 4.0, dtype)
        b = ctx.uniform((n,), 42, 0.5, 4.0, dtype)
        o = ctx.empty((n,), dtype)
        ew = {"add": (3, lambda: ctx.binary("add", a, b, out=o)), "mul": (3, lambda: ctx.binary("mul", a, b, out=o)),
              "div": (3, lambda: ctx.binary("div", a, b, out=o)), "relu": (2, lambda: ctx.unary("relu", a, out=o)),
              "sigmoid": (2, lambda: ctx.unary("sigmoid", a, out=o)), "tanh": (2, lambda: ctx.unary("tanh", a, out=o)),
              "exp": (2, lambda: ctx.unary("exp", a, out=o)), "sqrt": (2, lambda: ctx.unary("sqrt", b, out=o))}
        for name, (arrays, fn) in ew.items():
            ms = time_stream(ctx, fn, 10, 2)
            gbs = arrays * e * n / ms / 1e6
            out[f"elementwise_2^26_{name}_{sfx}"] = {"us": ms * 1e3, "GBps": gbs, "frac_hbm": gbs / PEAK_HBM_GBS}
        del a, b, o
        nr = 1 << 20
        r = ctx.normal((nr,), 43, 0.0, 1.0, dtype)
        res = ctx.empty((1024,), dtype)
        for kind in ("sum", "max", "min", "prod"):
            for label, view in (("all", (1, nr, 1)), ("axis_1000x1024", (1000, 1024, 1))):
                f = getattr(capi.lib, f"fx_reduce_{kind}_{sfx}")
                if kind in ("max", "min"):
                    fn = lambda f=f, view=view: capi.check(f(ctx.h, r.ptr, res.ptr, None, *view))  # noqa: E731
                else:
                    fn = lambda f=f, view=view: capi.check(f(ctx.h, r.ptr, res.ptr, *view))  # noqa: E731
                ms = time_stream(ctx, fn, 20, 3)
                nbytes = e * view[0] * view[1]
                out[f"reduce_2^20_{kind}_{label}_{sfx}"] = {"us": ms * 1e3, "GBps": nbytes / ms / 1e6}
        del r, res
        M = 1024
        ma, mb, mc = ctx.uniform((M, M), 44, -1.0, 1.0, dtype), ctx.uniform((M, M), 45, -1.0, 1.0, dtype), ctx.empty((M, M), dtype)
        fn = lambda: capi.check(getattr(capi.lib, f"fx_gemm_{sfx}")(ctx.h, 0, 0, M, M, M, ma.ptr, mb.ptr, mc.ptr))  # noqa: E731
        ms = time_stream(ctx, fn, 20, 3)
        peak = PEAK_F32_MFMA_TFLOPS if dtype == np.float32 else PEAK_F64_MFMA_TFLOPS
        out[f"matmul_1024_{sfx}"] = {"us": ms * 1e3, "tflops": 2.0 * M ** 3 / ms / 1e9, "frac_mfma": 2.0 * M ** 3 / ms / 1e9 / peak}
        del ma, mb, mc
        x = ctx.uniform((1, 3, 128, 128), 46, -1.0, 1.0, dtype)
        w = ctx.normal((32, 3, 3, 3), 47, 0.0, 0.27, dtype)
        g = ctx.normal((1, 32, 128, 128), 48, 0.0, 1.0, dtype)
        y, dx, dw = ctx.empty(g.shape, dtype), ctx.empty(x.shape, dtype), ctx.empty(w.shape, dtype)
        flop = 2.0 * 32 * 27 * 128 * 128
        for name, fn in (("conv2d_forward", lambda: ctx.conv2d_fwd(x, w, (1, 1), (1, 1), out=y)),
                         ("deconv2d", lambda: ctx.conv2d_dgrad(g, w, x.shape, (1, 1), (1, 1), 0, out=dx)),
                         ("cross_correlation2d", lambda: ctx.conv2d_wgrad(x, g, w.shape, (1, 1), (1, 1), 0, out=dw))):
            ms = time_stream(ctx, fn, 20, 3)
            out[f"conv_1x3x128x128_to_32_{name}_{sfx}"] = {"us": ms * 1e3, "tflops": flop / ms / 1e9}
        del x, w, g, y, dx, dw
    return out


def reference_pool_config():
    """PoolConfig::default() of the reference (src/backend/memory/mod.rs:50-82) with its allocation policy."""
    from ferrox_amd import capi
    cfg = capi.PoolConfig()
    cfg.n_buckets, cfg.literal_ids, cfg.best_fit = 4, 0, 0
    for i, b in enumerate([(1, 1024, 500, 50, -1), (1025, 262144, 50, 15, -1), (262145, 16777216, 10, 5, -1),
                           (16777217, 2**62, 2, 2, -1)]):
        cfg.buckets[i] = capi.BucketConfig(*b)
    return cfg


def bench_train_steps(steps=30, warmup=5, cpu=True, reference_pool=False, only=None):
    """Full training steps (forward + backward + optimizer step, allocations from the pool) through the mirrored
    Ferrox host stack; imgs/sec = batch / wall time per step with one final synchronisation."""
    from ferrox_amd import host_api
    host_api.init(0, 0, reference_pool_config() if reference_pool else None)
    out = {}
    for name, cfg in TRAIN_CONFIGS.items():
        for dtype in (np.float32, np.float64):
            if name in ("C2_mlp", "cnn_classifier") and dtype == np.float64:
                continue
            if only and (only[0] != name or only[1] != np.dtype(dtype).name):
                continue
            params, x, y = make_train_problem(cfg, dtype)
            key = f"{name}_{np.dtype(dtype).name}"
            out[key] = {"batch": int(x.shape[0])}
            # engine_literal: the reference's op sequence as is; engine_without_node_clones: the same minus the
            # engine's per-node deep clones; engine_fused: fused layers, loss and optimizer (extra entry points)
            # engine_fused_graph: the fused step recorded once into a HIP graph and replayed (one submission per step)
            # engine_literal_copying_clones: engine_literal with every clone_storage() as the device copy the reference's CUDA
            # backend makes; the other op-by-op lines share the block between a tensor and its clones
            for label, literal, fused in (("engine_literal", True, False), ("engine_literal_copying_clones", True, False),
                                          ("engine_without_node_clones", False, False),
                                          ("engine_fused", False, True), ("engine_fused_graph", False, True)):
                if (fused and reference_pool) or (only and only[2] != label):
                    continue
                host_api.set_share_clones(label != "engine_literal_copying_clones")
                m = host_api.Model(cfg["spec"], params, cfg["opt"], dtype, literal_engine=literal, fused=fused)
                if label == "engine_fused_graph":
                    m.enable_graph()
                m.set_batch(x, y)
                m.train_steps(warmup)
                st0 = host_api.pool_stats(dtype)
                loss, ms = m.train_steps(steps)
                st1 = host_api.pool_stats(dtype)
                req = (st1["pool_hits"] + st1["pool_misses"]) - (st0["pool_hits"] + st0["pool_misses"])
                out[key][label] = {
                    "ms_per_step": ms / steps, "imgs_per_s": x.shape[0] / (ms / steps / 1e3), "final_loss": loss,
                    "pool_requests_per_step": req / steps,
                    "pool_hit_rate": (st1["pool_hits"] - st0["pool_hits"]) / max(1, req),
                    "pool_underflow_misses": st1["underflow_misses"] - st0["underflow_misses"]}
                if label == "engine_fused_graph":
                    out[key][label]["graph"] = m.graph_info()  # kernel_nodes 0: the model has a Dropout layer and stayed eager
                m.close()
                host_api.set_share_clones(True)
            if cpu:
                from oracle import train as otrain
                ref = otrain.Sequential(cfg["spec"], params, dtype)
                kind, *nums = cfg["opt"].split()
                opt = otrain.SGD(float(nums[0])) if kind == "sgd" else otrain.Adam(*[float(v) for v in nums])
                n_cpu = 1 if name == "cnn_classifier" else 3
                t0 = time.perf_counter()
                for _ in range(n_cpu):
                    _, grads = ref.loss_and_grads(x, y)
                    opt.step(ref, grads)
                dt = (time.perf_counter() - t0) / n_cpu
                out[key]["cpu_baseline"] = {"value": x.shape[0] / dt, "unit": "imgs/s", "cores": 1, "kind": "port",
                                            "sample": f"{n_cpu} full steps of the same config, {dt:.2f} s per step"}
    host_api.shutdown()
    return out


def cpu_baseline_conv(batch=32, reps=4):
    """The CPU oracle (a restatement of Ferrox's ndarray path: im2col + single-thread GEMM + col2im) timed on this
    host, on a batch slice of the same layer; one thread, like the reference."""
    import oracle as orc
    c = dict(C3, B=batch)
    B, Cin, H, W, Cout, k, s, p = (c[n] for n in ("B", "Cin", "H", "W", "Cout", "k", "s", "p"))
    rng = np.random.default_rng(3)
    x = rng.uniform(-1, 1, (B, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, Cin, k, k)) * (2.0 / (Cin * k * k)) ** 0.5).astype(np.float32)
    g = rng.standard_normal((B, Cout, H, W)).astype(np.float32)
    flop = 3 * 2.0 * Cout * Cin * k * k * B * H * W
    t0 = time.perf_counter()
    for _ in range(reps):
        orc.conv2d_fwd(x, w, (s, s), (p, p))
        orc.conv2d_dgrad(g, w, x.shape, (s, s), (p, p), 0)
        orc.conv2d_wgrad(x, g, w.shape, (s, s), (p, p), 0)
    dt = (time.perf_counter() - t0) / reps
    out = {"value": flop / dt / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
           "sample": f"same layer at batch {B} of 128 (fwd+dgrad+wgrad, {reps} rep(s), {dt:.2f} s per rep), f32, "
                     f"im2col + blocked single-thread GEMM + col2im as in the reference CPU backend",
           "host_cpu": _cpu_model()}
    out["torch_cpu_comparator"] = _torch_cpu_conv(x, w, g, s, p, flop)
    return out


def _torch_cpu_conv(x, w, g, s, p, flop):
    """A tuned CPU library on the same slice (fwd + autograd backward), 1 thread and all threads: an upper-bound
    comparator for the CPU column, not the reference's algorithm."""
    import torch
    import torch.nn.functional as F
    res = {}
    keep = torch.get_num_threads()
    for label, nt in (("1_thread", 1), ("all_threads", keep)):
        torch.set_num_threads(nt)
        tx = torch.from_numpy(x).requires_grad_(True)
        tw = torch.from_numpy(w).requires_grad_(True)
        tg = torch.from_numpy(g)
        best = None
        for _ in range(2):
            t0 = time.perf_counter()
            F.conv2d(tx, tw, stride=s, padding=p).backward(tg)
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
            tx.grad = tw.grad = None
        res[label] = {"threads": nt, "tflops": flop / best / 1e12, "s_per_rep": best}
    torch.set_num_threads(keep)
    return res


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip() + f" ({os.cpu_count()} logical cores visible)"
    except OSError:
        pass
    return "unknown"


def bench_conv_sweep():
    """3x3, padding 1, f32: TFLOP/s of the three passes over channel counts and map sizes at stride 1, and over the
    channel-doubling layers at stride 2 (batch sized to a few GFLOP per pass).  Timed with the library's event timer on its own stream, 20 runs after 3 warm-up runs each."""
    from ferrox_amd import capi
    ctx = capi.Context(0)

    def timed(fn, runs=20, warm=3):
        for _ in range(warm):
            fn()
        ctx.sync()
        ctx.timer_start()
        for _ in range(runs):
            fn()
        return ctx.timer_stop() / runs

    out = {}

    def layer(key, batch, cin, hw, cout, stride, always_name):
        oh = (hw + 2 - 3) // stride + 1
        x = ctx.uniform((batch, cin, hw, hw), 1, -1.0, 1.0)
        g = ctx.normal((batch, cout, oh, oh), 2, 0.0, 1.0)
        w = ctx.normal((cout, cin, 3, 3), 3, 0.0, 0.05)
        y, dx, dw = ctx.empty(g.shape), ctx.empty(x.shape), ctx.empty(w.shape)
        gflop = 2.0 * cout * cin * 9 * batch * oh * oh / 1e9
        st = (stride, stride)
        ms, fam = [], []
        for fn in (lambda: ctx.conv2d_fwd(x, w, st, (1, 1), out=y),
                   lambda: ctx.conv2d_dgrad(g, w, x.shape, st, (1, 1), 0, out=dx),
                   lambda: ctx.conv2d_wgrad(x, g, w.shape, st, (1, 1), 0, out=dw)):
            ms.append(timed(fn))
            fam.append(ctx.conv2d_last_path())
        out[key] = [round(gflop / m, 1) for m in ms]
        if always_name or any("implicit" in f for f in fam):  # layers that fall off the specialised kernels say so
            out[key + "_kernel_families"] = fam
        for a in (x, g, w, y, dx, dw):
            a.free()

    for hw, batch in ((128, 16), (112, 16), (64, 64), (32, 128), (16, 256), (8, 512)):
        for cin in (32, 64, 128, 256):
            for cout in (32, 64, 128, 256):
                layer(f"B{batch}_{cin}to{cout}_{hw}x{hw}", batch, cin, hw, cout, 1, False)
    # stride 2 (padding 1), the channel-doubling layers between the stages of a residual network and the two of the CNN
    # example: which kernel family takes each pass is part of the figure
    for hw, batch in ((64, 128), (56, 128), (32, 256), (28, 256), (16, 512), (14, 512)):
        for cin, cout in ((32, 64), (64, 128), (128, 256)):
            layer(f"stride2_B{batch}_{cin}to{cout}_{hw}x{hw}", batch, cin, hw, cout, 2, True)
    ctx.close()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--skip-also", action="store_true")
    ap.add_argument("--skip-train", action="store_true", help="leave the train-step section out of `also` (short profiler runs)")
    ap.add_argument("--train-only", nargs="?", const="all", default=None, metavar="CONFIG,DTYPE,ENGINE",
                    help="run only the train-step section and print it (profiler runs); optional filter such as "
                         "C5_cnn,float32,engine_fused")
    ap.add_argument("--calibrate", action="store_true",
                    help="with --train-only: first run a streaming add over 2^26 floats four times (reads 2 x 256 MiB, writes "
                         "256 MiB per call): the kernel of known traffic that FETCH_SIZE / WRITE_SIZE readings of the same "
                         "profiler run are scaled by")
    ap.add_argument("--c4-profile", action="store_true",
                    help="run only the C4 bandwidth kernels, 4 calls each on rotating inputs with marker dispatches between "
                         "the cases, and print the case order (for rocprofv3 counter runs)")
    ap.add_argument("--conv-sweep", action="store_true",
                    help="run only a sweep of 3x3 f32 layer shapes (stride 1: Cin, Cout in 32..256 over 8x8..128x128 maps; stride 2: "
                         "channel-doubling layers over 14x14..64x64 maps) and print TFLOP/s per pass as one JSON line")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (the hot path has no cross-GPU exchange built); use --gpus 1")
    if args.conv_sweep:
        print(json.dumps({"conv_sweep_tflops_fwd_dgrad_wgrad": bench_conv_sweep()}))
        return
    if args.c4_profile:
        from ferrox_amd import capi
        with capi.Context(0) as ctx:
            print(json.dumps({"c4_profile_order": bench_c4_profile(ctx)}))
        return
    if args.train_only:
        if args.calibrate:
            from ferrox_amd import capi
            with capi.Context(0) as cctx:
                n = 1 << 26
                a, b, o = cctx.uniform((n,), 1, -1.0, 1.0), cctx.uniform((n,), 2, -1.0, 1.0), cctx.empty((n,))
                for _ in range(4):
                    cctx.binary("add", a, b, out=o)
                cctx.sync()
                del a, b, o
        only = None if args.train_only == "all" else tuple(args.train_only.split(","))
        print(json.dumps({"train_step": bench_train_steps(cpu=False, only=only)}))
        return

    from ferrox_amd import capi
    ctx = capi.Context(0)
    conv = bench_conv(ctx, args.steps, args.warmup)
    dominant = max(conv["per_pass"], key=lambda k: conv["per_pass"][k]["ms"])
    dom = conv["per_pass"][dominant]
    traffic, traffic_src = profile_traffic(CONV_C3_TRAFFIC_FILE, dominant)
    result = {
        "metric": "conv fwd+bwd TFLOP/s",
        "value": conv["tflops"],
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "priming_steps": PRIMING_STEPS,
        "ms_per_step": conv["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "C3: Conv2d N=128 Cin=64 56x56 -> Cout=128 3x3 s1 p1, f32; step = fwd + dgrad + wgrad",
                   "flop_per_step": 3 * conv["flop_per_pass"], "device": ctx.device_name()},
        "roofline": {"bound": "mfma", "kernel": CONV_KERNELS[dominant], "achieved": dom["tflops"],
                     "peak": PEAK_F32_MFMA_TFLOPS, "unit": "TFLOP/s", "frac": dom["tflops"] / PEAK_F32_MFMA_TFLOPS,
                     "traffic": traffic, "traffic_unit": "bytes per launch", "traffic_source": traffic_src,
                     "algorithmic_bytes": 308.6e6, "avg_launch_ms": dom["ms"],
                     # the other two metrics of the baseline: filled in below (slowest bandwidth kernel of config C4; the CNN
                     # training step of config C5 against the sum of its kernels' rooflines)
                     "others": {}},
        "conv_passes": {k: {"ms": v["ms"], "tflops": v["tflops"], "frac_mfma_f32": v["tflops"] / PEAK_F32_MFMA_TFLOPS, "kernel_family": v["kernel_family"]}
                        for k, v in conv["per_pass"].items()},
        "conv_fwd_bias_relu": conv.get("fwd_bias_relu"),
    }
    if not args.skip_also:
        c64 = bench_conv(ctx, max(3, args.steps // 4), 1, np.float64, B=C3["B"])
        result["also"] = {
            "conv_f64": {k: {"ms": v["ms"], "tflops": v["tflops"], "frac_mfma_f64": v["tflops"] / PEAK_F64_MFMA_TFLOPS, "kernel_family": v["kernel_family"]}
                         for k, v in c64["per_pass"].items()},
        }
        result["also"].update(bench_bandwidth(ctx))
        # second BASELINE metric: the slowest C4 bandwidth kernel against the HBM peak (reductions on rotating inputs)
        worst_name, worst = min([kv for kv in list(result["also"]["reductions"].items()) + list(result["also"]["elementwise"].items())
                                 if "frac_hbm" in kv[1]], key=lambda kv: kv[1]["frac_hbm"])
        w_traffic, w_src = profile_traffic(C4_TRAFFIC_FILE, worst_name)
        w_ms = worst["us"] / 1e3 if "us" in worst else worst["ms"]
        result["roofline"]["others"]["c4_worst"] = {
            "bound": "hbm", "kernel": worst_name, "achieved": worst["GBps"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "frac": worst["frac_hbm"], "traffic": w_traffic, "traffic_unit": "bytes per launch", "traffic_source": w_src,
            "algorithmic_bytes": worst["algorithmic_bytes"], "avg_launch_ms": w_ms}
        # every C4 case in one compact table: name -> [microseconds per call, fraction of the HBM peak]
        result["roofline"]["others"]["c4_cases_us_frac"] = {
            k: [round(v["us"] if "us" in v else v["ms"] * 1e3, 1), round(v["frac_hbm"], 3)]
            for k, v in list(result["also"]["reductions"].items()) + list(result["also"]["elementwise"].items()) if "frac_hbm" in v}
        result["also"]["reference_microbench"] = bench_reference_microbench(ctx)
    ctx.close()
    if not args.skip_also and not args.skip_train:
        result["also"]["train_step"] = bench_train_steps(cpu=not args.skip_cpu)
        result["also"]["train_step_reference_pool_config"] = bench_train_steps(cpu=False, reference_pool=True)
        # third BASELINE metric: the CNN training step (fused engine) -- algorithmic FLOP of its three GEMM-shaped layers
        # (forward, data gradient where one is needed, weight gradient) over the step's wall time, against the f32 MFMA peak
        c5_engines = result["also"]["train_step"].get("C5_cnn_float32", {})
        # the faster of the fused engine's two ways of launching the same kernels (one by one, or the step recorded once and replayed)
        c5_name = min((e for e in ("engine_fused", "engine_fused_graph") if e in c5_engines), key=lambda e: c5_engines[e]["ms_per_step"], default=None)
        c5 = c5_engines.get(c5_name) if c5_name else None
        if c5:
            flop = c5_step_flop()
            tfl = flop / (c5["ms_per_step"] * 1e-3) / 1e12
            rf = train_step_roofline_summary("C5_cnn", "float32", c5["ms_per_step"])
            rf.update({"kernel": "C5 CNN train step, %s (all kernels of the step)" % c5_name, "imgs_per_s": c5["imgs_per_s"],
                       "mfma_only": {"achieved": tfl, "peak": PEAK_F32_MFMA_TFLOPS, "unit": "TFLOP/s", "frac": tfl / PEAK_F32_MFMA_TFLOPS},
                       "traffic": None, "counters": "profiles/train_step_c5_f32_engine_fused_counters.txt"})
            result["roofline"]["others"]["c5_train_step"] = rf
        for key, cfg_name, dt in (("c5_train_step_f64", "C5_cnn", "float64"), ("c2_train_step", "C2_mlp", "float32")):
            eng = result["also"]["train_step"].get(f"{cfg_name}_{dt}", {})
            best = min((e for e in ("engine_fused", "engine_fused_graph") if e in eng), key=lambda e: eng[e]["ms_per_step"], default=None)
            if best:
                rf = train_step_roofline_summary(cfg_name, dt, eng[best]["ms_per_step"])
                rf.pop("kernels")
                rf.update({"kernel": f"{cfg_name} {dt} train step, {best}", "imgs_per_s": eng[best]["imgs_per_s"]})
                result["roofline"]["others"][key] = rf
    if not args.skip_cpu:
        result["cpu_baseline"] = cpu_baseline_conv()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
