"""Bounds check of the convolution and matrix-product paths on the CPU (no GPU): the library's own conv.hip and gemm.hip --
dispatch, planners and every kernel they launch -- are compiled as host C++ (second half of this file: the products).
The convolution path: conv.hip -- dispatch, planners and every
patch / image-layer / stride-2 / implicit-GEMM kernel it launches -- is compiled as host C++ against a stand-in HIP header
(tests/kernel_walk/) and every thread of every block of every launch is run on the CPU with each tensor, the workspace and the
dynamic LDS between inaccessible pages.  What runs is the kernels' own address arithmetic, not a restatement of it: an
off-by-one in a kernel's staging code or in a planner faults here, on the shapes of the GPU tests, the tile shapes the tuner
may pick, and the layers of the baseline configurations.  (It guards a bug class that has occurred: passes of grad_out rows
that start past the last output channel were once read up to 53 KB past the end of the tensor.)"""
import hashlib
import os
import subprocess

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
WALK_DIR = os.path.join(HERE, "kernel_walk")
CSRC = os.path.join(ROOT, "ferrox_amd", "csrc")
CLANG = os.environ.get("FX_WALK_CXX", "/opt/rocm/lib/llvm/bin/clang++")


def _sources():
    files = [os.path.join(WALK_DIR, "walk.cpp"), os.path.join(WALK_DIR, "walk_gemm.cpp"), os.path.join(WALK_DIR, "hip", "hip_runtime.h"),
             os.path.join(ROOT, "include", "ferrox_hip.h")]
    files += sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hpp") or f in ("conv.hip", "gemm.hip"))
    return files


def _build_walk(name):
    """Builds tests/kernel_walk/build/<name> from tests/kernel_walk/<name>.cpp (kept until a source it includes changes)."""
    if not os.path.exists(CLANG):
        pytest.skip("no clang++ to build the host emulation with")
    out_dir = os.path.join(WALK_DIR, "build")
    os.makedirs(out_dir, exist_ok=True)
    exe, stamp = os.path.join(out_dir, name), os.path.join(out_dir, name + ".sha1")
    # the index arithmetic also runs under the integer checks of the undefined-behaviour sanitizer (overflow, shifts,
    # static array bounds: the statically sized LDS arrays), any finding ends the walk
    cmd = [CLANG, "-x", "c++", "-std=c++17", "-O1", "-g", "-I", WALK_DIR, "-DFX_HOST_EMULATION=1", "-Wno-unknown-attributes",
           "-Wno-unused-value", "-Wno-psabi", "-fsanitize=signed-integer-overflow,shift,bounds,integer-divide-by-zero",
           "-fno-sanitize-recover=all", "-o", exe, os.path.join(WALK_DIR, name + ".cpp")]
    h = hashlib.sha1(" ".join(cmd).encode())
    for f in _sources():
        h.update(open(f, "rb").read())
    if not (os.path.exists(exe) and os.path.exists(stamp) and open(stamp).read() == h.hexdigest()):
        r = subprocess.run(cmd, capture_output=True, text=True, cwd=WALK_DIR)
        assert r.returncode == 0, r.stderr[-4000:]
        open(stamp, "w").write(h.hexdigest())
    return exe


@pytest.fixture(scope="module")
def walk_binaries():
    """Both harnesses, compiled side by side."""
    if not os.path.exists(CLANG):
        pytest.skip("no clang++ to build the host emulation with")
    from concurrent.futures import ThreadPoolExecutor
    with ThreadPoolExecutor(2) as pool:
        conv, gemm = pool.map(_build_walk, ("walk", "walk_gemm"))
    return {"walk": conv, "walk_gemm": gemm}


@pytest.fixture(scope="module")
def walk_binary(walk_binaries):
    return walk_binaries["walk"]


@pytest.fixture(scope="module")
def gemm_walk_binary(walk_binaries):
    return walk_binaries["walk_gemm"]


def run_walk(exe, cases, env=None, timeout=900):
    lines = "".join("%s %s %s\n" % (name, dt, " ".join(str(int(v)) for v in dims)) for name, dt, dims in cases)
    e = dict(os.environ)
    e.update(env or {})
    return subprocess.run([exe], input=lines, capture_output=True, text=True, env=e, timeout=timeout)


def dims_of(B, Cin, H, W, Cout, k, st, pd):
    kh, kw = (k, k) if isinstance(k, int) else k
    (sh, sw), (ph, pw) = (st, st) if isinstance(st, int) else st, (pd, pd) if isinstance(pd, int) else pd
    return (B, Cin, H, W, Cout, kh, kw, sh, sw, ph, pw)


BATCH_CAP = 1000


def gpu_test_cases():
    """The layer shapes of the GPU parity tests, batch capped at 4 (the batch only moves base addresses; the image-count logic
    of the planners is covered by the full-batch baseline layers below)."""
    import test_gpu_kernels as tk
    import test_gpu_fused as tf
    cases = []

    def add(tag, dt, B, Cin, H, W, Cout, k, st, pd):
        cases.append(("%s_%d" % (tag, len(cases)), dt, dims_of(min(B, BATCH_CAP), Cin, H, W, Cout, k, st, pd)))
    for (B, Cin, H, W, Cout, k, s, p) in tk.CONV_CASES:
        for dt in ("f32", "f64"):
            add("conv", dt, B, Cin, H, W, Cout, k, s, p)
    for (B, Cin, H, W, Cout, st, pd) in tk.WGRAD_PATCH_CASES:
        add("wgrad_patch", "f32", B, Cin, H, W, Cout, 3, st, pd)
    for (B, Cin, H, W, Cout, st, pd) in tk.CONV_PATCH_CASES:
        add("conv_patch", "f32", B, Cin, H, W, Cout, 3, st, pd)
    for (B, Cin, H, W, Cout, st, pd) in tk.CONV_F64_PATCH_CASES:
        add("conv_patch_f64", "f64", B, Cin, H, W, Cout, 3, st, pd)
    for (B, Cin, H, W, Cout, st, pd) in tk.CONV_F64_WGRAD_CASES:
        add("wgrad_patch_f64", "f64", B, Cin, H, W, Cout, 3, st if isinstance(st, tuple) else (st, 1), pd)
    for (B, Cin, H, W, Cout, st, pd) in tk.SMALLC_CASES:
        for dt in ("f32", "f64"):
            add("image_layer", dt, B, Cin, H, W, Cout, 3, st, pd)
    for (B, Cin, H, W, Cout, st, pd) in tk.IMAGE_F64_EXTRA:
        add("image_layer_f64", "f64", B, Cin, H, W, Cout, 3, st, pd)
    for (B, Cin, H, W, Cout) in tk.POINTWISE_CASES:
        add("pointwise", "f32", B, Cin, H, W, Cout, 1, 1, 0)
    for (B, Cin, H, W, Cout, k, st, pd) in tk.STRIDED_DGRAD_CASES:
        for dt in ("f32", "f64"):
            add("strided", dt, B, Cin, H, W, Cout, k, st, pd)
    for np_dt, dt in ((np.float32, "f32"), (np.float64, "f64")):
        for (B, Cin, H, W, Cout, st, pd) in tf.CONV_BWD_RELU_CASES[np_dt]:
            add("bwd_relu", dt, B, Cin, H, W, Cout, 3, st, pd)
    for (B, Cin, H, W, Cout, k, st, pd, np_dt), _ in tk.EXPECTED_PATHS:
        add("path", "f32" if np_dt == np.float32 else "f64", B, Cin, H, W, Cout, k, st, pd)
    for seed, np_dt in tk.RANDOM_CONV_SEEDS:
        for (it, B, Cin, H, W, Cout, k, st, pd) in tk.random_conv_shapes(seed):
            add("random_%d" % seed, "f32" if np_dt == np.float32 else "f64", B, Cin, H, W, Cout, k, st, pd)
    return cases


# the convolution layers of the baseline configurations: the plumbing layer and the two CNN layers at their full batch, the
# roofline layer at a slice of its batch (its blocks walk the same addresses for every image)
BASELINE_LAYERS = [
    ("plumbing_conv", "f32", (32, 1, 28, 28, 8, 3, 3, 1, 1, 1, 1)), ("plumbing_conv", "f64", (32, 1, 28, 28, 8, 3, 3, 1, 1, 1, 1)),
    ("cnn_conv1", "f32", (256, 3, 32, 32, 32, 3, 3, 1, 1, 1, 1)), ("cnn_conv1", "f64", (256, 3, 32, 32, 32, 3, 3, 1, 1, 1, 1)),
    ("cnn_conv2", "f32", (256, 32, 32, 32, 64, 3, 3, 2, 2, 1, 1)), ("cnn_conv2", "f64", (256, 32, 32, 32, 64, 3, 3, 2, 2, 1, 1)),
    ("roofline_layer_slice", "f32", (6, 64, 56, 56, 128, 3, 3, 1, 1, 1, 1)), ("roofline_layer_slice", "f64", (3, 64, 56, 56, 128, 3, 3, 1, 1, 1, 1)),
    ("reference_benchmark_conv", "f32", (1, 3, 128, 128, 32, 3, 3, 1, 1, 1, 1)), ("reference_benchmark_conv", "f64", (1, 3, 128, 128, 32, 3, 3, 1, 1, 1, 1)),
]


def test_every_access_of_the_convolution_path_stays_inside_its_buffers(walk_binary):
    from concurrent.futures import ThreadPoolExecutor
    cases = gpu_test_cases() + BASELINE_LAYERS
    # the cases are independent: interleaved shares of the list run as separate processes side by side
    shares = max(1, min(6, (os.cpu_count() or 2) - 1))
    parts = [cases[i::shares] for i in range(shares)]
    with ThreadPoolExecutor(shares) as pool:
        results = list(pool.map(lambda part: run_walk(walk_binary, part), parts))
    for part, r in zip(parts, results):
        assert r.returncode == 0, (r.stdout[-600:], r.stderr[-1500:])
        assert "walked %d cases" % len(part) in r.stdout, r.stdout[-300:]


@pytest.mark.parametrize("which", ["x", "w", "y", "g", "dx", "dw", "act", "ws", "lds"])
def test_the_walk_faults_when_a_buffer_is_16_bytes_short(walk_binary, which):
    """The detector's own test: with one tensor (or the workspace, or every block's dynamic LDS) 16 bytes shorter than the
    code is entitled to, the walk of layers that use it must end in a fault that names the case."""
    cases = [("cnn_conv1", "f32", (3, 3, 32, 32, 32, 3, 3, 1, 1, 1, 1)), ("cnn_conv2", "f32", (3, 32, 32, 32, 64, 3, 3, 2, 2, 1, 1)),
             ("stride1", "f32", (2, 64, 16, 16, 128, 3, 3, 1, 1, 1, 1)), ("cnn_conv2", "f64", (3, 32, 32, 32, 64, 3, 3, 2, 2, 1, 1))]
    if which == "ws":  # layers on the implicit GEMM, whose ordered K split fills the advertised workspace to the last byte
        cases += [("five_by_five", "f32", (4, 16, 12, 12, 32, 5, 5, 1, 1, 2, 2)), ("strided_14", "f32", (8, 32, 14, 14, 64, 3, 3, 2, 2, 1, 1))]
    if which == "act":  # only layers with a fused conv + ReLU backward read the activation
        cases = [c for c in cases if c[0] != "stride1"]
    faults = 0
    for case in cases:
        r = run_walk(walk_binary, [case], env={"FX_WALK_SHRINK": which})
        faulted = r.returncode == 3 and "FAULT" in r.stderr and case[0] in r.stderr
        assert faulted or r.returncode == 0, (which, case, r.returncode, r.stderr[-500:])
        # the advertised workspace is an upper bound over the kernels a call may take (a 128-row weight image whatever tile
        # runs, room for the masked variant's bias sums): a short one need not fault on every layer, but on some
        assert faulted or which == "ws", (which, case, "did not fault")
        faults += faulted
    assert faults >= 1, which


# ------------------------------------------------------------------------------------------ matrix products
def gemm_cases():
    """(name, dtype, (M, N, K)) for every product shape of the GPU tests, both types, plus the products of the baseline
    configurations; walk_gemm runs all four transpose forms with and without the bias epilogue on each."""
    import test_gpu_kernels as tk
    shapes = list(tk.GEMM_SHAPES) + list(tk.GEMM_LDS_SHAPES) + list(tk.GEMM_SMALL_SHAPES) + [(M, N, K) for (_, M, N, K) in tk.GEMM_THIN_SHAPES]
    # classifier head of the CNN step and its gradients, the MLP layers, the reference's benchmark product, a product of full tiles
    shapes += [(256, 10, 16384), (256, 16384, 10), (10, 16384, 256), (256, 256, 784), (256, 128, 256), (256, 10, 128), (784, 256, 256),
               (1024, 1024, 1024), (2048, 2048, 512)]
    cases = []
    for (M, N, K) in shapes:
        for dt in ("f32", "f64"):
            cases.append(("gemm_%d" % len(cases), dt, (M, N, K)))
    return cases


def test_every_access_of_the_matrix_product_path_stays_inside_its_buffers(gemm_walk_binary):
    from concurrent.futures import ThreadPoolExecutor
    cases = gemm_cases()
    shares = max(1, min(6, (os.cpu_count() or 2) - 1))
    parts = [cases[i::shares] for i in range(shares)]
    with ThreadPoolExecutor(shares) as pool:
        results = list(pool.map(lambda part: run_walk(gemm_walk_binary, part), parts))
    for part, r in zip(parts, results):
        assert r.returncode == 0, (r.stdout[-600:], r.stderr[-1500:])
        assert "walked %d cases" % len(part) in r.stdout, r.stdout[-300:]


@pytest.mark.parametrize("which", ["a", "b", "c"])
def test_the_product_walk_faults_when_a_matrix_is_16_bytes_short(gemm_walk_binary, which):
    """The detector's own test, as for the convolution walk: with A, B or C 16 bytes shorter than its shape the walk must end in a
    fault that names the case, on the slab kernel, the small-product kernel and the general tiles alike."""
    for case in [("slab", "f32", (2560, 2560, 128)), ("small", "f32", (33, 65, 36)), ("general", "f64", (130, 257, 75))]:
        r = run_walk(gemm_walk_binary, [case], env={"FX_WALK_SHRINK": which})
        assert r.returncode == 3 and "FAULT" in r.stderr and case[0] in r.stderr, (which, case, r.returncode, r.stderr[-500:])
