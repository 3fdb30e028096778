"""Builds libferrox_hip.so (gfx950 only) from csrc/*.hip with hipcc.

    python -m ferrox_amd.build            # compile everything, link in-tree
The library is built in-tree (ferrox_amd/libferrox_hip.so) so that it travels with the source tree.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libferrox_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# Packed FP32 instruction selection is switched off for all device code.
COMMON = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
# Files whose composed expressions must round op by op like the CPU backend (no a*b+c contraction).
NO_CONTRACT = {"elementwise.hip", "reduce.hip", "im2col.hip", "fused.hip", "pooling.hip", "batchnorm.hip"}


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src):
    obj = os.path.join(OBJ, src.replace(".hip", ".o"))
    cmd = [HIPCC] + COMMON + (["-ffp-contract=off"] if src in NO_CONTRACT else []) + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    return obj, err


def build(verbose=False, jobs=None):
    os.makedirs(OBJ, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(_compile, sources()))
    objs = [o for o, _ in results]
    if verbose:
        for _, err in results:
            if err:
                print(err, file=sys.stderr)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
