"""The C-ABI library loads without a GPU and exports every symbol include/ferrox_hip.h declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "ferrox_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = text.replace("\\\n", "\n")
    plain = set(re.findall(r"\b(fx_[a-z0-9_]+)\s*\(", text.split("#define FX_DECLARE_KERNELS")[0]))
    macro_body = text.split("#define FX_DECLARE_KERNELS")[1].split("FX_DECLARE_KERNELS(float")[0]
    templ = set(re.findall(r"\b(fx_[a-z0-9_]+)_##S\s*\(", macro_body))
    tail = text.split("FX_DECLARE_KERNELS(double, f64)")[1]
    syms = set(plain) | set(re.findall(r"\b(fx_[a-z0-9_]+)\s*\(", tail))
    for s in ("f32", "f64"):
        syms |= {f"{t}_{s}" for t in templ}
    return syms


def test_library_exports_every_declared_symbol():
    from ferrox_amd import capi
    lib = ctypes.CDLL(capi.LIB_PATH)
    syms = declared_symbols()
    assert len(syms) > 90
    assert "fx_reduce_max_noalloc_f32" in syms
    missing = [s for s in sorted(syms) if not hasattr(lib, s)]
    assert not missing, missing


def test_error_reporting_without_gpu():
    from ferrox_amd import capi
    # null context is rejected by every entry point before any GPU work
    assert capi.lib.fx_sync(None) == 1
    assert b"null context" in capi.lib.fx_last_error()
    assert capi.lib.fx_conv2d_workspace_bytes(capi.CONV_WGRAD, capi.FX_F32, 0, 128, 64, 56, 56, 128, 3, 3, 1, 1, 1, 1) > 0
    assert capi.lib.fx_conv2d_workspace_bytes(capi.CONV_FWD, capi.FX_F32, 0, 1, 1, 2, 2, 1, 5, 5, 1, 1, 0, 0) == -1
    assert b"kernel larger than padded input" in capi.lib.fx_last_error()
