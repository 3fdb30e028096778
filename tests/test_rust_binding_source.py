"""The Rust side of the boundary is delivered as source (no Rust toolchain in this image).  These checks keep it honest
mechanically: the FFI crate is generated from the header and complete, HipStorage writes out every method of Ferrox's
`trait StorageBackend`, and every FFI name the Rust modules use exists."""
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SYS_LIB = os.path.join(ROOT, "rust", "ferrox-hip-sys", "src", "lib.rs")
STORAGE = os.path.join(ROOT, "rust", "src", "backend", "storage", "hip.rs")
HIPMOD = os.path.join(ROOT, "rust", "src", "backend", "hip", "mod.rs")

# trait StorageBackend<T>, src/backend/storage/mod.rs:24-422 (expand_dims has a default body there)
TRAIT_METHODS = """shape as_any into_any ndim size is_gpu cpu_data cpu_data_mut owns_data clone_storage add sub mul div min max
add_scalar mul_scalar div_scalar sub_scalar neg abs clamp sqrt reciprocal greater_equal greater_equal_scalar less_equal
less_equal_scalar greater greater_scalar less less_scalar equal logical_not in_range sign matmul sigmoid softmax softmax_batched
relu exp log tanh powf power_scalar sum mean max_reduce min_reduce broadcast_to reshape transpose unsqueeze squeeze conv2d conv1d
deconv1d cross_correlation2d cross_correlation1d deconv2d iter_values get_flat get_multi maxpool2d avgpool2d maxpool1d avgpool1d
max_unpool2d avg_unpool2d max_unpool1d avg_unpool1d""".split()
# the hot-path methods the boundary has to serve with a kernel (not an Err)
HOT_PATH = """add sub mul div add_scalar sub_scalar mul_scalar div_scalar neg sqrt clamp greater_scalar greater_equal_scalar
less_equal_scalar equal matmul relu sigmoid tanh exp log softmax_batched sum mean max_reduce broadcast_to reshape transpose
unsqueeze squeeze conv2d deconv2d cross_correlation2d""".split()


def test_generated_bindings_are_current_and_complete():
    gen = os.path.join(ROOT, "rust", "ferrox-hip-sys", "generate.py")
    assert subprocess.run([sys.executable, gen, "--check"]).returncode == 0, "run rust/ferrox-hip-sys/generate.py"
    from test_cabi_exports import declared_symbols
    text = open(SYS_LIB).read()
    block = text[text.index('extern "C" {'):]
    rust_syms = set(re.findall(r"pub fn (fx_\w+)\(", block))
    assert rust_syms == declared_symbols()
    # struct layouts: same field order as the C structs
    from ferrox_amd import capi
    for cls, name in ((capi.PoolStats, "fx_pool_stats"), (capi.BucketStats, "fx_bucket_stats"), (capi.BucketConfig, "fx_bucket_config"),
                      (capi.PoolConfig, "fx_pool_config")):
        body = re.search(r"pub struct %s \{(.*?)\}" % name, text, flags=re.S).group(1)
        assert re.findall(r"pub (\w+):", body) == [f for f, _ in cls._fields_], name


def _method_bodies(text):
    """name -> body text of every `fn name(...) ... { ... }` inside the `impl StorageBackend` block."""
    impl = text[text.index("impl<T> StorageBackend<T> for HipStorage<T>"):]
    out = {}
    for m in re.finditer(r"\n    fn (\w+)\(", impl):
        start = impl.index("{", impl.index(")", m.end()))
        # the signature may carry a where clause before the body
        depth, i = 0, start
        while True:
            if impl[i] == "{":
                depth += 1
            elif impl[i] == "}":
                depth -= 1
                if depth == 0:
                    break
            i += 1
        out[m.group(1)] = impl[start + 1:i]
    return out


def test_hip_storage_writes_out_every_trait_method():
    bodies = _method_bodies(open(STORAGE).read())
    missing = [m for m in TRAIT_METHODS if m not in bodies]
    assert not missing, missing
    for name, body in bodies.items():
        code = re.sub(r"//.*", "", body).strip()
        assert code, f"{name} has a comment-only body"
    for name in HOT_PATH:
        assert "not implemented" not in bodies[name], name


def test_every_ffi_name_used_by_the_rust_modules_exists():
    sys_text = open(SYS_LIB).read()
    defined = set(re.findall(r"pub (?:fn|const|struct) (\w+)", sys_text))
    for path in (STORAGE, HIPMOD):
        used = set(re.findall(r"\bsys::(\w+)", open(path).read()))
        used -= {"check"}
        unknown = sorted(u for u in used if u not in defined and not u.startswith("$"))
        assert not unknown, (path, unknown)
    assert "pub fn check" in sys_text


def test_trait_method_list_matches_the_reference_when_it_is_present():
    ref = "/root/reference/src/backend/storage/mod.rs"
    if not os.path.exists(ref):
        import pytest
        pytest.skip("reference checkout not present")
    text = open(ref).read()
    trait = text[text.index("pub trait StorageBackend<T>"):text.index("#[cfg(test)]")]
    names = set(re.findall(r"\n    fn (\w+)", trait)) - {"expand_dims"}
    assert names == set(TRAIT_METHODS)
