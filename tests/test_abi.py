"""The C-ABI library loads without a GPU and exports exactly what include/rstorch_hip.h declares."""
import ctypes
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "rstorch_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rst_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from rstorch_amd import _ffi
    assert os.path.exists(_ffi.library_path()), "build the library first (__graft_entry__.build())"
    lib = ctypes.CDLL(_ffi.library_path())
    names = declared_functions()
    assert len(names) >= 40
    for n in names:
        assert hasattr(lib, n), "declared in the header but not exported: " + n


def test_binding_and_header_agree():
    from rstorch_amd import _ffi
    assert sorted(_ffi.EXPORTED_SYMBOLS) == declared_functions()


def test_rust_extern_block_in_the_integration_notes_matches_the_header():
    """The integration notes at the repository root show the Rust `extern "C"` block a maintainer of
    the reference would add; it is generated from the header and must declare every entry point, with
    the current signatures."""
    gen = os.path.join(ROOT, "include", "gen_rust_extern.py")
    block = subprocess.run([sys.executable, gen], capture_output=True, text=True, check=True).stdout
    assert sorted(re.findall(r"pub fn (rst_[a-z0-9_]+)", block)) == declared_functions()
    assert block.strip() in open(os.path.join(ROOT, "INTEGRATION.md")).read()
    for c_type, rust in (("const double* const*", "*const *const f64"), ("double* const*", "*const *mut f64"),
                         ("rst_engine**", "*mut *mut RstEngine"), ("const char*", "*const c_char")):
        sys.path.insert(0, os.path.join(ROOT, "include"))
        import gen_rust_extern
        assert gen_rust_extern.rust_type(c_type) == rust


def test_header_is_plain_c():
    src = '#include "rstorch_hip.h"\nint main(void){return (int)RST_OK + (int)sizeof(rst_kernel_record) * 0;}\n'
    out = subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"),
                          "-x", "c", "-", "-fsyntax-only"], input=src, text=True, capture_output=True)
    assert out.returncode == 0, out.stderr


def test_error_strings_without_gpu():
    from rstorch_amd import _ffi
    lib = _ffi.load()
    assert lib.rst_status_string(0) == b"ok"
    assert lib.rst_status_string(_ffi.RST_ERR_NAN) == b"NaN logits"
    assert lib.rst_engine_stream(None) is None
    assert lib.rst_engine_destroy(None) == 0 and lib.rst_model_destroy(None) == 0


def test_no_gpu_means_a_loud_failure():
    """Without a usable GPU the engine must fail with a HIP status, never fall back."""
    from rstorch_amd import _ffi
    lib = _ffi.load()
    h = ctypes.c_void_p()
    status = lib.rst_engine_create(0, ctypes.byref(h))
    if status == 0:  # a GPU is present (the GPU box): nothing to check here
        lib.rst_engine_destroy(h)
        pytest.skip("a GPU is visible")
    assert status in (_ffi.RST_ERR_HIP, _ffi.RST_ERR_INVALID_ARGUMENT)
    assert lib.rst_last_error()
    import rstorch_amd as rs
    with pytest.raises(rs.RstorchError):
        rs.Linear.new(2, 2)


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "rstorch_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".hpp", ".cpp")):
                text = open(os.path.join(base, f), errors="replace").read()
                assert "oracle" not in text.lower(), os.path.join(base, f)
