"""The C-ABI library loads and exports every symbol include/wick_rocm.h declares.
No compute is launched here (this file runs without a GPU)."""
import ctypes as C
import os
import re

import pytest

from conftest import ROOT

import wick_amd
from wick_amd import rocm


def declared_symbols(header="wick_rocm.h", prefix="wick_rocm_"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(" + prefix + r"[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_path():
    names = declared_symbols()
    for required in ("wick_rocm_quantize_q8_0", "wick_rocm_gemv_q8", "wick_rocm_gemm_q8", "wick_rocm_matmul_f32",
                     "wick_rocm_weight_upload", "wick_rocm_block_dots_i32", "wick_rocm_ctx_create"):
        assert required in names


def test_library_exports_every_declared_symbol():
    lib = wick_amd.load_library()
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} declared in wick_rocm.h but not exported"


def test_python_mirror_binds_every_declared_symbol():
    assert sorted(rocm._SIGNATURES) == declared_symbols()


def test_gguf_reader_symbols_are_exported_and_bound():
    from wick_amd import gguf

    names = declared_symbols("wick_gguf.h", "wick_gguf_")
    lib = wick_amd.load_library()
    for name in names:
        assert hasattr(lib, name), f"{name} declared in wick_gguf.h but not exported"
    assert sorted(gguf._SIGNATURES) == names


def test_lfm2_step_symbols_are_exported_and_bound():
    from wick_amd import lfm2

    names = declared_symbols("wick_rocm_lfm2.h", "wick_rocm_")
    lib = wick_amd.load_library()
    for name in names:
        assert hasattr(lib, name), f"{name} declared in wick_rocm_lfm2.h but not exported"
    assert sorted(lfm2._SIGNATURES) == names


def test_static_library_is_built_too():
    """What a Rust build.rs would link (cargo:rustc-link-lib=static=wick_rocm)."""
    assert os.path.exists(os.path.join(ROOT, "wick_amd", "lib", "libwick_rocm.a"))


def test_version_and_argument_checks_need_no_gpu():
    lib = wick_amd.load_library()
    assert lib.wick_rocm_version().startswith(b"wick-rocm")
    assert lib.wick_rocm_device_count(None) == -1  # INVALID_ARG
    assert lib.wick_rocm_ctx_create(0, None) == -1
    # null context: every entry point refuses instead of dereferencing
    assert lib.wick_rocm_sync(None) == -1
    assert lib.wick_rocm_quantize_q8_0(None, None, 1, 32, 32, None, None) == -1
    assert lib.wick_rocm_gemv_q8(None, None, None, None, None, 0) == -1


def test_no_device_is_an_error_not_a_fallback():
    if wick_amd.device_count() > 0:
        pytest.skip("a GPU is present")
    h = C.c_void_p()
    assert wick_amd.load_library().wick_rocm_ctx_create(0, C.byref(h)) == -5  # NO_DEVICE
    with pytest.raises(wick_amd.RocmError):
        wick_amd.RocmContext(0)


def test_product_path_does_not_import_the_oracle():
    """The shipped package must never route through the CPU oracle."""
    for dirpath, _, files in os.walk(os.path.join(ROOT, "wick_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.replace("no CPU fallback", ""), f"{f} mentions the oracle"
