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


def _documented_build():
    """The unit lists and flags of the build.rs shown to a maintainer in the integration notes at the repository root."""
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    lists = {}
    for name in ("HIP_UNITS", "PRELOAD_UNITS", "CPP_UNITS", "HIP_FLAGS", "PRELOAD_FLAGS", "CPP_FLAGS"):
        m = re.search(r"const " + name + r": &\[&str\] = &\[(.*?)\];", text, flags=re.S)
        assert m, f"the documented build.rs has no {name}"
        lists[name] = re.findall(r'"([^"]*)"', m.group(1))
    return lists


def _makefile_vars():
    text = open(os.path.join(ROOT, "wick_amd", "csrc", "Makefile")).read().replace("\\\n", " ")
    srcs = re.search(r"^SRCS\s*:=\s*(.*)$", text, flags=re.M).group(1).split()
    flags = re.search(r"^HIPFLAGS\s*:=\s*(.*)$", text, flags=re.M).group(1).split()
    preload = re.search(r"^((?:\$\(OBJ\)/\w+\.o\s*)+):\s*HIPFLAGS \+=\s*(.*)$", text, flags=re.M)
    return srcs, flags, re.findall(r"/(\w+)\.o", preload.group(1)), preload.group(2).split()


def test_documented_build_rs_matches_the_makefile():
    """The drop-in recipe cannot drift from what is built and tested here: same translation units, same flags."""
    doc = _documented_build()
    srcs, flags, preload_units, preload_flags = _makefile_vars()
    assert [u + ".hip" for u in doc["HIP_UNITS"]] == srcs
    assert doc["CPP_UNITS"] == ["gguf"]
    assert sorted(doc["PRELOAD_UNITS"]) == sorted(preload_units) and doc["PRELOAD_FLAGS"] == preload_flags
    warn = {"-Wall", "-Wno-unused-function"}  # diagnostics only
    assert doc["HIP_FLAGS"] == [f.replace("$(ARCH)", "gfx950") for f in flags if f not in warn]
    csrc = os.path.join(ROOT, "wick_amd", "csrc")
    assert sorted(f[:-4] for f in os.listdir(csrc) if f.endswith(".hip")) == sorted(doc["HIP_UNITS"]), "a .hip file is in neither list"


def test_archive_of_the_documented_units_links_the_host_mirror(tmp_path):
    """An archive made from exactly the documented units (their objects as the Makefile built them, same flags by the
    test above) resolves every symbol the statically linked C++ host mirror needs, i.e. the whole C ABI."""
    import subprocess

    doc = _documented_build()
    obj = os.path.join(ROOT, "wick_amd", "lib", "obj")
    objs = [os.path.join(obj, u + ".o") for u in doc["HIP_UNITS"] + doc["CPP_UNITS"]]
    for o in objs:
        assert os.path.exists(o), f"{o} has not been built (make -C wick_amd/csrc)"
    lib = str(tmp_path / "libwick_rocm.a")
    subprocess.run(["ar", "rcs", lib] + objs, check=True)
    exe = str(tmp_path / "host_selftest")
    out = subprocess.run(["g++", "-O1", "-std=c++17", "-o", exe, os.path.join(ROOT, "wick_amd", "host", "selftest.cpp"), lib,
                          "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,/opt/rocm/lib", "-lpthread"], capture_output=True, text=True)
    assert out.returncode == 0, out.stderr[-3000:]
    # and every symbol the three headers declare is defined in that archive
    nm = subprocess.run(["nm", "-g", "--defined-only", lib], capture_output=True, text=True, check=True).stdout
    defined = set(re.findall(r" T (\w+)", nm))
    for header, prefix in (("wick_rocm.h", "wick_rocm_"), ("wick_rocm_lfm2.h", "wick_rocm_"), ("wick_gguf.h", "wick_gguf_")):
        for name in declared_symbols(header, prefix):
            assert name in defined, f"{name} ({header}) is not defined by the documented units"
