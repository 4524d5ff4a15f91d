"""The C-ABI library loads and exports every symbol include/ftrocm.h declares;
the compile-only entry point works without a GPU. No device calls here."""
import ctypes
import os
import re

import pytest

from flextensor_amd import runtime as rt

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    with open(os.path.join(ROOT, "include", "ftrocm.h")) as f:
        text = f.read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ftr_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported():
    syms = declared_symbols()
    assert len(syms) >= 14
    L = ctypes.CDLL(rt.LIB_PATH)
    for s in syms:
        assert hasattr(L, s), "missing export %s" % s
    assert sorted(rt.EXPORTS) == syms
    assert rt.lib().ftr_abi_version() == rt.ABI_VERSION


def test_compile_to_code_without_device(tmp_path, monkeypatch):
    monkeypatch.setattr(rt, "CACHE_DIR", str(tmp_path))
    src = 'extern "C" __global__ void k(float* p, float s) { p[threadIdx.x] *= s; }'
    code = rt.compile_to_code(src, ["-DUNUSED=1"])
    assert code[:4] == b"\x7fELF" and len(code) > 1000
    files = os.listdir(str(tmp_path))
    assert len(files) == 1 and files[0].endswith(".hsaco")
    assert rt.compile_to_code(src, ["-DUNUSED=1"]) == code          # cache hit
    assert rt.code_key(src, ["-DUNUSED=1"]) != rt.code_key(src, ["-DUNUSED=2"])


def test_compile_error_is_reported(tmp_path, monkeypatch):
    monkeypatch.setattr(rt, "CACHE_DIR", str(tmp_path))
    with pytest.raises(rt.RuntimeError_) as e:
        rt.compile_to_code('extern "C" __global__ void k() { undeclared_symbol(); }')
    assert "undeclared_symbol" in str(e.value)
    assert os.listdir(str(tmp_path)) == []


def test_null_arguments_fail_cleanly():
    L = rt.lib()
    assert L.ftr_compile_to_code(None, b"gfx950", None, 0, None, None) != 0
    assert b"null" in L.ftr_last_error()
    code, size = ctypes.c_void_p(), ctypes.c_size_t()
    src = b'extern "C" __global__ void k() {}'
    assert L.ftr_compile_to_code(src, b"gfx950", None, 2, ctypes.byref(code), ctypes.byref(size)) != 0
    assert b"option" in L.ftr_last_error() and not code.value
    ms = ctypes.c_float()
    assert L.ftr_time_seq(None, 1, 1, 0, 1, None, ctypes.byref(ms)) != 0
    assert L.ftr_module_attrs(None, None, None, None, None) != 0
    L.ftr_module_free(None)  # no-op


def test_every_template_compiles_for_gfx950():
    from flextensor_amd.scheduler import schedule_with_config
    from flextensor_amd.utils import Config
    for key in ("gemm_gemm_(1024, 1024, 1024)_rocm(0)",
                "gemm_gemm_int8_(4096, 4096, 4096)_rocm(0)",
                "conv2d_baseline0_(1, 64, 56, 56, 64, 3, 1, 1, 1, 1)_rocm(0)",
                "conv2d_depthwise_(8, 512, 28, 28, 1, 3, 1, 1, 1)_rocm(0)"):
        s, _ = schedule_with_config(key, Config([], None))
        for code in s.compile():
            assert code[:4] == b"\x7fELF"
    from flextensor_amd.templates import gfx950
    assert rt.compile_to_code(gfx950.template_source("naive.hip"), [])[:4] == b"\x7fELF"
