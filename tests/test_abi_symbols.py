"""The C-ABI library loads and exports every symbol include/sofie_hip.h declares (no GPU needed)."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "sofie_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sofie_hip_\w+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared_symbols()
    for must in ("sofie_hip_ctx_create", "sofie_hip_arena_create", "sofie_hip_gemm_f32", "sofie_hip_gemm_i8", "sofie_hip_gemm_fp8",
                 "sofie_hip_conv_f32", "sofie_hip_conv_i8", "sofie_hip_quantize_linear", "sofie_hip_last_error"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from sofie_amd import runtime
    if not os.path.exists(runtime.lib_path()):
        pytest.fail("%s is not built (run __graft_entry__.build())" % runtime.lib_path())
    lib = C.CDLL(runtime.lib_path())
    missing = [n for n in declared_symbols() if not hasattr(lib, n)]
    assert not missing, missing
    assert set(runtime.SYMBOLS) == set(declared_symbols())
    lib.sofie_hip_abi_version.restype = C.c_int
    assert lib.sofie_hip_abi_version() == 4


def test_error_path_without_a_gpu_call():
    from sofie_amd import runtime
    lib = runtime.load_library()
    # NULL context: refused with a message, nothing is launched
    assert lib.sofie_hip_sync(None) != 0
    assert b"ctx is NULL" in lib.sofie_hip_last_error()
    d = runtime.GemmI8Desc()
    assert lib.sofie_hip_gemm_i8_workspace(C.byref(d)) == 0
    d.K, d.N = 100, 40
    assert lib.sofie_hip_gemm_i8_workspace(C.byref(d)) == 4096  # [K,N] B needs re-layout: 4000 rounded to 256
