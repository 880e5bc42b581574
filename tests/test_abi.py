"""The shared object loads without a GPU and exports exactly the symbols of include/lego_hip.h;
the Python binding declares the same set; argument checks reject bad input before any launch."""
import ctypes
import re
from pathlib import Path

import pytest

from lego_amd import runtime

HEADER = Path(__file__).resolve().parents[1] / "include" / "lego_hip.h"


def declared():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return set(re.findall(r"\bint\s+(lego_hip_\w+)\s*\(", text))


def test_header_and_binding_agree():
    assert declared() == set(runtime.SIGNATURES)


def test_library_exports_every_declared_symbol():
    if not runtime.LIB_PATH.exists():
        pytest.fail("liblego_hip.so is not built: run python -m lego_amd.build")
    lib = ctypes.CDLL(str(runtime.LIB_PATH))
    for name in declared():
        assert hasattr(lib, name), name
    assert runtime.load_library().lego_hip_abi_version() == 1


def test_argument_validation_needs_no_gpu():
    lib = runtime.load_library()
    # null pointers, misaligned pointers and sizes a kernel cannot take are rejected on
    # the host (hipErrorInvalidValue == 1) before anything touches a device
    assert lib.lego_hip_transpose_f32(None, None, 64, 64, None) == 1
    assert lib.lego_hip_transpose_f16(ctypes.c_void_p(16), ctypes.c_void_p(4096), 0, 64, None) == 1
    assert lib.lego_hip_transpose_f16(ctypes.c_void_p(4096), ctypes.c_void_p(4096), 64, 64, None) == 1   # in place
    assert lib.lego_hip_transpose_f16(ctypes.c_void_p(8), ctypes.c_void_p(4096), 64, 64, None) == 1
    assert lib.lego_hip_softmax_f16(ctypes.c_void_p(16), ctypes.c_void_p(4096), 4, 0, None) == 1
    assert lib.lego_hip_softmax_f16_wpr(ctypes.c_void_p(16), ctypes.c_void_p(4096), 4, 12, 4, None) == 1
    assert lib.lego_hip_softmax_f32(ctypes.c_void_p(16), ctypes.c_void_p(4096), 0, 64, None) == 1
    assert lib.lego_hip_softmax_f16_wpr(ctypes.c_void_p(16), ctypes.c_void_p(4096), 4, 32776, 16, None) == 1
    assert lib.lego_hip_softmax_f16_wpr(ctypes.c_void_p(16), ctypes.c_void_p(4096), 4, 1024, 3, None) == 1      # no such team
    assert lib.lego_hip_gemm_f16(ctypes.c_void_p(16), ctypes.c_void_p(32), ctypes.c_void_p(64), 256, 0, 64, None) == 1
    assert lib.lego_hip_gemm_f16(ctypes.c_void_p(17), ctypes.c_void_p(32), ctypes.c_void_p(64), 256, 100, 64, None) == 1
    assert lib.lego_hip_gemm_f16_ex(ctypes.c_void_p(16), ctypes.c_void_p(32), ctypes.c_void_p(64), 8, 8, 64, 0, 0, 2, None) == 1
    assert lib.lego_hip_grouped_gemm_f16(None, None, None, None, 1, None) == 1
    with pytest.raises(runtime.LegoHipError):
        runtime.call("lego_hip_transpose_f32", None, None, 64, 64, None)


def test_missing_library_fails_loudly(tmp_path):
    with pytest.raises(FileNotFoundError):
        runtime.load_library(tmp_path / "liblego_hip.so")
