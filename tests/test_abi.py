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
    assert lib.lego_hip_transpose_f16(ctypes.c_void_p(4097), ctypes.c_void_p(4096), 64, 64, None) == 1   # not even element aligned
    assert lib.lego_hip_transpose_f32(ctypes.c_void_p(4098), ctypes.c_void_p(8192), 64, 64, None) == 1
    assert lib.lego_hip_softmax_f16(ctypes.c_void_p(4097), ctypes.c_void_p(8192), 4, 64, None) == 1
    assert lib.lego_hip_layernorm_fwd_f32(ctypes.c_void_p(4096), ctypes.c_void_p(8194), ctypes.c_void_p(64), ctypes.c_void_p(128),
                                          ctypes.c_void_p(256), ctypes.c_void_p(512), 4, 64, ctypes.c_float(1e-5), None) == 1
    assert lib.lego_hip_softmax_f16_wpr(ctypes.c_void_p(4098), ctypes.c_void_p(8192), 4, 64, 1, None) == 1   # the tuning entry points keep 16 bytes
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


def test_workspace_sizes_follow_the_launch_rules():
    """The size queries are plain host functions.  LayerNorm backward: the partial rows are `N` rounded up to 8
    floats apart; when rows of any length are walked by fewer workgroups than rows, the number of workgroups is
    a multiple of eight, so that a workgroup's rows start at the same offset from a 16-byte boundary.  GEMM: a
    shape with N or K off the 16-byte grid asks for room for padded copies of both operands and the result."""
    lib = runtime.load_library()
    need = ctypes.c_ulonglong(0)
    for entry, elements_per_16_bytes in (("lego_hip_layernorm_bwd_workspace_bytes", 8),
                                         ("lego_hip_layernorm_bwd_bf16_workspace_bytes", 8),
                                         ("lego_hip_layernorm_bwd_f32_workspace_bytes", 4)):
        fn = getattr(lib, entry)
        for N in (1, 7, 33, 250, 781, 1001, 1023, 2050, 4099, 8191, 12001, 16383, 512, 4096, 16384):
            pitch = (N + 7) // 8 * 8
            for M in (1, 3, 8, 100, 255, 256, 257, 511, 513, 1000, 4097, 100000):
                assert fn(M, N, ctypes.byref(need)) == 0
                assert need.value % (2 * pitch * 4) == 0
                groups = need.value // (2 * pitch * 4)
                assert 1 <= groups <= max(M, 8) and groups <= 1024, (entry, M, N, groups)
                if N % 8 and groups < M:
                    assert groups % 8 == 0, (entry, M, N, groups)
                if N % 8 and N <= 1024:       # a wavefront per row: the four waves of a workgroup start alike too
                    assert groups % 8 == 0, (entry, M, N, groups)
        assert fn(4, 32769, ctypes.byref(need)) == 1 and fn(0, 8, ctypes.byref(need)) == 1
    for M, N, K in ((193, 131, 77), (4096, 4096, 4097), (4096, 4100, 4096), (5, 7, 3), (16, 8190, 8192)):
        assert lib.lego_hip_gemm_workspace_bytes(M, N, K, ctypes.byref(need)) == 0
        r8 = lambda v: (v + 7) // 8 * 8
        assert need.value >= 2 * (r8(M) * r8(K) + r8(K) * r8(N) + r8(M) * r8(N)), (M, N, K)
        assert need.value % 16 == 0
    for M, N, K in ((4096, 4096, 4096), (1001, 264, 200), (2048, 1024, 64)):     # M alone never asks for copies
        assert lib.lego_hip_gemm_workspace_bytes(M, N, K, ctypes.byref(need)) == 0 and need.value == 0, (M, N, K)
