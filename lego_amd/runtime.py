"""ctypes binding of liblego_hip.so (include/lego_hip.h).

The library is built ahead of time by ``python -m lego_amd.build``; loading never
compiles.  If the shared object is missing the import of an operator fails with a clear
error instead of falling back to another implementation.
"""
from __future__ import annotations

import ctypes
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "lib" / "liblego_hip.so"

_c_int, _c_void_p, _c_float = ctypes.c_int, ctypes.c_void_p, ctypes.c_float
_PTR_ARRAY = ctypes.POINTER(ctypes.c_void_p)
_INT_ARRAY = ctypes.POINTER(ctypes.c_int)

# name -> argument types, exactly the prototypes of include/lego_hip.h
SIGNATURES = {
    "lego_hip_abi_version": [],
    "lego_hip_transpose_f32": [_c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
    "lego_hip_transpose_f16": [_c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
    "lego_hip_transpose_f32_tiling": [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
    "lego_hip_transpose_f16_tiling": [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
    "lego_hip_softmax_f16": [_c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
    "lego_hip_softmax_f32": [_c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
    "lego_hip_softmax_bf16": [_c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
    "lego_hip_layernorm_fwd_f32": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                                   _c_int, _c_int, _c_float, _c_void_p],
    "lego_hip_layernorm_fwd_bf16": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                                    _c_int, _c_int, _c_float, _c_void_p],
    "lego_hip_layernorm_fwd_f16": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                                   _c_int, _c_int, _c_float, _c_void_p],
    "lego_hip_gemm_f16": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
    "lego_hip_gemm_f16_variant": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p],
    "lego_hip_gemm_plan": [_c_int, _c_int, _c_int, ctypes.POINTER(_c_int)],
    "lego_hip_rows_f16_plan": [_c_int, _c_int, ctypes.POINTER(_c_int)],
    "lego_hip_gemm_f16_act": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_void_p],
    "lego_hip_gemm_f16_ex": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                             _c_void_p],
    "lego_hip_gemm_bf16_ex": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                             _c_void_p],
    "lego_hip_gemm_bf16_f16_ex": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                  _c_void_p],
    "lego_hip_gemm_workspace_bytes": [_c_int, _c_int, _c_int, ctypes.POINTER(ctypes.c_ulonglong)],
    "lego_hip_gemm_ex_ws": [_c_int, _c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                            _c_void_p, ctypes.c_ulonglong, _c_void_p],
    "lego_hip_gemm_fp8_ex": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                             _c_int, _c_void_p],
    "lego_hip_stencil_f3d_f32": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
    "lego_hip_stencil_laplacian_f32": [_c_void_p, _c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
    "lego_hip_lud_f32": [_c_void_p, _c_int, _c_void_p],
    "lego_hip_lud_f32_plan": [_c_int, ctypes.POINTER(_c_int), _c_int, ctypes.POINTER(_c_int)],
    "lego_hip_nw_i32": [_c_void_p, _c_void_p, _c_int, _c_int, _c_void_p],
    "lego_hip_grouped_gemm_f16": [_PTR_ARRAY, _PTR_ARRAY, _PTR_ARRAY, _INT_ARRAY, _c_int, _c_void_p],
    "lego_hip_grouped_gemm_f16_plan": [_INT_ARRAY, _c_int, _INT_ARRAY],
    "lego_hip_grouped_gemm_f16_split": [_PTR_ARRAY, _PTR_ARRAY, _PTR_ARRAY, _INT_ARRAY, _c_int, _c_int, _c_void_p],
    "lego_hip_softmax_f16_wpr": [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
    "lego_hip_layernorm_fwd_f16_wpr": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p,
                                       _c_int, _c_int, _c_float, _c_int, _c_void_p],
    "lego_hip_layernorm_bwd_workspace_bytes": [_c_int, _c_int, ctypes.POINTER(ctypes.c_ulonglong)],
    "lego_hip_layernorm_bwd_f16": [_c_void_p] * 9 + [ctypes.c_ulonglong, _c_int, _c_int, _c_void_p],
    "lego_hip_layernorm_bwd_f16_noalloc": [_c_void_p] * 8 + [_c_int, _c_int, _c_void_p],
    "lego_hip_layernorm_bwd_f32_workspace_bytes": [_c_int, _c_int, ctypes.POINTER(ctypes.c_ulonglong)],
    "lego_hip_layernorm_bwd_f32": [_c_void_p] * 9 + [ctypes.c_ulonglong, _c_int, _c_int, _c_void_p],
    "lego_hip_layernorm_bwd_bf16_workspace_bytes": [_c_int, _c_int, ctypes.POINTER(ctypes.c_ulonglong)],
    "lego_hip_layernorm_bwd_bf16": [_c_void_p] * 9 + [ctypes.c_ulonglong, _c_int, _c_int, _c_void_p],
    "lego_hip_copy16": [_c_void_p, _c_void_p, ctypes.c_ulonglong, _c_void_p],
    "lego_hip_copy16_stream": [_c_void_p, _c_void_p, ctypes.c_ulonglong, _c_void_p],
    "lego_hip_hbm_probe": [_c_void_p, _c_void_p, ctypes.c_ulonglong, _c_int, _c_int, _c_void_p],
    "lego_hip_mfma_probe": [_c_void_p, _c_void_p, _c_int, _c_int, _c_int, _c_void_p],
    "lego_hip_grouped_gemm_f16_stamps": [_PTR_ARRAY, _PTR_ARRAY, _PTR_ARRAY, _INT_ARRAY, _c_int, _c_void_p],
    "lego_hip_gemm_stamps_read": [_c_void_p, _c_int],
}

_lib = None


class LegoHipError(RuntimeError):
    """A C-ABI entry point returned a non-zero ``hipError_t``."""

    def __init__(self, entry, code):
        super().__init__(f"{entry} failed with hipError_t {code}"
                         + (" (invalid value: null/misaligned pointer or unsupported shape)" if code == 1 else ""))
        self.entry, self.code = entry, code


def load_library(path=None):
    """Load the prebuilt library and set the prototypes.  Raises ``FileNotFoundError`` when it
    was not built."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = Path(path) if path else LIB_PATH
    if not p.exists():
        raise FileNotFoundError(
            f"{p} is missing: build it with `python -m lego_amd.build` (there is no fallback path)")
    lib = ctypes.CDLL(str(p))
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)      # AttributeError if the library does not export the ABI
        fn.argtypes = argtypes
        fn.restype = _c_int
    if path is None:
        _lib = lib
    return lib


_entry_points = {}


def call(entry, *args):
    """Call one entry point and raise ``LegoHipError`` on a non-zero return."""
    fn = _entry_points.get(entry)
    if fn is None:      # looked up once: the wrappers sit in front of kernels of a few microseconds
        fn = _entry_points[entry] = getattr(load_library(), entry)
    code = fn(*args)
    if code != 0:
        raise LegoHipError(entry, code)
