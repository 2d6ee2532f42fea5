"""ctypes binding of ``libave_fp4.so`` (the C ABI declared in ``include/ave_fp4.h``; the diagnostics of
``include/ave_fp4_debug.h`` for the tests and the benchmark).

The library is loaded from the package directory only, and loading fails loudly:
there is no Python or CPU fallback for any entry point.
"""
from __future__ import annotations

import ctypes
import os

_LIB_NAME = "libave_fp4.so"
_lib = None

AUTO, GENERIC, TILE, DECODE, NARROW, TILE_F16, TILE_STREAMED = 0, 1, 2, 3, 4, 5, 6

_vp = ctypes.c_void_p
_int = ctypes.c_int

#: symbol -> argtypes; every symbol ``include/ave_fp4.h`` and ``include/ave_fp4_debug.h`` declare
SIGNATURES = {
    "ave_fp4_gemm_mxfp4": [_vp, _vp, _vp, _vp, _vp, _int, _int, _int, _vp],
    "ave_fp4_gemm_mxfp4_ex": [_vp, _vp, _vp, _vp, _vp, _int, _int, _int, _vp, _int],
    "ave_fp4_gemm_mxfp4_workspace_bytes": [_int, _int, _int],
    "ave_fp4_gemm_mxfp4_ws": [_vp, _vp, _vp, _vp, _vp, _int, _int, _int, _vp, ctypes.c_size_t, _vp],
    "ave_fp4_gemm_mxfp4_noalloc": [_vp, _vp, _vp, _vp, _vp, _int, _int, _int, _vp],
    "ave_fp4_debug_split_plan": [_int, _int, _int, _int, ctypes.POINTER(_int), ctypes.POINTER(_int), ctypes.POINTER(_int),
                                 ctypes.POINTER(ctypes.c_size_t)],
    "ave_fp4_debug_split_plan_capped": [_int, _int, _int, _int, ctypes.c_size_t, ctypes.POINTER(_int), ctypes.POINTER(_int),
                                        ctypes.POINTER(_int), ctypes.POINTER(ctypes.c_size_t)],
    "ave_fp4_debug_gemm_mxfp4_splitk": [_vp, _vp, _vp, _vp, _vp, _int, _int, _int, _vp, ctypes.c_size_t, _int, _int, _vp],
    "ave_fp4_gemm_mxfp4_swiglu": [_vp, _vp, _vp, _vp, _vp, _int, _int, _int, _vp],
    "ave_fp4_gemm_mxfp4_swiglu_ex": [_vp, _vp, _vp, _vp, _vp, _int, _int, _int, _vp, _int],
    "ave_fp4_gemm_nvfp4": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _vp],
    "ave_fp4_gemm_nvfp4_ex": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _vp, _int],
    "ave_fp4_gemm_nvfp4_workspace_bytes": [_int, _int, _int],
    "ave_fp4_gemm_nvfp4_ws": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _vp, ctypes.c_size_t, _vp],
    "ave_fp4_grouped_gemm_mxfp4": [_vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _vp],
    "ave_fp4_grouped_gemm_mxfp4_ex": [_vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _vp, _int],
    "ave_fp4_gemm_mxfp4_swiglu_quant": [_vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _vp],
    "ave_fp4_grouped_gemm_mxfp4_swiglu": [_vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _vp],
    "ave_fp4_grouped_gemm_mxfp4_swiglu_quant": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _vp],
    "ave_fp4_quantize_mxfp4_f32": [_vp, _vp, _vp, _int, _int, _vp],
    "ave_fp4_quantize_mxfp4_bf16": [_vp, _vp, _vp, _int, _int, _vp],
    "ave_fp4_quantize_mxfp4_f32_padded": [_vp, _vp, _vp, _int, _int, _int, _vp],
    "ave_fp4_quantize_mxfp4_bf16_padded": [_vp, _vp, _vp, _int, _int, _int, _vp],
    "ave_fp4_gemm_mxfp4_swiglu_quant_padded": [_vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _vp],
    "ave_fp4_grouped_gemm_mxfp4_swiglu_quant_padded": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _int, _vp],
    "ave_fp4_quantize_nvfp4_f32": [_vp, _vp, _vp, _vp, _int, _int, _vp],
    "ave_fp4_quantize_nvfp4_bf16": [_vp, _vp, _vp, _vp, _int, _int, _vp],
    "ave_fp4_moe_route_top2": [_vp, _int, _int, _vp, _vp, _vp, _vp],
    "ave_fp4_moe_route_top2_ex": [_vp, _int, _int, _vp, _vp, _vp, _vp, _vp],
    "ave_fp4_moe_combine_top2": [_vp, _vp, _vp, _int, _int, _int, _vp, _vp],
    "ave_fp4_gather_rows_mxfp4": [_vp, _vp, _vp, _int, _int, _int, _vp, _vp, _vp],
    "ave_fp4_scales_to_blocked": [_vp, _int, _int, _vp, _vp],
    "ave_fp4_scales_from_blocked": [_vp, _int, _int, _vp, _vp],
    "ave_fp4_gemm_mxfp4_blocked_scales": [_vp, _vp, _vp, _vp, _vp, _int, _int, _int, _vp],
    "ave_fp4_last_error": [],
    "ave_fp4_abi_version": [],
    "ave_fp4_debug_weights_from_hbm": [_vp, ctypes.c_size_t],
    "ave_fp4_debug_tiles_per_workgroup": [_int, _int, _int, _int],
    "ave_fp4_debug_map_tile": [_int, _int, _int, ctypes.POINTER(_int), ctypes.POINTER(_int)],
    "ave_fp4_debug_locate_group_tile": [ctypes.POINTER(ctypes.c_int32), _int, _int, _int, _int, ctypes.POINTER(_int),
                                        ctypes.POINTER(_int), ctypes.POINTER(_int)],
    "ave_fp4_debug_generic_grid": [_int, _int, _int, ctypes.POINTER(ctypes.c_uint)],
    "ave_fp4_debug_stream_read": [_vp, ctypes.c_size_t, _int, _vp, _vp],
    "ave_fp4_debug_stream_read_write": [_vp, ctypes.c_size_t, _vp, ctypes.c_size_t, _int, _vp, _vp],
    "ave_fp4_debug_mfma_rate": [_vp, ctypes.c_size_t, _int, _int, _vp, _vp, ctypes.POINTER(ctypes.c_double)],
    "ave_fp4_debug_mfma_rate_f16": [_vp, ctypes.c_size_t, _int, _int, _vp, _vp, ctypes.POINTER(ctypes.c_double)],
}


ABI_VERSION = 1   # what ave_fp4_abi_version() of a matching library returns

_RESTYPES = {"ave_fp4_last_error": ctypes.c_char_p, "ave_fp4_gemm_mxfp4_workspace_bytes": ctypes.c_size_t,
             "ave_fp4_gemm_nvfp4_workspace_bytes": ctypes.c_size_t}


def library_path() -> str:
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), _LIB_NAME)


def load() -> ctypes.CDLL:
    """Load the shared library once; raise ``RuntimeError`` if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not os.path.exists(path):
        raise RuntimeError(
            f"{_LIB_NAME} not found at {path}: build it with `make -C avelang_amd/csrc` "
            "(or __graft_entry__.build()); there is no fallback path."
        )
    lib = ctypes.CDLL(path)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.argtypes = argtypes
        fn.restype = _RESTYPES.get(name, _int)
    if lib.ave_fp4_abi_version() != ABI_VERSION:
        raise RuntimeError(f"{path} has ABI version {lib.ave_fp4_abi_version()}, this package binds version "
                           f"{ABI_VERSION}: rebuild it with `make -C avelang_amd/csrc`")
    _lib = lib
    return lib


def last_error() -> str:
    return load().ave_fp4_last_error().decode("utf-8", "replace")


def check(rc: int) -> None:
    """0 -> ok; AVE_FP4_EINVAL -> ValueError; a hipError_t -> RuntimeError, the
    reference's convention for HIP failures (backends/amdgpu/driver.py:125-138)."""
    if rc == 0:
        return
    msg = last_error()
    if rc == -1:
        raise ValueError(msg)
    raise RuntimeError(msg or f"ave-lang Error [HIP]: error {rc}")
