"""Block-scaled FP4 GEMM for AMD MI355X under the reference's import path: the module a caller written against
``avelang_kernels.amdgpu_gemm.gemm_pipeline_transposed_b`` (reference ``python/avelang_kernels/amdgpu_gemm.py:458-494``)
imports for FP4 operands.

    from avelang_kernels.amdgpu_gemm_fp4 import gemm_mxfp4_transposed_b
    C = gemm_mxfp4_transposed_b(A, A_scale, B, B_scale)          # bf16 [M, N] = A . B^T, like the bf16 entry point

Same conventions as the reference entry point -- ``ValueError`` before anything is launched, ``out=`` semantics,
asynchronous launch on torch's current stream, no allocation at launch -- and the calls go through the pybind11
extension ``_ave_fp4_bindings`` (built from ``python/src/ave_fp4_bindings.cc``, linked against ``libave_fp4.so``), the
counterpart of the reference's ``_avelang_bindings`` module (``python/src/avelang_bindings.cc:493-529``), with the GIL
released around every launch (``python/avelang/backends/amdgpu/driver.py:357-359``).  The operand checks are those
of :mod:`avelang_amd.amdgpu_gemm_fp4`, which calls the same library through ctypes.
"""
from __future__ import annotations

import functools
import os
import sys

_ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
if _ROOT not in sys.path:   # the package with the operand checks lives at the root of this tree
    sys.path.insert(0, _ROOT)

from avelang_amd import amdgpu_gemm_fp4 as _impl  # noqa: E402
from avelang_amd._lib import ABI_VERSION  # noqa: E402

try:
    from . import _ave_fp4_bindings as _ext
except ImportError as exc:  # no fallback: without the extension this module does not import
    raise ImportError(
        "avelang_kernels._ave_fp4_bindings is not built: run `make -C avelang_amd/csrc` (or __graft_entry__.build()); "
        "avelang_amd.amdgpu_gemm_fp4 offers the same entry points through ctypes."
    ) from exc

if _ext.ave_fp4_abi_version() != ABI_VERSION:
    raise ImportError(f"_ave_fp4_bindings is linked against ABI version {_ext.ave_fp4_abi_version()} of libave_fp4.so, "
                      f"this package binds version {ABI_VERSION}: rebuild with `make -C avelang_amd/csrc`")

GROUP_K_MXFP4 = _impl.GROUP_K_MXFP4
GROUP_K_NVFP4 = _impl.GROUP_K_NVFP4


def _through_extension(fn):
    bound = functools.partial(fn, lib=_ext)
    functools.update_wrapper(bound, fn)
    return bound


gemm_mxfp4_transposed_b = _through_extension(_impl.gemm_mxfp4_transposed_b)
gemm_nvfp4_transposed_b = _through_extension(_impl.gemm_nvfp4_transposed_b)
grouped_gemm_mxfp4_transposed_b = _through_extension(_impl.grouped_gemm_mxfp4_transposed_b)
gemm_mxfp4_blocked_scales_transposed_b = _through_extension(_impl.gemm_mxfp4_blocked_scales_transposed_b)

__all__ = ["GROUP_K_MXFP4", "GROUP_K_NVFP4", "gemm_mxfp4_transposed_b", "gemm_nvfp4_transposed_b",
           "grouped_gemm_mxfp4_transposed_b", "gemm_mxfp4_blocked_scales_transposed_b"]
