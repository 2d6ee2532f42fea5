"""The pybind11 extension under the reference's import path (``python/avelang_kernels``): what it exports and how it
treats arguments, without a GPU.  Conventions being mirrored: pointer arguments are ints, None or objects with
``data_ptr()`` (reference python/avelang/backends/amdgpu/driver.py:154-189); errors raise ``ValueError`` /
``RuntimeError`` (python/src/avelang_bindings.cc:44,131-133)."""
import os
import re

import pytest
import torch

from avelang_amd import _lib
from avelang_kernels import _ave_fp4_bindings as ext
from avelang_kernels import amdgpu_gemm_fp4 as ak

HEADER = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "ave_fp4.h")


def test_extension_binds_the_c_abi_of_the_header():
    declared = set(re.findall(r"\b(ave_fp4_\w+)\s*\(", open(HEADER).read()))
    bound = {n for n in dir(ext) if n.startswith("ave_fp4_")}
    assert bound <= declared
    # every entry point that launches a GEMM or a quantiser is bound; diagnostics and MoE helpers stay with ctypes
    for name in declared:
        if re.match(r"ave_fp4_(grouped_)?gemm_|ave_fp4_quantize_", name):
            assert name in bound, name
    assert ext.ave_fp4_abi_version() == _lib.ABI_VERSION == _lib.load().ave_fp4_abi_version()


def test_pointer_arguments_and_error_types():
    class HasPtr:
        def data_ptr(self):
            return 64

    class BadPtr:
        def data_ptr(self):
            return "nope"

    assert ext.ave_fp4_gemm_mxfp4(HasPtr(), 64, HasPtr(), 64, 64, 0, 8, 32, None) == 0      # M = 0: nothing to launch
    with pytest.raises(ValueError, match="K must be a positive multiple of 32, got 33"):
        ext.ave_fp4_gemm_mxfp4(64, 64, 64, 64, 64, 4, 4, 33, None)
    assert "got 33" in ext.ave_fp4_last_error()
    with pytest.raises(ValueError, match="null device pointer"):
        ext.ave_fp4_gemm_mxfp4(None, 64, 64, 64, 64, 4, 4, 32, None)
    with pytest.raises(TypeError, match="either uint64 or have data_ptr"):
        ext.ave_fp4_gemm_mxfp4("A", 64, 64, 64, 64, 4, 4, 32, None)
    with pytest.raises(TypeError, match="must return 64-bit int"):
        ext.ave_fp4_gemm_mxfp4(BadPtr(), 64, 64, 64, 64, 4, 4, 32, None)
    with pytest.raises(ValueError, match="unknown kernel variant"):
        ext.ave_fp4_gemm_nvfp4_ex(64, 64, 64, 64, 64, 64, 64, 4, 4, 32, None, 99)


def test_reference_path_module_validates_like_the_reference():
    a = torch.zeros((4, 16), dtype=torch.uint8)
    s = torch.zeros((4, 1), dtype=torch.uint8)
    with pytest.raises(ValueError, match="K must be a multiple of 32, got 24"):
        ak.gemm_mxfp4_transposed_b(a[:, :12].contiguous(), s, a[:, :12].contiguous(), s)
    with pytest.raises(ValueError, match="ROCm GPU"):
        ak.gemm_mxfp4_transposed_b(a, s, a, s)
    with pytest.raises(ValueError, match="3-D"):
        ak.grouped_gemm_mxfp4_transposed_b(a, s, a, s, torch.zeros(2, dtype=torch.int32))
    with pytest.raises(ValueError, match="K must be a multiple of 16"):
        ak.gemm_nvfp4_transposed_b(a[:, :4].contiguous(), s, torch.ones(1), a[:, :4].contiguous(), s, torch.ones(1))
    assert ak.gemm_mxfp4_transposed_b.__doc__.startswith("MXFP4 GEMM")
