"""Kernel library of the avelang Python package (reference: ``python/avelang_kernels/``, which holds
``amdgpu_gemm.py``).  This tree adds the block-scaled FP4 GEMM beside it: :mod:`avelang_kernels.amdgpu_gemm_fp4`."""
