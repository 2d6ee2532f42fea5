"""MI355X-native block-scaled FP4 GEMM behind the ``avelang_kernels`` calling convention."""
from .amdgpu_gemm_fp4 import (  # noqa: F401
    GROUP_K_MXFP4,
    GROUP_K_NVFP4,
    gemm_mxfp4_blocked_scales_transposed_b,
    gemm_mxfp4_swiglu_quant_transposed_b,
    gemm_mxfp4_swiglu_transposed_b,
    gemm_mxfp4_transposed_b,
    gemm_nvfp4_transposed_b,
    grouped_gemm_mxfp4_swiglu_quant_transposed_b,
    grouped_gemm_mxfp4_swiglu_transposed_b,
    grouped_gemm_mxfp4_transposed_b,
    pad_k_mxfp4,
    quantize_mxfp4,
    quantize_nvfp4,
)
from .moe import gather_rows_mxfp4, moe_combine_top2, moe_route_top2  # noqa: F401
from .scale_layout import blocked_numel, scales_from_blocked, scales_to_blocked  # noqa: F401

__all__ = [
    "GROUP_K_MXFP4",
    "GROUP_K_NVFP4",
    "gemm_mxfp4_transposed_b",
    "gemm_mxfp4_blocked_scales_transposed_b",
    "gemm_mxfp4_swiglu_transposed_b",
    "gemm_mxfp4_swiglu_quant_transposed_b",
    "gemm_nvfp4_transposed_b",
    "grouped_gemm_mxfp4_transposed_b",
    "grouped_gemm_mxfp4_swiglu_transposed_b",
    "grouped_gemm_mxfp4_swiglu_quant_transposed_b",
    "pad_k_mxfp4",
    "quantize_mxfp4",
    "quantize_nvfp4",
    "moe_route_top2",
    "moe_combine_top2",
    "gather_rows_mxfp4",
    "blocked_numel",
    "scales_to_blocked",
    "scales_from_blocked",
]
