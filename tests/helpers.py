"""Shared helpers for the parity tests (CPU side: oracle; GPU side: the C ABI through
the package's wrappers)."""
from __future__ import annotations

import numpy as np

from oracle import fp4_oracle as orc


def mx_operand(rows, k, seed, std=1.0, outliers=False):
    x = orc.activations_with_outliers(rows, k, seed) if outliers else orc.randn((rows, k), seed, std)
    packed, scales = orc.quantize_mxfp4(x)
    return packed, scales


def nv_operand(rows, k, seed, std=1.0):
    x = orc.randn((rows, k), seed, std)
    return orc.quantize_nvfp4(x)


def to_dev(arr, device):
    import torch

    return torch.from_numpy(np.ascontiguousarray(arr)).to(device)


def bits(t):
    """bf16 torch tensor -> numpy uint16 bit patterns."""
    import torch

    return t.view(torch.uint16).cpu().numpy()


def run_mx(device, a, a_s, b, b_s, variant=0, out=None):
    from avelang_amd import gemm_mxfp4_transposed_b

    c = gemm_mxfp4_transposed_b(to_dev(a, device), to_dev(a_s, device), to_dev(b, device), to_dev(b_s, device),
                                out=out, variant=variant)
    return bits(c)


def run_nv(device, a, a_s, a_g, b, b_s, b_g, variant=0):
    import torch
    from avelang_amd import gemm_nvfp4_transposed_b

    ag = torch.tensor([a_g], dtype=torch.float32, device=device)
    bg = torch.tensor([b_g], dtype=torch.float32, device=device)
    c = gemm_nvfp4_transposed_b(to_dev(a, device), to_dev(a_s, device), ag, to_dev(b, device), to_dev(b_s, device),
                                bg, variant=variant)
    return bits(c)


def run_grouped(device, a, a_s, b, b_s, row_offsets, variant=0):
    from avelang_amd import grouped_gemm_mxfp4_transposed_b

    c = grouped_gemm_mxfp4_transposed_b(to_dev(a, device), to_dev(a_s, device), to_dev(b, device),
                                        to_dev(b_s, device), to_dev(np.asarray(row_offsets, dtype=np.int32), device),
                                        variant=variant)
    return bits(c)


def assert_mx_close(c_bits, a, a_s, b, b_s):
    """Stated tolerance: |c - ref64| <= 1 bf16 ulp + K*2^-24*sum|a||b| per element, and
    max relative error per row <= 2^-7."""
    adq = orc.dequantize_mxfp4(a, a_s, np.float64)
    bdq = orc.dequantize_mxfp4(b, b_s, np.float64)
    ref = adq @ bdq.T
    ok, rep = orc.check_bf16_against_fp64(c_bits, ref, np.abs(adq) @ np.abs(bdq).T, a.shape[1] * 2)
    assert ok, rep
    return rep


def assert_nv_close(c_bits, a, a_s, a_g, b, b_s, b_g):
    adq = orc.dequantize_nvfp4_block(a, a_s, np.float64)
    bdq = orc.dequantize_nvfp4_block(b, b_s, np.float64)
    g = np.float64(np.float32(a_g)) * np.float64(np.float32(b_g))
    ref = (adq @ bdq.T) * g
    # one extra fp32 rounding for the per-tensor scale product and one for its application
    ok, rep = orc.check_bf16_against_fp64(c_bits, ref, (np.abs(adq) @ np.abs(bdq).T) * abs(g), a.shape[1] * 2 + 2)
    assert ok, rep
    return rep
