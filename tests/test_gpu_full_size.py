"""Parity at the full benchmark sizes, where a CPU reference of the whole problem would take too
long: size-independent properties plus sampled rows against the fp64 oracle.

* sampled rows: C[rows] must meet the stated tolerance against the oracle for those rows;
* exponent shift: adding 1 to every E8M0 byte of A doubles every product, so C must double exactly
  (bf16 bit patterns move by one exponent step);
* row permutation: permuting the rows of A permutes the rows of C bit for bit;
* kernel agreement: the LDS-staged kernel and the shape-agnostic kernel meet the tolerance on the
  same sampled rows (they sum in different orders, so bit equality is not required).
"""
import numpy as np
import pytest
import torch

from avelang_amd import (gemm_mxfp4_transposed_b, gemm_nvfp4_transposed_b, grouped_gemm_mxfp4_transposed_b)
from avelang_amd import testing as synth
from oracle import fp4_oracle as orc
from tests import helpers as H

pytestmark = pytest.mark.gpu
GENERIC = 1


def _check_rows_mx(c, a, a_s, b, b_s, rows):
    a_np, as_np = a[rows].cpu().numpy(), a_s[rows].cpu().numpy()
    H.assert_mx_close(H.bits(c[rows]), a_np, as_np, b.cpu().numpy(), b_s.cpu().numpy())


def test_prefill_8192x14336x4096(gpu):
    m, n, k = 8192, 14336, 4096
    g = torch.Generator(device=gpu).manual_seed(0)
    a, a_s = synth.quantize_mxfp4(synth.activations_with_outliers(m, k, g, gpu))
    b, b_s = synth.quantize_mxfp4(torch.randn((n, k), generator=g, device=gpu) * 0.02)
    c = gemm_mxfp4_transposed_b(a, a_s, b, b_s)
    rows = torch.tensor([0, 1, 255, 256, 4095, 4096, 8191] + list(range(1000, 1025)), device=gpu)
    _check_rows_mx(c, a, a_s, b, b_s, rows)
    # exponent shift (scales stay far from the E8M0 ends for this data)
    c2 = gemm_mxfp4_transposed_b(a, a_s + 1, b, b_s)
    assert torch.equal(c2.float(), c.float() * 2)
    # row permutation
    perm = torch.randperm(m, generator=g, device=gpu)
    c3 = gemm_mxfp4_transposed_b(a[perm].contiguous(), a_s[perm].contiguous(), b, b_s)
    assert torch.equal(c3.view(torch.uint16), c[perm].view(torch.uint16))
    # the shape-agnostic kernel on a slice of the same problem
    cg = gemm_mxfp4_transposed_b(a[rows].contiguous(), a_s[rows].contiguous(), b, b_s, variant=GENERIC)
    H.assert_mx_close(H.bits(cg), a[rows].cpu().numpy(), a_s[rows].cpu().numpy(), b.cpu().numpy(), b_s.cpu().numpy())


def test_decode_16x28672x4096(gpu):
    m, n, k = 16, 28672, 4096
    g = torch.Generator(device=gpu).manual_seed(2)
    a, a_s = synth.quantize_mxfp4(torch.randn((m, k), generator=g, device=gpu))
    b, b_s = synth.quantize_mxfp4(torch.randn((n, k), generator=g, device=gpu) * 0.02)
    c = gemm_mxfp4_transposed_b(a, a_s, b, b_s)
    H.assert_mx_close(H.bits(c), a.cpu().numpy(), a_s.cpu().numpy(), b.cpu().numpy(), b_s.cpu().numpy())
    c2 = gemm_mxfp4_transposed_b(a, a_s, b, b_s + 1)
    assert torch.equal(c2.float(), c.float() * 2)


def test_nvfp4_4096x4096x14336(gpu):
    m, n, k = 4096, 4096, 14336
    g = torch.Generator(device=gpu).manual_seed(3)
    a, a_s, a_g = synth.quantize_nvfp4(torch.randn((m, k), generator=g, device=gpu))
    b, b_s, b_g = synth.quantize_nvfp4(torch.randn((n, k), generator=g, device=gpu) * 0.02)
    c = gemm_nvfp4_transposed_b(a, a_s, a_g, b, b_s, b_g)
    rows = torch.tensor([0, 31, 32, 2047, 4095] + list(range(500, 511)), device=gpu)
    H.assert_nv_close(H.bits(c[rows]), a[rows].cpu().numpy(), a_s[rows].cpu().numpy(), a_g.item(), b.cpu().numpy(),
                      b_s.cpu().numpy(), b_g.item())
    # per-tensor scale is linear: doubling A_global doubles C exactly
    c2 = gemm_nvfp4_transposed_b(a, a_s, a_g * 2, b, b_s, b_g)
    assert torch.equal(c2.float(), c.float() * 2)
    perm = torch.randperm(m, generator=g, device=gpu)
    c3 = gemm_nvfp4_transposed_b(a[perm].contiguous(), a_s[perm].contiguous(), a_g, b, b_s, b_g)
    assert torch.equal(c3.view(torch.uint16), c[perm].view(torch.uint16))


def test_grouped_moe_8_experts_top2(gpu):
    tokens, experts, top_k, n, k = 16384, 8, 2, 14336, 4096
    g = torch.Generator(device=gpu).manual_seed(4)
    x = torch.randn((tokens, k), generator=g, device=gpu)
    token_of_row, row_offsets = synth.moe_routing(tokens, experts, top_k, g, gpu)
    a, a_s = synth.quantize_mxfp4(x[token_of_row])
    del x
    qs = [synth.quantize_mxfp4(torch.randn((n, k), generator=g, device=gpu) * 0.02) for _ in range(experts)]
    b, b_s = torch.stack([q[0] for q in qs]), torch.stack([q[1] for q in qs])
    c = grouped_gemm_mxfp4_transposed_b(a, a_s, b, b_s, row_offsets)
    ro = row_offsets.cpu().numpy()
    assert ro[0] == 0 and ro[-1] == tokens * top_k
    for e in range(experts):
        r0, r1 = int(ro[e]), int(ro[e + 1])
        # first, last and a few interior rows of every expert (the last tile of an expert is ragged)
        rows = torch.tensor(sorted({r0, r0 + 1, (r0 + r1) // 2, r1 - 2, r1 - 1}), device=gpu)
        H.assert_mx_close(H.bits(c[rows]), a[rows].cpu().numpy(), a_s[rows].cpu().numpy(), b[e].cpu().numpy(),
                          b_s[e].cpu().numpy())
    # grouped == plain GEMM per expert, bit for bit (same kernel, same tile walk inside an expert)
    e = 3
    r0, r1 = int(ro[e]), int(ro[e + 1])
    plain = gemm_mxfp4_transposed_b(a[r0:r1].contiguous(), a_s[r0:r1].contiguous(), b[e], b_s[e], variant=2)
    assert torch.equal(plain.view(torch.uint16), c[r0:r1].view(torch.uint16))


@pytest.mark.parametrize("m,n,k", [(128, 28672, 4096), (256, 28672, 4096), (128, 4096, 14336), (512, 4096, 14336)])
def test_decode_batch_shapes_at_full_size(gpu, m, n, k):
    """A few hundred rows against the gate/up and the down projection's weights: the narrow-tile kernel, and its K split
    through a workspace.  Sampled rows against the oracle, the exponent shift (exact for both: every partial sum
    doubles), and agreement with the one-launch 256 x 256 kernel -- bit for bit without the split, within the
    tolerance of both with it."""
    g = torch.Generator(device=gpu).manual_seed(m + n)
    a, a_s = synth.quantize_mxfp4(synth.activations_with_outliers(m, k, g, gpu))
    b, b_s = synth.quantize_mxfp4(torch.randn((n, k), generator=g, device=gpu) * 0.02)
    c = gemm_mxfp4_transposed_b(a, a_s, b, b_s)
    rows = torch.tensor([0, 1, 63, 64, m // 2, m - 1], device=gpu)
    _check_rows_mx(c, a, a_s, b, b_s, rows)
    c2 = gemm_mxfp4_transposed_b(a, a_s, b, b_s + 1)
    assert torch.equal(c2.float(), c.float() * 2)
    wide = gemm_mxfp4_transposed_b(a, a_s, b, b_s, variant=2)
    unsplit = gemm_mxfp4_transposed_b(a, a_s, b, b_s, split_k=False)
    assert torch.equal(unsplit.view(torch.uint16), wide.view(torch.uint16))
    _check_rows_mx(wide, a, a_s, b, b_s, rows)


@pytest.mark.parametrize("m,n,k", [(16, 28672, 4096), (64, 4096, 14336), (128, 4096, 14336)])
def test_nvfp4_decode_batch_shapes_at_full_size(gpu, m, n, k):
    """The NVFP4 weight-streaming kernel (16 and 64 rows) and the K split of the tile kernel (128 rows): all rows
    against the oracle, and doubling one per-tensor scale doubles the result exactly."""
    g = torch.Generator(device=gpu).manual_seed(m + k)
    a, a_s, a_g = synth.quantize_nvfp4(torch.randn((m, k), generator=g, device=gpu))
    b, b_s, b_g = synth.quantize_nvfp4(torch.randn((n, k), generator=g, device=gpu) * 0.02)
    c = gemm_nvfp4_transposed_b(a, a_s, a_g, b, b_s, b_g)
    rows = list(range(0, m, max(1, m // 8)))
    H.assert_nv_close(H.bits(c[rows]), a[rows].cpu().numpy(), a_s[rows].cpu().numpy(), float(a_g), b.cpu().numpy(),
                      b_s.cpu().numpy(), float(b_g))
    c2 = gemm_nvfp4_transposed_b(a, a_s, a_g * 2, b, b_s, b_g)
    assert torch.equal(c2.float(), c.float() * 2)
