"""Grouped (MoE) GEMMs with more than 64 experts.  Up to 256 experts -- what the routing kernel takes -- the LDS-staged
kernels find a tile's expert in a table of their own (the 256 x 256 kernel in LDS, the narrow-tile kernel in registers;
a lane looks at experts l, l + 64, l + 128, l + 192); above that they walk the caller's row table entry by entry, and
the persistent kernels keep the host's bound on the tile list (rows / tile + experts slots, most of them behind the
last tile).

Every case: most experts empty, a few ragged ones, small N, K = 512 (whole pairs of stages) or a K with a tail.  Every
expert's rows must equal the plain call on that expert bit for bit, whichever kernel runs the grouped launch, and
the whole result must lie within the stated tolerance of the fp64 grouped oracle."""
import numpy as np
import pytest
import torch

from avelang_amd import (gemm_mxfp4_swiglu_transposed_b, grouped_gemm_mxfp4_swiglu_quant_transposed_b,
                         grouped_gemm_mxfp4_swiglu_transposed_b, quantize_mxfp4)
from oracle import fp4_oracle as orc
from tests import helpers as H

pytestmark = pytest.mark.gpu
GENERIC, TILE, NARROW = 1, 2, 4


def _offsets(experts, rows_of, seed):
    """row_offsets for `experts` experts of which those in `rows_of` (expert -> rows) are not empty."""
    rows = np.zeros(experts, dtype=np.int64)
    for e, r in rows_of.items():
        rows[e] = r
    return np.concatenate([[0], np.cumsum(rows)]).astype(np.int32)


# (experts, {expert: rows}, N, K): first and last expert used, neighbours, one with several 256-row tiles
CASES = [
    (65, {0: 3, 1: 300, 31: 129, 63: 1, 64: 257}, 72, 512),
    (96, {5: 700, 64: 64, 65: 65, 95: 2}, 136, 736),            # K tail: 512 + 7 blocks
    (256, {0: 1, 100: 513, 128: 31, 254: 128, 255: 260}, 40, 512),
    (256, {17: 40, 200: 90}, 264, 1056),                          # two small experts, K tail: 1024 + 1 block
    (300, {0: 5, 150: 300, 299: 130}, 40, 512),                   # more experts than the kernels' tables hold: the walk
    (200, {e: 3 + e % 5 for e in range(0, 200, 3)}, 48, 512),     # every set of 64 experts has rows, none has many
]


def _operands(experts, rows_of, n, k, seed, gate_up=False):
    ro = _offsets(experts, rows_of, seed)
    total = int(ro[-1])
    a, a_s = H.mx_operand(total, k, seed=seed)
    wn = (2 if gate_up else 1) * n
    b, b_s = H.mx_operand(experts * wn, k, seed=seed + 1, std=0.05)
    return ro, a, a_s, b.reshape(experts, wn, k // 2), b_s.reshape(experts, wn, k // 32)


@pytest.mark.parametrize("experts,rows_of,n,k", CASES)
def test_grouped_gemm_many_experts_equals_per_expert_calls(gpu, experts, rows_of, n, k):
    ro, a, a_s, b, b_s = _operands(experts, rows_of, n, k, seed=300 + experts)
    tile = H.run_grouped(gpu, a, a_s, b, b_s, ro, variant=TILE)
    narrow = H.run_grouped(gpu, a, a_s, b, b_s, ro, variant=NARROW)
    auto = H.run_grouped(gpu, a, a_s, b, b_s, ro)
    generic = H.run_grouped(gpu, a, a_s, b, b_s, ro, variant=GENERIC)
    for e in rows_of:
        r0, r1 = int(ro[e]), int(ro[e + 1])
        # the 256 x 256 kernel, forced: bit for bit what it gives for the expert alone
        assert np.array_equal(H.run_mx(gpu, a[r0:r1], a_s[r0:r1], b[e], b_s[e], variant=TILE), tile[r0:r1]), e
        assert np.array_equal(H.run_mx(gpu, a[r0:r1], a_s[r0:r1], b[e], b_s[e], variant=NARROW), narrow[r0:r1]), e
    if k % 512 == 0:   # the two LDS-staged kernels add K up in the same order (their K tails do not)
        assert np.array_equal(tile, narrow)
    assert np.array_equal(auto, narrow if ro[-1] <= 128 * experts else tile)
    want = orc.grouped_gemm_mxfp4_fp64(a, a_s, b, b_s, ro)
    adq = orc.dequantize_mxfp4(a, a_s, np.float64)
    for c in (tile, narrow, generic):
        for e in rows_of:
            r0, r1 = int(ro[e]), int(ro[e + 1])
            bdq = orc.dequantize_mxfp4(b[e], b_s[e], np.float64)
            ok, rep = orc.check_bf16_against_fp64(c[r0:r1], want[r0:r1], np.abs(adq[r0:r1]) @ np.abs(bdq).T, k)
            assert ok, (e, rep)


@pytest.mark.parametrize("experts,rows_of,n,k", [
    (65, {0: 3, 1: 300, 31: 129, 63: 1, 64: 257}, 64, 512),        # at most 128 rows per expert on average: narrow tiles
    (96, {5: 700, 64: 64, 65: 65, 95: 2}, 96, 736),
    (256, {0: 1, 100: 513, 128: 31, 254: 128, 255: 260}, 32, 512),
    (65, {2: 4000, 40: 3000, 64: 1500}, 64, 512),                  # more than 128 rows per expert: the 256 x 256 kernel
    (96, {0: 6000, 70: 5000, 95: 1400}, 32, 1056),                 # ... with a K tail
])
def test_grouped_swiglu_many_experts_with_and_without_the_quantiser(gpu, experts, rows_of, n, k):
    ro, a, a_s, b, b_s = _operands(experts, rows_of, n, k, seed=400 + experts, gate_up=True)
    da, das, db, dbs = (H.to_dev(v, gpu) for v in (a, a_s, b, b_s))
    dro = torch.from_numpy(ro).to(gpu)
    c = grouped_gemm_mxfp4_swiglu_transposed_b(da, das, db, dbs, dro)
    q, q_s = grouped_gemm_mxfp4_swiglu_quant_transposed_b(da, das, db, dbs, dro)
    torch.cuda.synchronize()
    narrow = int(ro[-1]) <= 128 * experts   # what shape-based dispatch takes: narrow tiles up to 128 rows per expert on average
    for e in rows_of:
        r0, r1 = int(ro[e]), int(ro[e + 1])
        # (copies, not views: a row range of a scale tensor whose rows are no multiple of 16 bytes starts unaligned)
        alone = gemm_mxfp4_swiglu_transposed_b(da[r0:r1].clone(), das[r0:r1].clone(), db[e].clone(), dbs[e].clone(),
                                               variant=NARROW if narrow else TILE)
        assert torch.equal(alone, c[r0:r1]), e
        ok, rep = orc.check_swiglu_bf16(H.bits(c[r0:r1]), a[r0:r1], a_s[r0:r1], b[e], b_s[e])
        assert ok, (e, rep)
    want_q, want_s = quantize_mxfp4(c)
    assert torch.equal(q, want_q) and torch.equal(q_s, want_s)


@pytest.mark.parametrize("experts,rows_of,n,k", [
    (8, {0: 16, 1: 130, 2: 1, 3: 77, 5: 128, 6: 40, 7: 129}, 6144, 1024),     # 10 m-tiles x 48 n-tiles: two rounds
    (70, {0: 5, 9: 33, 30: 128, 31: 2, 64: 100, 69: 17}, 8192, 736),          # 70 experts: two per lane of the register table; K tail
])
def test_grouped_narrow_tiles_over_several_rounds_of_the_persistent_walk(gpu, experts, rows_of, n, k):
    """More 128-row tiles than compute units: the grouped narrow-tile kernel's workgroups walk several tiles each and
    request a tile's first stages while the previous tile's results leave.  Every expert's rows must equal the plain call
    on the same kernel bit for bit (plain, with SwiGLU, with SwiGLU and the quantiser) and lie within tolerance of the
    oracle."""
    ro = _offsets(experts, rows_of, 0)
    total = int(ro[-1])
    assert total <= 128 * experts   # what sends shape-based dispatch to the narrow tiles
    a, a_s = H.mx_operand(total, k, seed=500 + experts)
    b, b_s = H.mx_operand(experts * n, k, seed=501 + experts, std=0.05)
    b, b_s = b.reshape(experts, n, k // 2), b_s.reshape(experts, n, k // 32)
    c = H.run_grouped(gpu, a, a_s, b, b_s, ro)
    assert np.array_equal(c, H.run_grouped(gpu, a, a_s, b, b_s, ro, variant=NARROW))
    for e in rows_of:
        r0, r1 = int(ro[e]), int(ro[e + 1])
        assert np.array_equal(H.run_mx(gpu, a[r0:r1], a_s[r0:r1], b[e], b_s[e], variant=NARROW), c[r0:r1]), e
        H.assert_mx_close(c[r0:r1], a[r0:r1], a_s[r0:r1], b[e], b_s[e])
    # the same weights as N/2 gate rows followed by N/2 up rows per expert
    da, das, db, dbs = (H.to_dev(v, gpu) for v in (a, a_s, b, b_s))
    dro = torch.from_numpy(ro).to(gpu)
    cs = grouped_gemm_mxfp4_swiglu_transposed_b(da, das, db, dbs, dro)
    q, q_s = grouped_gemm_mxfp4_swiglu_quant_transposed_b(da, das, db, dbs, dro)
    torch.cuda.synchronize()
    for e in rows_of:
        r0, r1 = int(ro[e]), int(ro[e + 1])
        alone = gemm_mxfp4_swiglu_transposed_b(da[r0:r1].clone(), das[r0:r1].clone(), db[e].clone(), dbs[e].clone(), variant=NARROW)
        assert torch.equal(alone, cs[r0:r1]), e
    want_q, want_s = quantize_mxfp4(cs)
    assert torch.equal(q, want_q) and torch.equal(q_s, want_s)
