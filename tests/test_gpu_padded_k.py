"""Operands padded along K with zero blocks.  A K whose packed rows are no multiple of 128 bytes (2880, 4128) costs the
LDS-staged kernels' main loop about a quarter more per stage; padded to a multiple of 512 the same sums run at the
padded length's speed.  The quantiser and the fused quantising epilogues write into padded rows directly, so the
activations need no copy; weights are padded once with ``pad_k_mxfp4``.

What is checked: the padded quantiser gives the plain quantiser's bytes followed by zero blocks; the fused epilogues
write the unpadded call's bytes into the first N columns and leave the padding alone; a GEMM over padded operands equals
the unpadded GEMM within the stated tolerance of the fp64 oracle on the UNPADDED operands, and exactly on operands whose
sums are exact in fp32; a two-GEMM MLP block with K = 2880 runs end to end on padded rows."""
import numpy as np
import pytest
import torch

from avelang_amd import (gemm_mxfp4_swiglu_quant_transposed_b, gemm_mxfp4_transposed_b,
                         grouped_gemm_mxfp4_swiglu_quant_transposed_b, pad_k_mxfp4, quantize_mxfp4)
from oracle import fp4_oracle as orc
from tests import helpers as H

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,k,k_pad", [(1, 32, 64), (5, 96, 512), (33, 2880, 3072), (257, 4128, 4608), (16, 512, 512)])
def test_padded_quantiser_is_the_plain_one_followed_by_zero_blocks(gpu, dtype, rows, k, k_pad):
    g = torch.Generator(device="cpu").manual_seed(rows * 131 + k)
    x = (torch.randn((rows, k), generator=g) * 3).to(dtype).to(gpu)
    q, s = quantize_mxfp4(x)
    # buffers that hold something else beforehand: every padded byte must be written
    qp = torch.full((rows, k_pad // 2), 0xAB, dtype=torch.uint8, device=gpu)
    sp = torch.full((rows, k_pad // 32), 0xCD, dtype=torch.uint8, device=gpu)
    got_q, got_s = quantize_mxfp4(x, qp, sp, k_pad=k_pad)
    assert got_q is qp and got_s is sp
    assert torch.equal(qp[:, :k // 2], q) and torch.equal(sp[:, :k // 32], s)
    assert int(qp[:, k // 2:].max().item() if k_pad > k else 0) == 0
    assert k_pad == k or bool((sp[:, k // 32:] == 127).all())
    want_q, want_s = pad_k_mxfp4(q, s, k_pad)
    assert torch.equal(qp, want_q) and torch.equal(sp, want_s)


def test_padded_quantiser_rejects_bad_padding(gpu):
    x = torch.zeros((4, 64), dtype=torch.float32, device=gpu)
    for bad in (32, 80, 63):
        with pytest.raises(ValueError, match="k_pad must be a multiple of 32 and at least 64"):
            quantize_mxfp4(x, k_pad=bad)
    with pytest.raises(ValueError, match="packed must have shape"):
        quantize_mxfp4(x, torch.empty((4, 32), dtype=torch.uint8, device=gpu), k_pad=128)


@pytest.mark.parametrize("m,n,k", [(200, 2880, 2880), (16, 736, 4128), (300, 520, 992)])
def test_gemm_over_padded_operands_matches_the_unpadded_one(gpu, m, n, k):
    k_pad = (k + 511) // 512 * 512
    a, a_s = H.mx_operand(m, k, seed=m + k)
    b, b_s = H.mx_operand(n, k, seed=n + k + 1, std=0.05)
    da, das, db, dbs = (H.to_dev(v, gpu) for v in (a, a_s, b, b_s))
    c = gemm_mxfp4_transposed_b(da, das, db, dbs)
    pa, pas = pad_k_mxfp4(da, das, k_pad)
    pb, pbs = pad_k_mxfp4(db, dbs, k_pad)
    assert pa.shape == (m, k_pad // 2) and pbs.shape == (n, k_pad // 32)
    cp = gemm_mxfp4_transposed_b(pa, pas, pb, pbs)
    torch.cuda.synchronize()
    want = orc.gemm_mxfp4_fp64(a, a_s, b, b_s)
    adq, bdq = orc.dequantize_mxfp4(a, a_s, np.float64), orc.dequantize_mxfp4(b, b_s, np.float64)
    for got in (c, cp):
        ok, rep = orc.check_bf16_against_fp64(H.bits(got), want, np.abs(adq) @ np.abs(bdq).T, k)
        assert ok, rep


def test_gemm_over_padded_operands_is_exact_where_fp32_sums_are(gpu):
    """Scale bytes 127 and codes of small magnitude: every product is a multiple of 0.25 and every sum stays far below
    2^24 quarter units, so fp32 accumulation is exact in any order and the two GEMMs must agree bit for bit -- also when
    the padding's scale bytes are zero (2^-127), the other byte a zero-filled buffer holds."""
    m, n, k, k_pad = 130, 264, 2880, 3072
    rng = np.random.default_rng(5)
    a = rng.integers(0, 256, (m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, (n, k // 2), dtype=np.uint8)
    a_s = np.full((m, k // 32), 127, dtype=np.uint8)
    b_s = np.full((n, k // 32), 127, dtype=np.uint8)
    da, das, db, dbs = (H.to_dev(v, gpu) for v in (a, a_s, b, b_s))
    c = gemm_mxfp4_transposed_b(da, das, db, dbs)
    pa, pas = pad_k_mxfp4(da, das, k_pad)
    pb, pbs = pad_k_mxfp4(db, dbs, k_pad)
    assert torch.equal(gemm_mxfp4_transposed_b(pa, pas, pb, pbs), c)
    pas[:, k // 32:] = 0
    pbs[:, k // 32:] = 0
    assert torch.equal(gemm_mxfp4_transposed_b(pa, pas, pb, pbs), c)
    want = orc.gemm_mxfp4_fp64(a, a_s, b, b_s)
    assert np.array_equal(H.bits(c), orc.f64_to_bf16_bits(want))


@pytest.mark.parametrize("m,n,k,n_pad", [
    (16, 2880, 1024, 3072),     # weight-streaming kernel
    (32, 96, 544, 512),         # ... with a K tail, padding far beyond N
    (100, 2880, 1024, 3072),    # narrow tiles
    (700, 2880, 512, 3072),     # 256 x 256 kernel
    (300, 160, 736, 192),       # ... with a K tail
])
def test_fused_quantiser_writes_padded_rows_and_leaves_the_padding_alone(gpu, m, n, k, n_pad):
    a, a_s = H.mx_operand(m, k, seed=m + n)
    b, b_s = H.mx_operand(2 * n, k, seed=m + n + 1, std=0.05)
    da, das, db, dbs = (H.to_dev(v, gpu) for v in (a, a_s, b, b_s))
    q, s = gemm_mxfp4_swiglu_quant_transposed_b(da, das, db, dbs)
    # allocated by the wrapper: zero-filled padding
    zq, zs = gemm_mxfp4_swiglu_quant_transposed_b(da, das, db, dbs, n_pad=n_pad)
    assert zq.shape == (m, n_pad // 2) and zs.shape == (m, n_pad // 32)
    assert torch.equal(zq[:, :n // 2], q) and torch.equal(zs[:, :n // 32], s)
    assert int(zq[:, n // 2:].max().item()) == 0 and int(zs[:, n // 32:].max().item()) == 0
    # passed in: the padding keeps what it held
    pq = torch.full((m, n_pad // 2), 0x5A, dtype=torch.uint8, device=gpu)
    ps = torch.full((m, n_pad // 32), 0x33, dtype=torch.uint8, device=gpu)
    gemm_mxfp4_swiglu_quant_transposed_b(da, das, db, dbs, pq, ps, n_pad=n_pad)
    assert torch.equal(pq[:, :n // 2], q) and torch.equal(ps[:, :n // 32], s)
    assert bool((pq[:, n // 2:] == 0x5A).all()) and bool((ps[:, n // 32:] == 0x33).all())
    with pytest.raises(ValueError, match="n_pad must be a multiple of 32 and at least"):
        gemm_mxfp4_swiglu_quant_transposed_b(da, das, db, dbs, n_pad=n - 32)


@pytest.mark.parametrize("rows,n,k,n_pad", [
    ([0, 300, 1, 260], 96, 512, 512),        # 256 x 256 kernel
    ([40, 0, 17, 64], 160, 1056, 512),       # narrow tiles, K tail
])
def test_grouped_fused_quantiser_writes_padded_rows(gpu, rows, n, k, n_pad):
    ro = np.concatenate([[0], np.cumsum(rows)]).astype(np.int32)
    e, total = len(rows), int(ro[-1])
    a, a_s = H.mx_operand(total, k, seed=total + n)
    b, b_s = H.mx_operand(e * 2 * n, k, seed=total + n + 1, std=0.05)
    da, das = H.to_dev(a, gpu), H.to_dev(a_s, gpu)
    db, dbs = H.to_dev(b.reshape(e, 2 * n, k // 2), gpu), H.to_dev(b_s.reshape(e, 2 * n, k // 32), gpu)
    dro = torch.from_numpy(ro).to(gpu)
    q, s = grouped_gemm_mxfp4_swiglu_quant_transposed_b(da, das, db, dbs, dro)
    pq = torch.full((total, n_pad // 2), 0x5A, dtype=torch.uint8, device=gpu)
    ps = torch.full((total, n_pad // 32), 0x33, dtype=torch.uint8, device=gpu)
    grouped_gemm_mxfp4_swiglu_quant_transposed_b(da, das, db, dbs, dro, pq, ps, n_pad=n_pad)
    assert torch.equal(pq[:, :n // 2], q) and torch.equal(ps[:, :n // 32], s)
    assert bool((pq[:, n // 2:] == 0x5A).all()) and bool((ps[:, n // 32:] == 0x33).all())


def test_mlp_block_with_a_hidden_size_of_2880_on_padded_rows(gpu):
    """quantiser -> gate+up GEMM with SwiGLU and quantiser -> down projection, hidden = intermediate = 2880, every K
    padded to 3072: the block's bf16 result equals the unpadded chain's within one bf16 step of the latter per element
    on all but a sliver of the elements (the two chains add the same products in different orders, and the fused
    quantiser in between turns a last-bit difference into at most one E2M1 step of one element), and the padded
    intermediate tensors hold exactly the unpadded ones."""
    tokens, hidden, inter, pad = 384, 2880, 2880, 3072
    g = torch.Generator(device="cpu").manual_seed(77)
    x = torch.randn((tokens, hidden), generator=g).to(torch.bfloat16).to(gpu)
    w1 = (torch.randn((2 * inter, hidden), generator=g) * 0.02).to(gpu)
    w2 = (torch.randn((hidden, inter), generator=g) * 0.02).to(gpu)
    w1q, w1s = quantize_mxfp4(w1)
    w2q, w2s = quantize_mxfp4(w2)
    # unpadded chain
    xq, xs = quantize_mxfp4(x)
    hq, hs = gemm_mxfp4_swiglu_quant_transposed_b(xq, xs, w1q, w1s)
    y = gemm_mxfp4_transposed_b(hq, hs, w2q, w2s)
    # padded chain: weights once, activations by the producers
    w1qp, w1sp = pad_k_mxfp4(w1q, w1s, pad)
    w2qp, w2sp = pad_k_mxfp4(w2q, w2s, pad)
    xqp, xsp = quantize_mxfp4(x, k_pad=pad)
    assert torch.equal(xqp[:, :hidden // 2], xq) and torch.equal(xsp[:, :hidden // 32], xs)
    hqp, hsp = gemm_mxfp4_swiglu_quant_transposed_b(xqp, xsp, w1qp, w1sp, n_pad=pad)
    yp = gemm_mxfp4_transposed_b(hqp, hsp, w2qp, w2sp)
    torch.cuda.synchronize()
    same_codes = (hqp[:, :inter // 2] == hq).float().mean().item()
    assert same_codes > 0.999, same_codes
    yf, ypf = y.float(), yp.float()
    close = (yf - ypf).abs() <= 2.0 ** -7 * yf.abs() + 1e-6
    assert close.float().mean().item() > 0.99, close.float().mean().item()
    # and against the oracle's block on the unpadded operands
    hdq = orc.dequantize_mxfp4(hq.cpu().numpy(), hs.cpu().numpy(), np.float64)
    w2dq = orc.dequantize_mxfp4(w2q.cpu().numpy(), w2s.cpu().numpy(), np.float64)
    want = hdq @ w2dq.T
    ok, rep = orc.check_bf16_against_fp64(H.bits(y), want, np.abs(hdq) @ np.abs(w2dq).T, inter)
    assert ok, rep
