"""Device-side MoE routing and row gather against the oracle (indices and bytes bit-exact, softmax
probabilities to 2e-6 relative), and the whole expert layer -- route, gather, grouped GEMM -- captured
in one graph."""
import numpy as np
import pytest
import torch

from avelang_amd import (gather_rows_mxfp4, grouped_gemm_mxfp4_swiglu_quant_transposed_b, grouped_gemm_mxfp4_transposed_b,
                         moe_combine_top2, moe_route_top2, quantize_mxfp4)
from oracle import fp4_oracle as orc
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _route(gpu, logits):
    tok, off, w = moe_route_top2(torch.from_numpy(logits).to(gpu))
    torch.cuda.synchronize()
    return tok.cpu().numpy(), off.cpu().numpy(), w.cpu().numpy()


@pytest.mark.parametrize("t,e,seed", [(1, 2, 0), (5, 3, 1), (1000, 8, 2), (1024, 8, 3), (1025, 8, 4), (16384, 8, 5),
                                      (3000, 32, 6), (70000, 16, 7), (5000, 256, 8), (2500, 7, 9)])
def test_route_top2_equals_oracle(gpu, t, e, seed):
    logits = orc.randn((t, e), seed)
    if t >= 1000:
        logits[3] = 0.25                   # all scores equal: experts 0 and 1
        logits[7, 1:] = logits[7, 0]
        logits[9, -1] = logits[9].max()    # a tie for first place
        logits[11] = -1e30                 # far below anything else, still finite
    want_tok, want_off, want_w = orc.route_top2(logits)
    tok, off, w = _route(gpu, logits)
    assert np.array_equal(off, want_off)
    assert np.array_equal(tok, want_tok)
    assert np.allclose(w, want_w, rtol=2e-6, atol=1e-30)


@pytest.mark.parametrize("t,e,seed", [(2065, 249, 20), (1363, 256, 21), (13343, 235, 22)])
def test_route_top2_probabilities_with_hundreds_of_experts(gpu, t, e, seed):
    """Logits on a grid of halves: many equal terms in the softmax denominator, which a float sum of 250 of them would
    get wrong by more than the stated 2e-6 (the kernel adds them up in double)."""
    logits = (np.round(orc.randn((t, e), seed) * 2) / 2).astype(np.float32)
    want_tok, want_off, want_w = orc.route_top2(logits)
    tok, off, w = _route(gpu, logits)
    assert np.array_equal(off, want_off) and np.array_equal(tok, want_tok)
    assert np.allclose(w, want_w, rtol=2e-6, atol=1e-30), float(np.max(np.abs(w - want_w) / want_w))


def test_route_top2_skewed_and_empty_experts(gpu):
    logits = orc.randn((2048, 8), 11)
    logits[:, 5] -= 100.0                  # expert 5 receives nothing
    logits[:, 2] += 100.0                  # expert 2 receives every token
    want_tok, want_off, _ = orc.route_top2(logits)
    tok, off, _ = _route(gpu, logits)
    assert want_off[6] == want_off[5] and want_off[3] - want_off[2] == 2048
    assert np.array_equal(off, want_off) and np.array_equal(tok, want_tok)


def test_route_top2_no_tokens_and_validation(gpu):
    tok, off, w = moe_route_top2(torch.zeros((0, 4), device=gpu))
    torch.cuda.synchronize()
    assert tok.numel() == 0 and w.numel() == 0 and off.cpu().tolist() == [0] * 5
    with pytest.raises(ValueError, match="E must be between 2 and 256"):
        moe_route_top2(torch.zeros((4, 1), device=gpu))
    with pytest.raises(ValueError, match="E must be between 2 and 256"):
        moe_route_top2(torch.zeros((4, 257), device=gpu))
    with pytest.raises(ValueError, match="float32"):
        moe_route_top2(torch.zeros((4, 8), device=gpu, dtype=torch.bfloat16))
    with pytest.raises(ValueError, match="row_offsets must have shape"):
        moe_route_top2(torch.zeros((4, 8), device=gpu), row_offsets=torch.zeros(8, dtype=torch.int32, device=gpu))


@pytest.mark.parametrize("rows,src,k", [(64, 16, 4096), (37, 9, 512), (50, 20, 128), (33, 7, 32), (20, 5, 96),
                                        (4096, 1000, 1024)])
def test_gather_rows_equals_oracle(gpu, rows, src, k):
    a, a_s = H.mx_operand(src, k, seed=rows)
    rng = np.random.default_rng(k)
    idx = rng.integers(0, src, size=rows).astype(np.int32)
    idx[0], idx[-1] = src - 1, 0
    if rows > 10:
        idx[3], idx[5] = -1, src           # outside the source: rows of zeros
    want, want_s = orc.gather_rows(a, a_s, idx)
    out, out_s = gather_rows_mxfp4(H.to_dev(a, gpu), H.to_dev(a_s, gpu), H.to_dev(idx, gpu))
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), want)
    assert np.array_equal(out_s.cpu().numpy(), want_s)


def test_gather_rows_validation_and_empty(gpu):
    a, a_s = H.mx_operand(4, 64, seed=1)
    a, a_s = H.to_dev(a, gpu), H.to_dev(a_s, gpu)
    out, out_s = gather_rows_mxfp4(a, a_s, torch.zeros(0, dtype=torch.int32, device=gpu))
    assert out.shape == (0, 32) and out_s.shape == (0, 2)
    with pytest.raises(ValueError, match="index must be a 1-D torch.int32"):
        gather_rows_mxfp4(a, a_s, torch.zeros(3, dtype=torch.int64, device=gpu))
    with pytest.raises(ValueError, match="A_scale must have shape"):
        gather_rows_mxfp4(a, a_s[:, :1].contiguous(), torch.zeros(3, dtype=torch.int32, device=gpu))


def test_expert_layer_in_one_graph(gpu):
    """logits -> routing -> gather -> grouped GEMM recorded once and replayed: equals the oracle's
    routing, and the per-expert plain GEMMs of the gathered rows, bit for bit."""
    tokens, experts, n, k = 700, 8, 256, 512
    x = orc.randn((tokens, k), 31)
    a, a_s = orc.quantize_mxfp4(x)
    ws = [orc.quantize_mxfp4(orc.randn((n, k), 40 + e, std=0.02)) for e in range(experts)]
    b, b_s = np.stack([w[0] for w in ws]), np.stack([w[1] for w in ws])
    logits = torch.from_numpy(orc.randn((tokens, experts), 32)).to(gpu)
    da, das, db, dbs = (H.to_dev(v, gpu) for v in (a, a_s, b, b_s))

    tok = torch.zeros(2 * tokens, dtype=torch.int32, device=gpu)
    off = torch.zeros(experts + 1, dtype=torch.int32, device=gpu)
    w = torch.zeros(2 * tokens, dtype=torch.float32, device=gpu)
    ga = torch.zeros((2 * tokens, k // 2), dtype=torch.uint8, device=gpu)
    gs = torch.zeros((2 * tokens, k // 32), dtype=torch.uint8, device=gpu)
    out = torch.zeros((2 * tokens, n), dtype=torch.bfloat16, device=gpu)

    def layer():
        moe_route_top2(logits, tok, off, w)
        gather_rows_mxfp4(da, das, tok, ga, gs)
        grouped_gemm_mxfp4_transposed_b(ga, gs, db, dbs, off, out=out)

    layer()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=torch.cuda.Stream()):
        layer()
    for rep, seed in enumerate((32, 33, 34)):
        new_logits = orc.randn((tokens, experts), seed)
        logits.copy_(torch.from_numpy(new_logits))
        out.fill_(0)                        # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want_tok, want_off, _ = orc.route_top2(new_logits)
        assert np.array_equal(tok.cpu().numpy(), want_tok), f"replay {rep}"
        assert np.array_equal(off.cpu().numpy(), want_off), f"replay {rep}"
        got = H.bits(out)
        for e in range(experts):
            r0, r1 = want_off[e], want_off[e + 1]
            if r1 > r0:
                rows = want_tok[r0:r1]
                ref = orc.f64_to_bf16_bits(orc.gemm_mxfp4_fp64(a[rows], a_s[rows], b[e], b_s[e]))
                ok, rep_ = orc.check_bf16_against_fp64(
                    got[r0:r1], orc.gemm_mxfp4_fp64(a[rows], a_s[rows], b[e], b_s[e]),
                    np.abs(orc.dequantize_mxfp4(a[rows], a_s[rows], np.float64))
                    @ np.abs(orc.dequantize_mxfp4(b[e], b_s[e], np.float64)).T, k)
                assert ok, (rep, e, rep_)
                assert ref.shape == got[r0:r1].shape


@pytest.mark.parametrize("t,e,h,seed", [(1, 2, 8, 0), (37, 8, 64, 1), (2500, 7, 4096, 2), (16384, 8, 512, 3)])
def test_rows_of_token_and_combine_equal_the_oracle(gpu, t, e, h, seed):
    """The inverse map is bit-exact; the combine is two float32 products, one float32 sum and one rounding to bf16
    per element: bit-exact against the same numpy operations, with and without renormalised weights."""
    logits = orc.randn((t, e), seed)
    inv = torch.full((t, 2), -7, dtype=torch.int32, device=gpu)
    tok, off, w = moe_route_top2(torch.from_numpy(logits).to(gpu), rows_of_token=inv)
    torch.cuda.synchronize()
    want_inv = orc.rows_of_token(tok.cpu().numpy(), logits)
    assert np.array_equal(inv.cpu().numpy(), want_inv)
    rows_bits = orc.f64_to_bf16_bits(orc.randn((2 * t, h), seed + 50).astype(np.float64) * 2.0)
    rows = torch.from_numpy(rows_bits.view(np.int16)).to(gpu).view(torch.bfloat16)
    for renorm in (False, True):
        got = moe_combine_top2(rows, inv, w, renormalize=renorm)
        torch.cuda.synchronize()
        want = orc.combine_top2(rows_bits, want_inv, w.cpu().numpy(), renormalize=renorm)
        assert np.array_equal(H.bits(got), want), renorm
    if t > 10:
        bad = inv.clone()
        bad[3, 0] = 2 * t          # out of range: that term counts as zeros
        bad[5, 1] = -1
        got = moe_combine_top2(rows, bad, w)
        torch.cuda.synchronize()
        assert np.array_equal(H.bits(got), orc.combine_top2(rows_bits, bad.cpu().numpy(), w.cpu().numpy()))


def test_combine_validation(gpu):
    rows = torch.zeros((8, 16), dtype=torch.bfloat16, device=gpu)
    inv = torch.zeros((4, 2), dtype=torch.int32, device=gpu)
    w = torch.ones(8, dtype=torch.float32, device=gpu)
    assert moe_combine_top2(rows, inv, w).shape == (4, 16)
    with pytest.raises(ValueError, match="multiple of 8"):
        moe_combine_top2(torch.zeros((8, 12), dtype=torch.bfloat16, device=gpu), inv, w)
    with pytest.raises(ValueError, match="rows_of_token must have shape"):
        moe_combine_top2(rows, inv[:3], w)
    with pytest.raises(ValueError, match="required"):
        moe_combine_top2(rows, None, w)
    with pytest.raises(ValueError, match="bfloat16"):
        moe_combine_top2(rows.float(), inv, w)


def test_whole_expert_layer_with_swiglu_and_combine_in_one_graph(gpu):
    """route -> quantise -> gather -> grouped gate+up+SwiGLU+quantiser -> grouped down projection -> combine, captured
    once and replayed with new logits; every replay equals the eager sequence bit for bit, and the combine of the
    eager sequence equals the oracle's combine of its down-projection output."""
    t, e, hidden, inter = 1536, 4, 512, 1024
    g = torch.Generator(device=gpu).manual_seed(9)
    x = torch.randn((t, hidden), generator=g, device=gpu, dtype=torch.bfloat16)
    w1 = [H.mx_operand(2 * inter, hidden, seed=80 + i, std=0.05) for i in range(e)]
    w2 = [H.mx_operand(hidden, inter, seed=90 + i, std=0.05) for i in range(e)]
    W1, W1s = (H.to_dev(np.stack([w[j] for w in w1]), gpu) for j in (0, 1))
    W2, W2s = (H.to_dev(np.stack([w[j] for w in w2]), gpu) for j in (0, 1))
    logits = torch.randn((t, e), generator=g, device=gpu)
    tok = torch.empty(2 * t, dtype=torch.int32, device=gpu)
    off = torch.empty(e + 1, dtype=torch.int32, device=gpu)
    wgt = torch.empty(2 * t, dtype=torch.float32, device=gpu)
    inv = torch.empty((t, 2), dtype=torch.int32, device=gpu)
    xa = torch.empty((t, hidden // 2), dtype=torch.uint8, device=gpu)
    xs = torch.empty((t, hidden // 32), dtype=torch.uint8, device=gpu)
    ga, gs = torch.empty((2 * t, hidden // 2), dtype=torch.uint8, device=gpu), torch.empty((2 * t, hidden // 32), dtype=torch.uint8, device=gpu)
    ha, hs = torch.empty((2 * t, inter // 2), dtype=torch.uint8, device=gpu), torch.empty((2 * t, inter // 32), dtype=torch.uint8, device=gpu)
    y = torch.empty((2 * t, hidden), dtype=torch.bfloat16, device=gpu)
    out = torch.empty((t, hidden), dtype=torch.bfloat16, device=gpu)

    def layer():
        moe_route_top2(logits, token_of_row=tok, row_offsets=off, row_weight=wgt, rows_of_token=inv)
        quantize_mxfp4(x, xa, xs)
        gather_rows_mxfp4(xa, xs, tok, out=ga, out_scale=gs)
        grouped_gemm_mxfp4_swiglu_quant_transposed_b(ga, gs, W1, W1s, off, out=ha, out_scale=hs)
        grouped_gemm_mxfp4_transposed_b(ha, hs, W2, W2s, off, out=y)
        moe_combine_top2(y, inv, wgt, out=out, renormalize=True)

    layer()
    torch.cuda.synchronize()
    eager = out.clone()
    want = orc.combine_top2(H.bits(y), inv.cpu().numpy(), wgt.cpu().numpy(), renormalize=True)
    assert np.array_equal(H.bits(eager), want)
    assert bool(torch.isfinite(eager.float()).all()) and float(eager.float().abs().max()) > 0
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=torch.cuda.Stream()):
        layer()
    for i in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), i
    logits.copy_(torch.randn((t, e), generator=g, device=gpu))
    graph.replay()
    torch.cuda.synchronize()
    replayed = out.clone()
    layer()
    torch.cuda.synchronize()
    assert torch.equal(out, replayed)
    assert not torch.equal(replayed, eager)
