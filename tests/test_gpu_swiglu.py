"""SwiGLU-fused gate+up MXFP4 GEMM against exact arithmetic (tolerance stated in
``oracle.check_swiglu_bf16``), on the weight-streaming kernel, the LDS-staged kernel and the shape-agnostic one,
and against the unfused GEMM followed by the same activation."""
import numpy as np
import pytest
import torch

from avelang_amd import (gemm_mxfp4_swiglu_quant_transposed_b, gemm_mxfp4_swiglu_transposed_b,
                         gemm_mxfp4_transposed_b, grouped_gemm_mxfp4_swiglu_quant_transposed_b,
                         grouped_gemm_mxfp4_swiglu_transposed_b, quantize_mxfp4)
from oracle import fp4_oracle as orc
from tests import helpers as H

pytestmark = pytest.mark.gpu
GENERIC, TILE, DECODE = 1, 2, 3


def _operands(m, n, k, seed):
    a, a_s = H.mx_operand(m, k, seed=seed)
    b, b_s = H.mx_operand(2 * n, k, seed=seed + 1, std=0.05)
    return a, a_s, b, b_s


def _run(gpu, a, a_s, b, b_s, variant):
    c = gemm_mxfp4_swiglu_transposed_b(H.to_dev(a, gpu), H.to_dev(a_s, gpu), H.to_dev(b, gpu), H.to_dev(b_s, gpu),
                                       variant=variant)
    torch.cuda.synchronize()
    return H.bits(c)


@pytest.mark.parametrize("m,n,k", [(16, 128, 4096), (16, 1792, 4096), (1, 8, 512), (7, 104, 1024), (16, 2056, 2048),
                                   (13, 520, 14336), (16, 7 * 8 * 256 + 24, 1024), (5, 1000, 5120), (32, 1792, 4096), (64, 904, 2048),
                                   (40, 128, 1024), (24, 520, 14336),
                                   # whole 512-units on the rings and 1 / 15 / 3 / 10 more blocks behind them
                                   (16, 128, 4128), (7, 104, 992), (64, 904, 2144), (32, 1792, 1056), (16, 2880, 2880)])
def test_swiglu_decode_kernel(gpu, m, n, k):
    a, a_s, b, b_s = _operands(m, n, k, seed=m + n)
    ok, rep = orc.check_swiglu_bf16(_run(gpu, a, a_s, b, b_s, DECODE), a, a_s, b, b_s)
    assert ok, rep


@pytest.mark.parametrize("m,n,k", [(16, 128, 512), (33, 50, 96), (1, 1, 32), (100, 72, 160), (40, 129, 2048)])
def test_swiglu_generic_kernel(gpu, m, n, k):
    a, a_s, b, b_s = _operands(m, n, k, seed=m * n)
    ok, rep = orc.check_swiglu_bf16(_run(gpu, a, a_s, b, b_s, GENERIC), a, a_s, b, b_s)
    assert ok, rep


@pytest.mark.parametrize("m,n,k", [(256, 128, 512), (300, 200, 512), (512, 384, 1024), (65, 8, 512), (1000, 131, 1024),
                                   (2100, 8400, 512), (300, 200, 736), (256, 136, 2880), (70, 50, 544), (2100, 4300, 992)])
def test_swiglu_tile_kernel(gpu, m, n, k):
    """256 x 128-output tiles whose gate and up halves meet in LDS; ragged rows and columns, N % 8 != 0 (scalar
    stores), 594 tiles for 256 compute units (the persistent tile loop), and K with a tail behind the last multiple
    of 512 (1, 7, 10 and 15 blocks of 32)."""
    a, a_s, b, b_s = _operands(m, n, k, seed=m + n)
    ok, rep = orc.check_swiglu_bf16(_run(gpu, a, a_s, b, b_s, TILE), a, a_s, b, b_s)
    assert ok, rep


def test_swiglu_tile_kernel_with_look_ahead_touches_gives_the_same_bits(gpu):
    """More tiles than compute units: the form that touches the next round's weight panels (TILE_STREAMED, what dispatch
    takes for weights it has not just seen) against the form without, for the fused SwiGLU and for SwiGLU + quantiser
    (two calls in a row on the same weights run first the one form, then the other)."""
    m, n, k = 4100, 2100, 512
    a, a_s, b, b_s = _operands(m, n, k, seed=77)
    want = _run(gpu, a, a_s, b, b_s, TILE)
    assert np.array_equal(_run(gpu, a, a_s, b, b_s, 6), want)
    ok, rep = orc.check_swiglu_bf16(want, a, a_s, b, b_s)
    assert ok, rep
    m, n = 4100, 2112   # N % 32 == 0 for the quantiser
    a, a_s, b, b_s = _operands(m, n, k, seed=78)
    ops = tuple(H.to_dev(v, gpu) for v in (a, a_s, b, b_s))
    q1, s1 = gemm_mxfp4_swiglu_quant_transposed_b(*ops)
    q2, s2 = gemm_mxfp4_swiglu_quant_transposed_b(*ops)
    want_q, want_s = quantize_mxfp4(gemm_mxfp4_swiglu_transposed_b(*ops, variant=TILE))
    for q, sc in ((q1, s1), (q2, s2)):
        assert torch.equal(q, want_q) and torch.equal(sc, want_s)


@pytest.mark.parametrize("m,n,k", [(300, 264, 2048), (4100, 2112, 2048), (130, 1000, 4096)])
def test_swiglu_tile_kernel_64_byte_scale_chunks_give_the_same_bits(gpu, m, n, k):
    """K % 2048 == 0: the fused forms fetch their scale rows in 64-byte chunks (TILE) or, with touches, in 16-byte pieces
    per pair of stages (TILE_STREAMED): the same bits; and the quantised form equals the quantiser on that output."""
    a, a_s, b, b_s = _operands(m, n, k, seed=m + k)
    c = _run(gpu, a, a_s, b, b_s, TILE)
    assert np.array_equal(c, _run(gpu, a, a_s, b, b_s, 6))
    ok, rep = orc.check_swiglu_bf16(c, a, a_s, b, b_s)
    assert ok, rep
    if n % 32 == 0:
        ops = tuple(H.to_dev(v, gpu) for v in (a, a_s, b, b_s))
        q, q_s = gemm_mxfp4_swiglu_quant_transposed_b(*ops)
        want_q, want_s = quantize_mxfp4(gemm_mxfp4_swiglu_transposed_b(*ops, variant=TILE))
        assert torch.equal(q, want_q) and torch.equal(q_s, want_s)


def test_swiglu_tile_kernel_exact_on_integer_valued_operands(gpu):
    rng = np.random.default_rng(6)
    m, n, k = 320, 136, 512
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(2 * n, k // 2), dtype=np.uint8)
    a_s = np.full((m, k // 32), 127 - 3, dtype=np.uint8)
    b_s = np.full((2 * n, k // 32), 127 - 3, dtype=np.uint8)
    h, _, _ = orc.gemm_mxfp4_swiglu_fp64(a, a_s, b, b_s)
    got = orc.bf16_bits_to_f32(_run(gpu, a, a_s, b, b_s, TILE)).astype(np.float64)
    assert np.all(np.abs(got - h) <= orc.bf16_ulp(h) * 0.5 + 2.0 ** -20 * np.abs(h))


def test_swiglu_auto_dispatch_and_the_unfused_route(gpu):
    """AUTO takes the streaming kernel for M <= 64 (N % 8 == 0), the LDS-staged one for larger M with K % 512 == 0
    and the generic one otherwise; all agree with the plain
    GEMM's gate/up columns pushed through silu(g)*u in fp32 to within the bf16 roundings of that route."""
    for m, n, k in ((16, 256, 1024), (48, 256, 1024), (16, 100, 1024), (100, 256, 1024), (100, 256, 768)):
        a, a_s, b, b_s = _operands(m, n, k, seed=3)
        da, das, db, dbs = (H.to_dev(v, gpu) for v in (a, a_s, b, b_s))
        fused = gemm_mxfp4_swiglu_transposed_b(da, das, db, dbs)
        ok, rep = orc.check_swiglu_bf16(H.bits(fused), a, a_s, b, b_s)
        assert ok, (m, n, k, rep)
        plain = gemm_mxfp4_transposed_b(da, das, db, dbs).float()
        gate, up = plain[:, :n], plain[:, n:]
        unfused = torch.nn.functional.silu(gate) * up
        # gate and up went through a bf16 rounding (2^-9 each) on this route; silu amplifies the relative
        # error of a negative gate by about |g|
        tol = unfused.abs() * (2 + gate.abs()) * 2.0 ** -7 + 1e-6
        assert bool(((fused.float() - unfused).abs() <= tol).all()), (m, n, k)


def test_swiglu_exact_on_integer_valued_operands(gpu):
    """Unit scales and small integer-valued codes: gate and up are exact integers in fp32, so the only
    rounding is exp, the division, the product and the bf16 store."""
    rng = np.random.default_rng(5)
    m, n, k = 16, 64, 512
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(2 * n, k // 2), dtype=np.uint8)
    a_s = np.full((m, k // 32), 127 - 3, dtype=np.uint8)
    b_s = np.full((2 * n, k // 32), 127 - 3, dtype=np.uint8)
    h, _, _ = orc.gemm_mxfp4_swiglu_fp64(a, a_s, b, b_s)
    got = orc.bf16_bits_to_f32(_run(gpu, a, a_s, b, b_s, DECODE)).astype(np.float64)
    assert np.all(np.abs(got - h) <= orc.bf16_ulp(h) * 0.5 + 2.0 ** -20 * np.abs(h))


def test_swiglu_validation(gpu):
    a, a_s, b, b_s = (H.to_dev(v, gpu) for v in _operands(4, 8, 64, seed=1))
    with pytest.raises(ValueError, match="gate rows followed by as many up rows"):
        gemm_mxfp4_swiglu_transposed_b(a, a_s, b[:15], b_s[:15])
    with pytest.raises(ValueError, match="out must have shape"):
        gemm_mxfp4_swiglu_transposed_b(a, a_s, b, b_s, out=torch.empty((4, 16), dtype=torch.bfloat16, device=gpu))
    with pytest.raises(ValueError, match="swiglu decode kernel does not support"):
        gemm_mxfp4_swiglu_transposed_b(a, a_s, b, b_s, variant=DECODE)      # K % 512 != 0
    with pytest.raises(ValueError, match="swiglu tile kernel does not support"):
        gemm_mxfp4_swiglu_transposed_b(a, a_s, b, b_s, variant=TILE)        # K % 512 != 0


@pytest.mark.parametrize("m,n,k", [(256, 128, 512), (300, 224, 512), (70, 32, 1024), (2100, 8384, 512),
                                   (128, 1024, 1024), (200, 96, 2048), (65, 64, 1536), (129, 160, 2560), (16, 256, 1024), (64, 1792, 512),
                                   (300, 224, 992), (2100, 4320, 736), (256, 128, 2880),
                                   # up to 32 rows: the weight-streaming kernel's fused quantiser (one block of 32 outputs
                                   # or two per workgroup, one and two row blocks, every panel length, a K tail, a last
                                   # workgroup with a single block)
                                   (16, 14336, 4096), (1, 32, 512), (13, 96, 1024), (32, 14336, 2048), (17, 2080, 1536),
                                   (16, 160, 4128), (32, 8224, 992), (7, 32 * 300, 8192), (24, 64, 14336)])
def test_swiglu_with_fused_quantiser_equals_the_two_calls(gpu, m, n, k):
    """Codes and scales of the fused launch equal, bit for bit, the stand-alone quantiser applied to the bf16
    output of the fused SwiGLU GEMM on the same kernel (itself checked against exact arithmetic above), and the CPU
    quantiser applied to that output.  Up to 32 rows run on the weight-streaming kernel, shapes with few tiles on the
    256 x 64-output tile kernel, the rest on the 256 x 128-output one."""
    a, a_s, b, b_s = _operands(m, n, k, seed=m + n)
    da, das, db, dbs = (H.to_dev(v, gpu) for v in (a, a_s, b, b_s))
    h = gemm_mxfp4_swiglu_transposed_b(da, das, db, dbs, variant=DECODE if m <= 32 else TILE)
    want_q, want_s = quantize_mxfp4(h)
    got_q, got_s = gemm_mxfp4_swiglu_quant_transposed_b(da, das, db, dbs)
    torch.cuda.synchronize()
    assert got_q.shape == (m, n // 2) and got_s.shape == (m, n // 32)
    assert torch.equal(got_s, want_s)
    assert torch.equal(got_q, want_q)
    cpu_q, cpu_s = orc.quantize_mxfp4(h.float().cpu().numpy())
    assert np.array_equal(got_s.cpu().numpy(), cpu_s) and np.array_equal(got_q.cpu().numpy(), cpu_q)


@pytest.mark.parametrize("m,n,k", [(300, 224, 512), (70, 64, 1024), (2100, 8384, 512), (16, 2048, 1024), (30, 96, 512)])
def test_fused_quantiser_marks_blocks_with_non_finite_values(gpu, m, n, k):
    """silu(gate) * up is formed inside the kernel, so the caller cannot promise finite values: rows and columns with
    huge scales overflow to infinities and NaNs in bf16, and the fused quantiser must mark exactly those blocks with
    the NaN scale byte and zero codes, as the stand-alone quantiser and the oracle do on the bf16 output."""
    a, a_s, b, b_s = _operands(m, n, k, seed=m + n)
    a_s, b_s = a_s.copy(), b_s.copy()
    a_s[3::17, :] = 230                      # rows of A 2^103 times larger ...
    b_s[5::29, :] = 200                      # ... against gate and up rows 2^73 times larger: fp32 overflow
    b_s[n + 11::31, :] = 250                 # up rows alone: bf16 overflow of the product
    da, das, db, dbs = (H.to_dev(v, gpu) for v in (a, a_s, b, b_s))
    h = gemm_mxfp4_swiglu_transposed_b(da, das, db, dbs, variant=DECODE if m <= 32 else TILE)
    assert (~torch.isfinite(h.float())).any() and torch.isfinite(h.float()).any()
    got_q, got_s = gemm_mxfp4_swiglu_quant_transposed_b(da, das, db, dbs)
    want_q, want_s = quantize_mxfp4(h)
    torch.cuda.synchronize()
    assert torch.equal(got_s, want_s) and torch.equal(got_q, want_q)
    cpu_q, cpu_s = orc.quantize_mxfp4(h.float().cpu().numpy())
    assert (cpu_s == 0xFF).any()
    assert np.array_equal(got_s.cpu().numpy(), cpu_s) and np.array_equal(got_q.cpu().numpy(), cpu_q)


def test_swiglu_with_fused_quantiser_validation(gpu):
    a, a_s, b, b_s = (H.to_dev(v, gpu) for v in _operands(64, 48, 512, seed=2))
    with pytest.raises(ValueError, match="multiple of 32"):
        gemm_mxfp4_swiglu_quant_transposed_b(a, a_s, b, b_s)                      # N = 48
    a, a_s, b, b_s = (H.to_dev(v, gpu) for v in _operands(64, 64, 256, seed=2))
    with pytest.raises(ValueError, match="LDS-staged kernels only"):
        gemm_mxfp4_swiglu_quant_transposed_b(a, a_s, b, b_s)                      # K < 512


@pytest.mark.parametrize("n,k,offsets", [(256, 512, [0, 300, 300, 811, 1000]),          # LDS-staged kernel, an empty expert
                                         (96, 160, [0, 40, 41, 100, 130]),              # shape-agnostic kernel
                                         (2048, 512, [0, 1500, 1500, 4321, 4400, 7000, 9000]),    # 672 tile slots
                                         (256, 736, [0, 300, 300, 811, 1000]),          # LDS-staged kernel with a K tail
                                         # decode-sized expert layers (at most 128 rows per expert on average) run on the
                                         # 256 x 64-output tile kernel: an empty expert, one with two tiles of rows
                                         (256, 1024, [0, 30, 30, 95, 130, 400]),
                                         (96, 1536, [0, 1, 17, 17, 64, 100, 101, 140, 200])])
def test_grouped_swiglu_equals_per_expert_calls(gpu, n, k, offsets):
    """Every expert's rows equal the plain fused call on that expert, bit for bit (same kernel, same tiles), and one
    expert is checked against exact arithmetic."""
    e, total = len(offsets) - 1, offsets[-1]
    a, a_s = H.mx_operand(total, k, seed=60)
    bw = [H.mx_operand(2 * n, k, seed=70 + i, std=0.05) for i in range(e)]
    b, b_s = np.stack([w[0] for w in bw]), np.stack([w[1] for w in bw])
    da, das, db, dbs = (H.to_dev(v, gpu) for v in (a, a_s, b, b_s))
    ro = torch.tensor(offsets, dtype=torch.int32, device=gpu)
    c = grouped_gemm_mxfp4_swiglu_transposed_b(da, das, db, dbs, ro)
    torch.cuda.synchronize()
    for i in range(e):
        r0, r1 = offsets[i], offsets[i + 1]
        if r1 > r0:
            alone = gemm_mxfp4_swiglu_transposed_b(da[r0:r1], das[r0:r1], db[i], dbs[i],
                                                   variant=TILE if k >= 512 else GENERIC)
            assert torch.equal(alone, c[r0:r1]), i
    r0, r1 = offsets[-2], offsets[-1]
    ok, rep = orc.check_swiglu_bf16(H.bits(c[r0:r1]), a[r0:r1], a_s[r0:r1], b[e - 1], b_s[e - 1])
    assert ok, rep
    if k >= 512:
        q, q_s = grouped_gemm_mxfp4_swiglu_quant_transposed_b(da, das, db, dbs, ro)
        want_q, want_s = quantize_mxfp4(c)
        assert torch.equal(q, want_q) and torch.equal(q_s, want_s)
    else:
        with pytest.raises(ValueError, match="LDS-staged kernels only"):
            grouped_gemm_mxfp4_swiglu_quant_transposed_b(da, das, db, dbs, ro)
