"""GPU parity of the small-M weight-streaming kernel and of the LDS-staged NVFP4 kernel."""
import numpy as np
import pytest

from oracle import fp4_oracle as orc
from tests import helpers as H

pytestmark = pytest.mark.gpu
GENERIC, TILE, DECODE = 1, 2, 3


@pytest.mark.parametrize("m,n,k", [(16, 256, 4096), (16, 1792, 4096), (1, 16, 128), (7, 100, 384), (16, 5000, 1024),
                                   (13, 8192, 8192), (16, 520, 14336), (5, 1000, 5120), (16, 300, 6656),
                                   (3, 4100, 512), (16, 7 * 16 * 256 + 48, 1024)])
def test_mx_decode_matches_oracle(gpu, m, n, k):
    a, a_s = H.mx_operand(m, k, seed=0)
    b, b_s = H.mx_operand(n, k, seed=1, std=0.02)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=DECODE)
    H.assert_mx_close(c, a, a_s, b, b_s)


@pytest.mark.parametrize("m,n,k", [(17, 256, 4096), (32, 1792, 4096), (33, 640, 2048), (64, 1808, 4096), (48, 100, 1024), (24, 100, 512),
                                   (64, 7 * 16 * 256 + 48, 1024), (20, 520, 14336), (50, 300, 3072), (32, 300, 6656),
                                   (64, 128, 8192), (40, 4100, 1024)])
def test_mx_decode_up_to_64_rows(gpu, m, n, k):
    """Two or four blocks of 16 activation rows per weight tile."""
    a, a_s = H.mx_operand(m, k, seed=m)
    b, b_s = H.mx_operand(n, k, seed=n, std=0.02)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=DECODE)
    H.assert_mx_close(c, a, a_s, b, b_s)
    assert np.array_equal(c, H.run_mx(gpu, a, a_s, b, b_s))          # what shape-based dispatch picks


def test_mx_decode_row_blocks_equal_the_16_row_kernel_bit_for_bit(gpu):
    """Each block of 16 rows is accumulated in the same order as a 16-row call on those rows."""
    m, n, k = 64, 448, 4096
    a, a_s = H.mx_operand(m, k, seed=5)
    b, b_s = H.mx_operand(n, k, seed=6, std=0.02)
    whole = H.run_mx(gpu, a, a_s, b, b_s, variant=DECODE)
    for r0 in range(0, m, 16):
        part = H.run_mx(gpu, a[r0:r0 + 16], a_s[r0:r0 + 16], b, b_s, variant=DECODE)
        assert np.array_equal(whole[r0:r0 + 16], part)


@pytest.mark.parametrize("m,n,k", [(16, 300, 2880), (5, 1000, 160), (16, 64, 32), (9, 333, 1504), (1, 17, 96), (16, 7 * 16 * 3 + 40, 4128),
                                   (32, 520, 1056), (64, 300, 2528), (48, 100, 3104), (13, 4100, 992)])
def test_mx_decode_k_of_any_multiple_of_32(gpu, m, n, k):
    """Below 512 the register kernel, whose last step of 128 elements may hold one to three blocks; from 512 up the
    rings on the whole units of 512 and up to 15 blocks behind them from global memory (one, two, four row blocks)."""
    a, a_s = H.mx_operand(m, k, seed=3)
    b, b_s = H.mx_operand(n, k, seed=4, std=0.02)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=DECODE)
    H.assert_mx_close(c, a, a_s, b, b_s)
    assert np.array_equal(c, H.run_mx(gpu, a, a_s, b, b_s))          # what shape-based dispatch picks


def test_mx_decode_partial_step_ignores_the_next_row(gpu):
    """K = 160: the last step holds one block, and the lanes behind it see the next row's first blocks.  Every other
    weight row carries the NaN scale byte in those blocks: its own outputs are NaN, its neighbours' must not be."""
    m, n, k = 16, 96, 160
    a, a_s = H.mx_operand(m, k, seed=5)
    b, b_s = H.mx_operand(n, k, seed=6, std=0.02)
    b_s[1::2, :3] = 0xFF
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=DECODE)
    nan = (c & 0x7FFF) > 0x7F80
    assert nan[:, 1::2].all() and not nan[:, 0::2].any()
    H.assert_mx_close(c[:, 0::2], a, a_s, b[0::2], b_s[0::2])


def test_mx_decode_rejects_what_it_cannot_run(gpu):
    a, a_s = H.mx_operand(65, 512, seed=1)
    b, b_s = H.mx_operand(64, 512, seed=2)
    with pytest.raises(ValueError, match="decode kernel does not support"):
        H.run_mx(gpu, a, a_s, b, b_s, variant=DECODE)                 # M > 64
    a, a_s = H.mx_operand(16, 256, seed=1)
    b, b_s = H.mx_operand(64, 256, seed=2)
    H.assert_mx_close(H.run_mx(gpu, a, a_s, b, b_s, variant=DECODE), a, a_s, b, b_s)   # K < 512: the register kernel
    a, a_s = H.mx_operand(17, 256, seed=1)
    with pytest.raises(ValueError, match="decode kernel does not support"):
        H.run_mx(gpu, a, a_s, b, b_s, variant=DECODE)                 # K < 512 with more than 16 rows
    H.assert_mx_close(H.run_mx(gpu, a, a_s, b, b_s), a, a_s, b, b_s)  # shape-based dispatch still has a kernel


@pytest.mark.parametrize("m,n,k", [(40, 64, 1536), (64, 1808, 2560), (33, 300, 2880), (50, 4100, 512)])
def test_mx_decode_four_row_blocks_on_an_odd_number_of_units(gpu, m, n, k):
    """33..64 rows on an odd number of 512-element units: panels of 1024 or 2048 elements with a short panel at the end
    (a single unit: two launches of up to 32 rows) -- either way bit-identical to calls on the two row ranges alone."""
    a, a_s = H.mx_operand(m, k, seed=m)
    b, b_s = H.mx_operand(n, k, seed=n, std=0.02)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=DECODE)
    H.assert_mx_close(c, a, a_s, b, b_s)
    assert np.array_equal(c, H.run_mx(gpu, a, a_s, b, b_s))          # what shape-based dispatch picks
    assert np.array_equal(c[:32], H.run_mx(gpu, a[:32], a_s[:32], b, b_s, variant=DECODE))
    assert np.array_equal(c[32:], H.run_mx(gpu, a[32:], a_s[32:], b, b_s, variant=DECODE))


@pytest.mark.parametrize("m,n,k", [(16, 300, 11008), (32, 200, 13824), (64, 136, 17920), (5, 1000, 1536), (48, 64, 3584),
                                   (16, 7 * 16 * 2 + 8, 5632), (32, 100, 13312), (33, 100, 11264)])
def test_mx_decode_short_last_panel(gpu, m, n, k):
    """K that no long panel divides -- 21.5, 27, 35, 3, 7, 11 and 26 units of 512 (the hidden sizes 11008, 13824 and
    17920 among them): panels of 2048 (1024) elements and a short panel of 1..3 units at the end (33 rows and more stay
    below K = 12288 here: above it shape-based dispatch splits K over a workspace instead).  Random codes under
    random scale bytes per row and block, so that a wrong chunk, step or scale byte in the short panel cannot pass;
    then unit scales, where the result must equal the correctly rounded exact sum bit for bit."""
    rng = np.random.default_rng(m + k)
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    a_s = rng.integers(118, 132, size=(m, k // 32), dtype=np.uint8)
    b_s = rng.integers(118, 132, size=(n, k // 32), dtype=np.uint8)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=DECODE)
    H.assert_mx_close(c, a, a_s, b, b_s)
    assert np.array_equal(c, H.run_mx(gpu, a, a_s, b, b_s))
    a_s[:] = 127
    b_s[:] = 127
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=DECODE)
    assert np.array_equal(c, orc.f64_to_bf16_bits(orc.gemm_mxfp4_fp64(a, a_s, b, b_s)))


def test_mx_decode_short_last_panel_with_swiglu_quantiser_and_blocked_scales(gpu):
    import torch
    from avelang_amd import (gemm_mxfp4_blocked_scales_transposed_b, gemm_mxfp4_swiglu_quant_transposed_b,
                             gemm_mxfp4_swiglu_transposed_b, quantize_mxfp4, scales_to_blocked)

    m, n, k = 24, 96, 13824   # 27 units
    a, a_s = H.mx_operand(m, k, seed=91)
    b, b_s = H.mx_operand(2 * n, k, seed=92, std=0.05)
    d = [H.to_dev(v, gpu) for v in (a, a_s, b, b_s)]
    c = gemm_mxfp4_swiglu_transposed_b(*d, variant=DECODE)
    q, q_s = gemm_mxfp4_swiglu_quant_transposed_b(*d)
    want_q, want_s = quantize_mxfp4(c)
    torch.cuda.synchronize()
    ok, rep = orc.check_swiglu_bf16(H.bits(c), a, a_s, b, b_s)
    assert ok, rep
    assert torch.equal(q, want_q) and torch.equal(q_s, want_s)
    plain = H.run_mx(gpu, a, a_s, b, b_s, variant=DECODE)
    blocked = gemm_mxfp4_blocked_scales_transposed_b(d[0], scales_to_blocked(d[1]), d[2], scales_to_blocked(d[3]))
    torch.cuda.synchronize()
    assert np.array_equal(H.bits(blocked), plain)


def test_mx_decode_random_scales_every_kblock(gpu):
    rng = np.random.default_rng(7)
    m, n, k = 16, 640, 2048
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    a_s = rng.integers(117, 138, size=(m, k // 32), dtype=np.uint8)
    b_s = rng.integers(117, 138, size=(n, k // 32), dtype=np.uint8)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=DECODE)
    H.assert_mx_close(c, a, a_s, b, b_s)


def test_mx_decode_unit_scales_integer_exact(gpu):
    rng = np.random.default_rng(8)
    m, n, k = 16, 448, 4096
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    a_s = np.full((m, k // 32), 127, dtype=np.uint8)
    b_s = np.full((n, k // 32), 127, dtype=np.uint8)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=DECODE)
    assert np.array_equal(c, orc.f64_to_bf16_bits(orc.gemm_mxfp4_fp64(a, a_s, b, b_s)))


@pytest.mark.parametrize("m,n,k", [(256, 256, 256), (512, 256, 1024), (300, 200, 512), (1, 8, 256), (257, 264, 768)])
def test_nv_tile_matches_oracle(gpu, m, n, k):
    a, a_s, a_g = H.nv_operand(m, k, seed=2)
    b, b_s, b_g = H.nv_operand(n, k, seed=3, std=0.02)
    c = H.run_nv(gpu, a, a_s, a_g, b, b_s, b_g, variant=TILE)
    H.assert_nv_close(c, a, a_s, a_g, b, b_s, b_g)


def test_nv_tile_equals_generic_on_random_bytes(gpu):
    """Random codes under random finite E4M3 scales: both kernels dequantise exactly, so they may
    differ only by fp32 summation order; each is checked against the oracle."""
    rng = np.random.default_rng(9)
    m, n, k = 256, 256, 512
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    a_s = rng.integers(0x20, 0x50, size=(m, k // 16), dtype=np.uint8)
    b_s = rng.integers(0x20, 0x50, size=(n, k // 16), dtype=np.uint8)
    for variant in (GENERIC, TILE):
        c = H.run_nv(gpu, a, a_s, 0.5, b, b_s, 0.25, variant=variant)
        H.assert_nv_close(c, a, a_s, 0.5, b, b_s, 0.25)


# ---- the NVFP4 weight-streaming kernel (at most 64 rows) ---------------------------------------------------------------

@pytest.mark.parametrize("m,n,k", [(16, 256, 4096), (16, 1792, 4096), (1, 16, 128), (7, 100, 384), (16, 5000, 1024),
                                   (13, 4096, 8192), (16, 520, 14336), (5, 1000, 5120), (16, 7 * 16 * 256 + 48, 1024),
                                   (17, 256, 4096), (32, 1792, 2048), (33, 640, 2048), (64, 1808, 1024), (48, 100, 1024),
                                   (64, 2 * 16 * 256 + 48, 512), (20, 520, 14336)])
def test_nv_decode_matches_oracle(gpu, m, n, k):
    """One, two and four blocks of 16 activation rows; one to seven tiles per workgroup; ragged N and M; K that
    is not a whole chunk of 16 steps."""
    a, a_s, a_g = H.nv_operand(m, k, seed=m)
    b, b_s, b_g = H.nv_operand(n, k, seed=n, std=0.02)
    c = H.run_nv(gpu, a, a_s, a_g, b, b_s, b_g, variant=DECODE)
    H.assert_nv_close(c, a, a_s, a_g, b, b_s, b_g)


def test_nv_decode_random_bytes_and_scales(gpu):
    """Random codes under random finite E4M3 scales that differ per row and per 16-block: a wrong scale byte, block
    or lane assignment cannot pass.  Dispatch takes this kernel by itself for at most 64 rows."""
    rng = np.random.default_rng(19)
    m, n, k = 40, 328, 1664
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    a_s = rng.integers(0x20, 0x50, size=(m, k // 16), dtype=np.uint8)
    b_s = rng.integers(0x20, 0x50, size=(n, k // 16), dtype=np.uint8)
    c = H.run_nv(gpu, a, a_s, 0.5, b, b_s, 0.25, variant=DECODE)
    H.assert_nv_close(c, a, a_s, 0.5, b, b_s, 0.25)
    assert np.array_equal(c, H.run_nv(gpu, a, a_s, 0.5, b, b_s, 0.25))


def test_nv_decode_unit_scales_integer_exact(gpu):
    """Scale byte 0x38 (1.0) and per-tensor scales of 1: every product is a multiple of 0.25 and every partial sum
    exact in fp32, so the result must equal the correctly rounded exact sum bit for bit."""
    rng = np.random.default_rng(20)
    m, n, k = 64, 264, 2048
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    a_s = np.full((m, k // 16), 0x38, dtype=np.uint8)
    b_s = np.full((n, k // 16), 0x38, dtype=np.uint8)
    c = H.run_nv(gpu, a, a_s, 1.0, b, b_s, 1.0, variant=DECODE)
    assert np.array_equal(c, orc.f64_to_bf16_bits(orc.gemm_nvfp4_fp64(a, a_s, 1.0, b, b_s, 1.0)))


def test_nv_decode_rejects_what_it_cannot_run(gpu):
    a, a_s, a_g = H.nv_operand(65, 256, seed=1)
    b, b_s, b_g = H.nv_operand(64, 256, seed=2)
    with pytest.raises(ValueError, match="decode kernel does not support"):
        H.run_nv(gpu, a, a_s, a_g, b, b_s, b_g, variant=DECODE)              # 65 rows
    a, a_s, a_g = H.nv_operand(16, 192, seed=1)
    b, b_s, b_g = H.nv_operand(64, 192, seed=2)
    with pytest.raises(ValueError, match="decode kernel does not support"):
        H.run_nv(gpu, a, a_s, a_g, b, b_s, b_g, variant=DECODE)              # K % 128 != 0
    H.assert_nv_close(H.run_nv(gpu, a, a_s, a_g, b, b_s, b_g), a, a_s, a_g, b, b_s, b_g)   # dispatch falls back


@pytest.mark.parametrize("m,n,k", [(16, 328, 2048), (24, 328, 1536), (32, 1000, 1024), (9, 136, 512), (16, 2056, 3584),
                                   (16, 328, 2080), (24, 328, 1504), (32, 1000, 1056), (16, 520, 4576), (7, 4100, 2880),
                                   (33, 328, 1024), (64, 1808, 2048), (50, 7 * 16 * 3 + 40, 4096), (40, 100, 3104),
                                   (64, 4100, 1056),
                                   (16, 300, 11008), (32, 200, 13824), (9, 136, 1536), (24, 64, 3584), (16, 100, 5632)])
def test_nv_ring_random_bytes_and_scales(gpu, m, n, k):
    """Up to 32 rows run on the LDS rings: panels of 2048, 1024 and 512 elements, one and two blocks of 16 activation
    rows, random codes under random finite E4M3 scales that differ per row and 16-block; the second half of the list
    has K with 1, 15, 1, 15 and 10 blocks of 32 behind the last whole unit of 512, which come from global memory.  The
    next five: 33..64 rows, four blocks of activation rows over panels of 1024 elements (an even number of units),
    two of them with a K tail.  The last five: up to 32 rows on K that no long panel divides (21.5, 27, 3, 7 and 11
    units): panels of 2048 (1024) elements with a short panel at the end."""
    rng = np.random.default_rng(m + k)
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    a_s = rng.integers(0x20, 0x50, size=(m, k // 16), dtype=np.uint8)
    b_s = rng.integers(0x20, 0x50, size=(n, k // 16), dtype=np.uint8)
    c = H.run_nv(gpu, a, a_s, 0.5, b, b_s, 0.25, variant=DECODE)
    H.assert_nv_close(c, a, a_s, 0.5, b, b_s, 0.25)
    # unit scales: integer-exact sums whatever the order of summation
    a_s[:] = 0x38
    b_s[:] = 0x38
    c = H.run_nv(gpu, a, a_s, 1.0, b, b_s, 1.0, variant=DECODE)
    assert np.array_equal(c, orc.f64_to_bf16_bits(orc.gemm_nvfp4_fp64(a, a_s, 1.0, b, b_s, 1.0)))
