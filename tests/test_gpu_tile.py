"""GPU parity of the LDS-staged 256x256 MXFP4 kernel (plain and grouped) against the oracle."""
import numpy as np
import pytest

from oracle import fp4_oracle as orc
from tests import helpers as H

pytestmark = pytest.mark.gpu
GENERIC, TILE = 1, 2


@pytest.mark.parametrize("m,n,k", [(256, 256, 256), (512, 768, 512), (300, 520, 256), (1, 8, 256), (257, 250, 768),
                                   (64, 1024, 1024)])
def test_mx_tile_matches_oracle(gpu, m, n, k):
    a, a_s = H.mx_operand(m, k, seed=0, outliers=True)
    b, b_s = H.mx_operand(n, k, seed=1, std=0.02)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=TILE)
    H.assert_mx_close(c, a, a_s, b, b_s)


def test_mx_tile_unit_scales_integer_exact(gpu):
    rng = np.random.default_rng(4)
    m, n, k = 256, 512, 1024
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    a_s = np.full((m, k // 32), 127, dtype=np.uint8)
    b_s = np.full((n, k // 32), 127, dtype=np.uint8)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=TILE)
    assert np.array_equal(c, orc.f64_to_bf16_bits(orc.gemm_mxfp4_fp64(a, a_s, b, b_s)))


def test_mx_tile_random_scales_every_kblock(gpu):
    """Scale bytes differ per row and per 32-block, so a wrong byte select or a wrong row
    permutation in the scale path cannot cancel out."""
    rng = np.random.default_rng(5)
    m, n, k = 256, 256, 512
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    a_s = rng.integers(117, 138, size=(m, k // 32), dtype=np.uint8)
    b_s = rng.integers(117, 138, size=(n, k // 32), dtype=np.uint8)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=TILE)
    H.assert_mx_close(c, a, a_s, b, b_s)


def test_grouped_tile_matches_per_expert(gpu):
    e, n, k = 4, 512, 512
    row_offsets = np.array([0, 300, 300, 811, 1000], dtype=np.int32)
    a, a_s = H.mx_operand(1000, k, seed=6)
    bw = [H.mx_operand(n, k, seed=20 + i, std=0.02) for i in range(e)]
    b = np.stack([w[0] for w in bw])
    b_s = np.stack([w[1] for w in bw])
    c = H.run_grouped(gpu, a, a_s, b, b_s, row_offsets, variant=TILE)
    for i in range(e):
        r0, r1 = row_offsets[i], row_offsets[i + 1]
        if r1 > r0:
            H.assert_mx_close(c[r0:r1], a[r0:r1], a_s[r0:r1], b[i], b_s[i])
            plain = H.run_mx(gpu, a[r0:r1], a_s[r0:r1], b[i], b_s[i], variant=TILE)
            assert np.array_equal(plain, c[r0:r1])


@pytest.mark.parametrize("m,n,k", [(4100, 4300, 512), (4352, 4100, 1024), (4100, 4300, 768)])
def test_mx_tile_more_tiles_than_compute_units(gpu, m, n, k):
    """289 tiles and more: with K % 512 == 0 one persistent workgroup per compute unit walks several tiles
    (ragged last row and column of tiles included); K = 768 takes the one-workgroup-per-tile form."""
    a, a_s = H.mx_operand(m, k, seed=30, outliers=True)
    b, b_s = H.mx_operand(n, k, seed=31, std=0.02)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=TILE)
    H.assert_mx_close(c, a, a_s, b, b_s)
    # every tile on its own (one workgroup, no tile loop) gives the same bits
    for (r0, r1, c0, c1) in ((0, 256, 0, 256), (3840, m, 4096, n), (2048, 2304, 1024, 1280)):
        part = H.run_mx(gpu, a[r0:r1], a_s[r0:r1], b[c0:c1], b_s[c0:c1], variant=TILE)
        assert np.array_equal(part, c[r0:r1, c0:c1])


@pytest.mark.parametrize("m,n,k", [(8192, 2400, 512), (8200, 2100, 1024), (4100, 4300, 512), (300, 300, 512), (8192, 2304, 768)])
def test_mx_tile_with_look_ahead_touches_gives_the_same_bits(gpu, m, n, k):
    """The form for weights that come from HBM (TILE_STREAMED: touches of the next round's panels; whole groups of 32
    m-tiles, a ragged group, a single round, a K it does not apply to) against the form without: same bits.  Shape-based
    dispatch takes one or the other by whether the weights are those of the previous call, so two calls in a row on
    the same operands run both."""
    TILE_STREAMED = 6
    a, a_s = H.mx_operand(m, k, seed=40)
    b, b_s = H.mx_operand(n, k, seed=41, std=0.02)
    want = H.run_mx(gpu, a, a_s, b, b_s, variant=TILE)
    assert np.array_equal(H.run_mx(gpu, a, a_s, b, b_s, variant=TILE_STREAMED), want)
    import torch
    from avelang_amd import gemm_mxfp4_transposed_b
    ops = tuple(H.to_dev(v, gpu) for v in (a, a_s, b, b_s))
    first = gemm_mxfp4_transposed_b(*ops, split_k=False)    # new weights: the form with touches
    second = gemm_mxfp4_transposed_b(*ops, split_k=False)   # the same weights again: the form without
    torch.cuda.synchronize()
    assert np.array_equal(H.bits(first), want) and np.array_equal(H.bits(second), want)
    if m * n * k <= 1 << 33:
        H.assert_mx_close(want, a, a_s, b, b_s)


@pytest.mark.parametrize("m,n,k", [(300, 520, 2048), (4100, 4300, 2048), (257, 130, 4096), (1000, 777, 6144), (8192, 2100, 4096), (65, 3000, 8192)])
def test_mx_tile_64_byte_scale_chunks_give_the_same_bits(gpu, m, n, k):
    """K % 2048 == 0 without touches: the scale rows are fetched 64 bytes at a time into one chunk buffer (one, two, three
    and four chunks; one tile per workgroup and the persistent walk; ragged last tiles).  The form with touches keeps
    the 16-byte pieces per pair of stages: same MFMAs on the same scale bytes, so the same bits.  Scale bytes differ in
    every block of every row, so a piece taken from the wrong row, chunk or slot changes the result."""
    rng = np.random.default_rng(k + m)
    a, a_s = H.mx_operand(m, k, seed=50)
    b, b_s = H.mx_operand(n, k, seed=51, std=0.02)
    a_s = (a_s.astype(np.int32) + rng.integers(-3, 4, size=a_s.shape)).clip(1, 254).astype(np.uint8)
    b_s = (b_s.astype(np.int32) + rng.integers(-3, 4, size=b_s.shape)).clip(1, 254).astype(np.uint8)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=TILE)
    assert np.array_equal(c, H.run_mx(gpu, a, a_s, b, b_s, variant=6))
    if m * n * k <= 1 << 33:
        H.assert_mx_close(c, a, a_s, b, b_s)


def test_grouped_tile_persistent_with_empty_and_ragged_experts(gpu):
    """336 tile slots for 256 compute units: the tile loop skips the slots behind an expert's last tile and
    an expert without rows; every expert's rows equal the plain GEMM on that expert bit for bit."""
    e, n, k = 6, 2048, 512
    row_offsets = np.array([0, 1500, 1500, 4321, 4400, 7000, 9000], dtype=np.int32)
    a, a_s = H.mx_operand(9000, k, seed=40)
    bw = [H.mx_operand(n, k, seed=50 + i, std=0.02) for i in range(e)]
    b = np.stack([w[0] for w in bw])
    b_s = np.stack([w[1] for w in bw])
    c = H.run_grouped(gpu, a, a_s, b, b_s, row_offsets, variant=TILE)
    for i in range(e):
        r0, r1 = row_offsets[i], row_offsets[i + 1]
        if r1 > r0:
            plain = H.run_mx(gpu, a[r0:r1], a_s[r0:r1], b[i], b_s[i], variant=TILE)
            assert np.array_equal(plain, c[r0:r1])
    H.assert_mx_close(c[4321:4400], a[4321:4400], a_s[4321:4400], b[3], b_s[3])
    H.assert_mx_close(c[:1500], a[:1500], a_s[:1500], b[0], b_s[0])


@pytest.mark.parametrize("k", [3072, 3104])
def test_grouped_tile_whole_groups_of_bands_and_a_long_k(gpu, k):
    """More than 32 m-tiles and more than 8 stages per tile: the walk has whole groups of 8 bands, whose next round's
    weight panels (and A rows) the kernel touches ahead from inside the stage loop; 3104 adds a K tail.  The touches
    write nothing but an LDS sink, so every expert's rows must still equal the plain GEMM on that expert bit for bit."""
    e, n = 5, 768
    row_offsets = np.array([0, 2100, 4097, 4097, 7300, 9000], dtype=np.int32)
    a, a_s = H.mx_operand(9000, k, seed=41)
    bw = [H.mx_operand(n, k, seed=60 + i, std=0.02) for i in range(e)]
    b = np.stack([w[0] for w in bw])
    b_s = np.stack([w[1] for w in bw])
    c = H.run_grouped(gpu, a, a_s, b, b_s, row_offsets, variant=TILE)
    for i in range(e):
        r0, r1 = row_offsets[i], row_offsets[i + 1]
        if r1 > r0:
            plain = H.run_mx(gpu, a[r0:r1], a_s[r0:r1], b[i], b_s[i], variant=TILE)
            assert np.array_equal(plain, c[r0:r1])
    H.assert_mx_close(c[7300:7400], a[7300:7400], a_s[7300:7400], b[4], b_s[4])


# K of any multiple of 32 from 512 up: whole pairs of stages from LDS, the K % 512 elements behind them straight from
# global memory.  640: scale rows of 20 bytes (4-byte aligned); 544, 992: odd pitches (17, 31 bytes), 1 and 15 tail
# blocks; 2880: 90-byte scale rows, 1440-byte data rows (not a multiple of the 128-byte line).
@pytest.mark.parametrize("m,n,k", [(256, 256, 640), (300, 520, 544), (257, 250, 992), (512, 300, 2880), (70, 1024, 1504),
                                   (4100, 4300, 736)])
def test_mx_tile_k_tail_matches_oracle(gpu, m, n, k):
    a, a_s = H.mx_operand(m, k, seed=50, outliers=True)
    b, b_s = H.mx_operand(n, k, seed=51, std=0.02)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=TILE)
    H.assert_mx_close(c, a, a_s, b, b_s)
    auto = H.run_mx(gpu, a, a_s, b, b_s)
    H.assert_mx_close(auto, a, a_s, b, b_s)


@pytest.mark.parametrize("k", [544, 800, 992])
def test_mx_tile_k_tail_integer_exact(gpu, k):
    """Unit scales and codes whose products are small integers: every partial sum is exact in fp32, so the result is
    the exact sum whatever the order -- a tail block that is skipped, read twice or read from a neighbouring row
    changes it."""
    rng = np.random.default_rng(k)
    m, n = 256, 512
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    a_s = np.full((m, k // 32), 127, dtype=np.uint8)
    b_s = np.full((n, k // 32), 127, dtype=np.uint8)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=TILE)
    assert np.array_equal(c, orc.f64_to_bf16_bits(orc.gemm_mxfp4_fp64(a, a_s, b, b_s)))


def test_mx_tile_k_tail_scales_every_kblock(gpu):
    rng = np.random.default_rng(52)
    m, n, k = 256, 256, 992
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    a_s = rng.integers(117, 138, size=(m, k // 32), dtype=np.uint8)
    b_s = rng.integers(117, 138, size=(n, k // 32), dtype=np.uint8)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=TILE)
    H.assert_mx_close(c, a, a_s, b, b_s)


def test_grouped_tile_k_tail_matches_per_expert(gpu):
    e, n, k = 4, 512, 2880
    row_offsets = np.array([0, 300, 300, 811, 1000], dtype=np.int32)
    a, a_s = H.mx_operand(1000, k, seed=56)
    bw = [H.mx_operand(n, k, seed=60 + i, std=0.02) for i in range(e)]
    b = np.stack([w[0] for w in bw])
    b_s = np.stack([w[1] for w in bw])
    c = H.run_grouped(gpu, a, a_s, b, b_s, row_offsets, variant=TILE)
    for i in range(e):
        r0, r1 = row_offsets[i], row_offsets[i + 1]
        if r1 > r0:
            H.assert_mx_close(c[r0:r1], a[r0:r1], a_s[r0:r1], b[i], b_s[i])
            assert np.array_equal(H.run_mx(gpu, a[r0:r1], a_s[r0:r1], b[i], b_s[i], variant=TILE), c[r0:r1])
