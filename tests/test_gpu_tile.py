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
