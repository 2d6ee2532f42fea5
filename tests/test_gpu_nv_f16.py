"""GPU parity of the NVFP4 kernel that stages its operands in LDS as f16 (steps of 64 elements of K): the LDS-staged
kernel for every K where K % 256 != 0 keeps the fp4-staged tile kernel out, a last step of 16, 32 or 48 elements
(K % 64 != 0, rows that start at 8-byte boundaries only, scale rows anywhere) included."""
import numpy as np
import pytest

from tests import helpers as H
from tests.onehot_patterns import nv_expect, nv_onehot, nv_varied, same_bits

pytestmark = pytest.mark.gpu
AUTO, GENERIC, TILE, TILE_F16 = 0, 1, 2, 5


# one step, an odd and an even number of steps, up to the four-step tail and beyond; ragged tiles, rows that leave
# whole waves without work (M <= 64, <= 128, <= 192), several tiles in both directions
@pytest.mark.parametrize("m,n,k", [(256, 256, 64), (256, 256, 128), (300, 520, 320), (65, 8, 192), (130, 264, 1088),
                                   (200, 100, 448), (257, 250, 576), (1, 9, 64), (512, 768, 1344), (100, 300, 256),
                                   (96, 4100, 704),
                                   # K % 64 != 0: one, two and three scale blocks in the last step; K below one step
                                   (300, 520, 336), (65, 8, 208), (130, 264, 1072), (257, 250, 16), (200, 100, 48),
                                   (512, 768, 1360), (1, 9, 80), (96, 2100, 736)])
def test_nv_f16_tile_matches_oracle(gpu, m, n, k):
    a, a_s, a_g = H.nv_operand(m, k, seed=m + k)
    b, b_s, b_g = H.nv_operand(n, k, seed=n + k, std=0.02)
    c = H.run_nv(gpu, a, a_s, a_g, b, b_s, b_g, variant=TILE_F16)
    H.assert_nv_close(c, a, a_s, a_g, b, b_s, b_g)


def test_dispatch_takes_it_where_the_fp4_staged_kernel_cannot_run(gpu):
    m, n, k = 1300, 1330, 832     # K % 64 == 0, K % 256 != 0, more than 1536 blocks of 32 x 32 outputs
    a, a_s, a_g = H.nv_operand(m, k, seed=1)
    b, b_s, b_g = H.nv_operand(n, k, seed=2, std=0.02)
    auto = H.run_nv(gpu, a, a_s, a_g, b, b_s, b_g)
    assert np.array_equal(auto, H.run_nv(gpu, a, a_s, a_g, b, b_s, b_g, variant=TILE_F16))
    H.assert_nv_close(auto, a, a_s, a_g, b, b_s, b_g)
    # a few hundred outputs blocks: the one-wave-per-block kernel is the faster one (measured), and dispatch takes it
    small = (a[:200], a_s[:200], a_g, b[:300], b_s[:300], b_g)
    assert np.array_equal(H.run_nv(gpu, *small), H.run_nv(gpu, *small, variant=GENERIC))
    H.assert_nv_close(H.run_nv(gpu, *small, variant=TILE_F16), *small)
    with pytest.raises(ValueError, match="tile kernel does not support"):
        H.run_nv(gpu, a, a_s, a_g, b, b_s, b_g, variant=TILE)
    # K % 64 != 0 runs on it as well; operands that are not 8-byte aligned do not
    m, n = 200, 300
    a, a_s, a_g = H.nv_operand(m, 848, seed=3)
    b, b_s, b_g = H.nv_operand(n, 848, seed=4, std=0.02)
    H.assert_nv_close(H.run_nv(gpu, a, a_s, a_g, b, b_s, b_g, variant=TILE_F16), a, a_s, a_g, b, b_s, b_g)
    H.assert_nv_close(H.run_nv(gpu, a, a_s, a_g, b, b_s, b_g), a, a_s, a_g, b, b_s, b_g)
    big_m, big_n = 1300, 1330   # enough output blocks for dispatch to take it: the same bits as with the kernel forced
    a, a_s, a_g = H.nv_operand(big_m, 848, seed=5)
    b, b_s, b_g = H.nv_operand(big_n, 848, seed=6, std=0.02)
    assert np.array_equal(H.run_nv(gpu, a, a_s, a_g, b, b_s, b_g), H.run_nv(gpu, a, a_s, a_g, b, b_s, b_g, variant=TILE_F16))


@pytest.mark.parametrize("k", [960, 944, 976, 1008])
def test_nv_f16_unit_scales_integer_exact(gpu, k):
    """E4M3 scale 1.0 everywhere, per-tensor scales 1: products are multiples of 0.25 and the sum is exact in fp32."""
    from oracle import fp4_oracle as orc
    rng = np.random.default_rng(14)
    m, n = 192, 392
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    a_s = np.full((m, k // 16), 0x38, dtype=np.uint8)
    b_s = np.full((n, k // 16), 0x38, dtype=np.uint8)
    c = H.run_nv(gpu, a, a_s, 1.0, b, b_s, 1.0, variant=TILE_F16)
    assert np.array_equal(c, orc.f64_to_bf16_bits(orc.gemm_nvfp4_fp64(a, a_s, 1.0, b, b_s, 1.0)))


@pytest.mark.parametrize("k", [576, 592])
def test_nv_f16_decoded_values_bit_exact_both_sides(gpu, k):
    """All 16 codes under every finite E4M3 byte, on the weight side and on the activation side."""
    g = (0.5, 4.0)
    b, b_s = nv_varied(528, k)
    a, a_s = nv_onehot(0, k, k)
    same_bits(H.run_nv(gpu, a, a_s, g[0], b, b_s, g[1], variant=TILE_F16), nv_expect(a, a_s, g[0], b, b_s, g[1]))
    a, a_s = nv_varied(272, k)
    b, b_s = nv_onehot(0, k, k)
    same_bits(H.run_nv(gpu, a, a_s, g[0], b, b_s, g[1], variant=TILE_F16), nv_expect(a, a_s, g[0], b, b_s, g[1]))
