"""GPU parity of the shape-agnostic kernels against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

from oracle import fp4_oracle as orc
from tests import helpers as H

pytestmark = pytest.mark.gpu
GENERIC = 1


@pytest.mark.parametrize("m,n,k", [(32, 32, 64), (256, 256, 256), (100, 200, 96), (1, 1, 32), (33, 129, 160),
                                   (16, 300, 512)])
def test_mx_generic_matches_oracle(gpu, m, n, k):
    a, a_s = H.mx_operand(m, k, seed=0)
    b, b_s = H.mx_operand(n, k, seed=1)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=GENERIC)
    H.assert_mx_close(c, a, a_s, b, b_s)


def _onehot_mx_problem(scale_bytes):
    """A: row i is one-hot at k=i with code 2 (=1.0) and scale 1.0, so C[i][j] is exactly the
    dequantised B[j][i]; B runs through all 16 codes under the given scale bytes."""
    k = 64
    a_codes = np.zeros((k, k), dtype=np.uint8)
    a_codes[np.arange(k), np.arange(k)] = 2
    a = orc.pack_fp4(a_codes)
    a_s = np.full((k, k // 32), 127, dtype=np.uint8)
    n = 16 * len(scale_bytes)
    b_codes = np.zeros((n, k), dtype=np.uint8)
    b_s = np.zeros((n, k // 32), dtype=np.uint8)
    for si, sb in enumerate(scale_bytes):
        for code in range(16):
            row = si * 16 + code
            b_codes[row, :] = (code + np.arange(k)) % 16
            b_s[row, :] = sb
    return a, a_s, orc.pack_fp4(b_codes), b_s


def test_mx_decoded_values_bit_exact(gpu):
    # every E2M1 code under every E8M0 scale whose products are normal bf16 numbers
    scale_bytes = list(range(2, 253))
    a, a_s, b, b_s = _onehot_mx_problem(scale_bytes)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=GENERIC)
    expect = orc.f32_to_bf16_bits(orc.dequantize_mxfp4(b, b_s).T.copy())
    # +0 and -0 both count as zero
    got = np.where((c & 0x7FFF) == 0, 0, c)
    expect = np.where((expect & 0x7FFF) == 0, 0, expect)
    assert np.array_equal(got, expect)


def test_mx_unit_scales_integer_exact(gpu):
    """All scales 1.0: every product is a multiple of 0.25 and the sum is exact in fp32,
    so the bf16 result must equal the correctly rounded exact sum bit for bit."""
    rng = np.random.default_rng(3)
    m, n, k = 64, 96, 256
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    a_s = np.full((m, k // 32), 127, dtype=np.uint8)
    b_s = np.full((n, k // 32), 127, dtype=np.uint8)
    c = H.run_mx(gpu, a, a_s, b, b_s, variant=GENERIC)
    ref = orc.gemm_mxfp4_fp64(a, a_s, b, b_s)
    assert np.array_equal(c, orc.f64_to_bf16_bits(ref))


@pytest.mark.parametrize("m,n,k", [(32, 32, 64), (64, 128, 256), (50, 70, 48), (3, 5, 16), (130, 40, 1040)])
def test_nv_generic_matches_oracle(gpu, m, n, k):
    a, a_s, a_g = H.nv_operand(m, k, seed=2)
    b, b_s, b_g = H.nv_operand(n, k, seed=3, std=0.02)
    c = H.run_nv(gpu, a, a_s, a_g, b, b_s, b_g, variant=GENERIC)
    H.assert_nv_close(c, a, a_s, a_g, b, b_s, b_g)


def test_nv_decoded_values_bit_exact(gpu):
    """One-hot A (code 1.0, E4M3 scale 1.0 = 0x38, global 1.0): C[i][j] = E2M1(code) * E4M3(scale)
    of B, for all 16 codes under every finite E4M3 byte."""
    k = 64
    a_codes = np.zeros((k, k), dtype=np.uint8)
    a_codes[np.arange(k), np.arange(k)] = 2
    a = orc.pack_fp4(a_codes)
    a_s = np.full((k, k // 16), 0x38, dtype=np.uint8)
    scale_bytes = [s for s in range(256) if (s & 0x7F) != 0x7F]
    n = 16 * len(scale_bytes)
    b_codes = np.zeros((n, k), dtype=np.uint8)
    b_s = np.zeros((n, k // 16), dtype=np.uint8)
    for si, sb in enumerate(scale_bytes):
        for code in range(16):
            b_codes[si * 16 + code, :] = (code + np.arange(k)) % 16
            b_s[si * 16 + code, :] = sb
    b = orc.pack_fp4(b_codes)
    c = H.run_nv(gpu, a, a_s, 1.0, b, b_s, 1.0, variant=GENERIC)
    expect = orc.f32_to_bf16_bits(orc.dequantize_nvfp4_block(b, b_s).T.copy())
    got = np.where((c & 0x7FFF) == 0, 0, c)
    expect = np.where((expect & 0x7FFF) == 0, 0, expect)
    assert np.array_equal(got, expect)


def test_grouped_generic_matches_per_expert(gpu):
    e, n, k = 4, 160, 128
    row_offsets = np.array([0, 37, 37, 101, 150], dtype=np.int32)  # one empty expert, ragged sizes
    a, a_s = H.mx_operand(150, k, seed=5)
    bw = [H.mx_operand(n, k, seed=10 + i, std=0.02) for i in range(e)]
    b = np.stack([w[0] for w in bw])
    b_s = np.stack([w[1] for w in bw])
    c = H.run_grouped(gpu, a, a_s, b, b_s, row_offsets, variant=GENERIC)
    for i in range(e):
        r0, r1 = row_offsets[i], row_offsets[i + 1]
        if r1 > r0:
            H.assert_mx_close(c[r0:r1], a[r0:r1], a_s[r0:r1], b[i], b_s[i])
            plain = H.run_mx(gpu, a[r0:r1], a_s[r0:r1], b[i], b_s[i], variant=GENERIC)
            assert np.array_equal(plain, c[r0:r1])
