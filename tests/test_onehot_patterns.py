"""CPU checks of the operand patterns behind the decoded-value GPU tests."""
import numpy as np

from oracle import fp4_oracle as orc
from tests.onehot_patterns import E4M3_FINITE, mx_comp_byte, mx_expect, mx_onehot, mx_varied, nv_expect, nv_onehot, nv_varied


def test_patterns_cover_every_finite_scale_byte():
    _, s = mx_varied(16, 512)
    assert set(s.reshape(-1).tolist()) == set(range(255))
    _, s = nv_varied(8, 512)
    assert set(s.reshape(-1).tolist()) == set(E4M3_FINITE.tolist())
    _, s = nv_varied(16, 1024)
    assert set(s[8:].reshape(-1).tolist()) == set(E4M3_FINITE.tolist())




def test_mx_products_are_normal_numbers_and_exact_in_bf16():
    """The compensating scale keeps every one-hot product a normal number, and the product of a code and two
    powers of two has at most two significant bits: the bf16 expectation is the exact value."""
    for k in (512, 768, 2048):
        v, v_s = mx_varied(48, k)
        o, o_s = mx_onehot(0, k, k)
        ref = orc.dequantize_mxfp4(v, v_s, np.float64) @ orc.dequantize_mxfp4(o, o_s, np.float64).T
        nz = ref[ref != 0]
        assert np.all(np.abs(nz) >= 2.0 ** -126) and np.all(np.abs(nz) < 2.0 ** 127)
        assert np.array_equal(orc.bf16_bits_to_f32(mx_expect(v, v_s, o, o_s)).astype(np.float64), ref)
        # element (r, j) is code (r + j) % 16 of the varied operand under its byte of block j // 32, compensated
        codes = orc.unpack_fp4(v)
        j = np.arange(k)
        want = (orc.decode_e2m1(codes[:, j]).astype(np.float64) * orc.decode_e8m0(v_s[:, j // 32]).astype(np.float64)
                * orc.decode_e8m0(mx_comp_byte(j // 32)).astype(np.float64)[None, :])
        assert np.array_equal(ref, want)


def test_nv_products_are_exact_in_bf16():
    v, v_s = nv_varied(16, 512)
    o, o_s = nv_onehot(0, 512, 512)
    ref = orc.dequantize_nvfp4_block(v, v_s, np.float64) @ orc.dequantize_nvfp4_block(o, o_s, np.float64).T * 2.0
    assert np.array_equal(orc.bf16_bits_to_f32(nv_expect(v, v_s, 0.5, o, o_s, 4.0)).astype(np.float64), ref)
    assert np.abs(ref).max() == 448 * 6 * 2 and np.abs(ref[ref != 0]).min() == 2.0 ** -10 * 2
