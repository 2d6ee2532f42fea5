"""Operand patterns for the decoded-value parity tests: one operand carries all 16 E2M1 codes under every finite
scale byte, the other is one-hot, so that every element of C is a single exactly representable product."""
import numpy as np

from oracle import fp4_oracle as orc

E4M3_FINITE = np.array([s for s in range(256) if (s & 0x7F) != 0x7F], dtype=np.uint8)   # 254 bytes


def _codes(rows, k):
    r = np.arange(rows)[:, None]
    kk = np.arange(k)[None, :]
    return ((r + kk) % 16).astype(np.uint8)   # any 16 consecutive k of a row hold all 16 codes


def mx_varied(rows, k):
    """Scale byte of (row r, block b): 16 (b % 16) + (r + r // 16) % 16 -- all of 0..254 in any 16 consecutive rows
    (255, the NaN, is replaced by 254)."""
    r = np.arange(rows)[:, None]
    b = np.arange(k // 32)[None, :]
    s = 16 * (b % 16) + (r + r // 16) % 16
    s = np.where(s == 255, 254, s).astype(np.uint8)
    return orc.pack_fp4(_codes(rows, k)), s


def mx_comp_byte(block):
    cls = (block % 16) // 4
    return np.where(cls == 0, 191, np.where(cls == 3, 63, 127)).astype(np.uint8)


def mx_onehot(first_k, rows, k):
    """Row i holds code 2 (= 1.0) at k = first_k + i and zeros elsewhere; block b has the compensating scale."""
    codes = np.zeros((rows, k), dtype=np.uint8)
    codes[np.arange(rows), first_k + np.arange(rows)] = 2
    s = np.broadcast_to(mx_comp_byte(np.arange(k // 32))[None, :], (rows, k // 32)).copy()
    return orc.pack_fp4(codes), s


def nv_varied(rows, k):
    """E4M3 byte of (row r, block b): all 254 finite bytes inside any 8 consecutive rows (K >= 512)."""
    nblk = k // 16
    r = np.arange(rows)[:, None]
    b = np.arange(nblk)[None, :]
    s = E4M3_FINITE[(b + nblk * (r % 8) + 5 * (r // 8)) % 254]
    return orc.pack_fp4(_codes(rows, k)), s.astype(np.uint8)


def nv_onehot(first_k, rows, k):
    codes = np.zeros((rows, k), dtype=np.uint8)
    codes[np.arange(rows), first_k + np.arange(rows)] = 2
    return orc.pack_fp4(codes), np.full((rows, k // 16), 0x38, dtype=np.uint8)   # 0x38 = 1.0


def same_bits(got, want):
    got = np.where((got & 0x7FFF) == 0, 0, got)      # +0 and -0 both count as zero
    want = np.where((want & 0x7FFF) == 0, 0, want)
    bad = np.argwhere(got != want)
    assert bad.size == 0, f"{len(bad)} elements differ, first at {bad[0]}: got {got[tuple(bad[0])]:#06x} want {want[tuple(bad[0])]:#06x}"


def mx_expect(a, a_s, b, b_s):
    ref = orc.dequantize_mxfp4(a, a_s, np.float64) @ orc.dequantize_mxfp4(b, b_s, np.float64).T
    assert np.all(np.isfinite(ref)) and np.all((ref == 0) | (np.abs(ref) >= 2.0 ** -126))
    return orc.f64_to_bf16_bits(ref)


def nv_expect(a, a_s, a_g, b, b_s, b_g):
    ref = orc.dequantize_nvfp4_block(a, a_s, np.float64) @ orc.dequantize_nvfp4_block(b, b_s, np.float64).T
    return orc.f64_to_bf16_bits(ref * (np.float64(np.float32(a_g)) * np.float64(np.float32(b_g))))


