"""Pins the CPU oracle (no GPU).  The reference holds no FP4 vectors, so each function is
checked against something independent of its own formula: published format tables, torch's
FP8/bf16 casts, ``math.ldexp``, exact rational arithmetic, and invariants a plausible mistake
(wrong nibble order, wrong tie rule, off-by-one exponent, transposed operand) would break."""
import math
import os
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import fp4_oracle as orc

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")

# OCP Microscaling v1.0, table of FP4 E2M1 encodings (S EE M)
E2M1_SPEC = {0b0000: 0.0, 0b0001: 0.5, 0b0010: 1.0, 0b0011: 1.5, 0b0100: 2.0, 0b0101: 3.0, 0b0110: 4.0, 0b0111: 6.0}


def e2m1_from_fields(code):
    """Independent decode from the bit fields: sign, 2-bit exponent (bias 1), 1-bit mantissa."""
    s, e, m = (code >> 3) & 1, (code >> 1) & 3, code & 1
    v = Fraction(m, 2) if e == 0 else (1 + Fraction(m, 2)) * Fraction(2) ** (e - 1)
    return -v if s else v


def test_e2m1_table_matches_spec_and_bitfields():
    for code in range(16):
        v = float(orc.decode_e2m1(np.array([code], dtype=np.uint8))[0])
        assert abs(v) == E2M1_SPEC[code & 7]
        assert Fraction(v) == e2m1_from_fields(code)
        assert math.copysign(1.0, v) == (-1.0 if code & 8 else 1.0)


def test_e8m0_exhaustive_against_ldexp():
    b = np.arange(256, dtype=np.uint8)
    d = orc.decode_e8m0(b)
    for i in range(255):
        assert d[i] == math.ldexp(1.0, i - 127)
    assert math.isnan(d[255])
    if hasattr(torch, "float8_e8m0fnu"):
        t = torch.from_numpy(b[:255].copy()).view(torch.float8_e8m0fnu).float().numpy().astype(np.float64)
        assert np.array_equal(t, d[:255])


def test_e4m3_decode_exhaustive_against_torch():
    b = np.arange(256, dtype=np.uint8)
    t = torch.from_numpy(b).view(torch.float8_e4m3fn).float().numpy()
    d = orc.decode_e4m3(b)
    assert np.array_equal(np.isnan(t), np.isnan(d))
    assert np.array_equal(t[~np.isnan(t)], d[~np.isnan(d)])
    assert d[0x7E] == 448.0 and d[0x38] == 1.0 and d[0x01] == 2.0 ** -9


def test_e4m3_encode_against_torch_cast():
    rng = np.random.default_rng(0)
    grid = orc.decode_e4m3(np.arange(0x7F, dtype=np.uint8)).astype(np.float64)
    mids = (grid[:-1] + grid[1:]) / 2                      # every tie point
    x = np.concatenate([rng.uniform(-448, 448, 20000), rng.standard_normal(20000) * 0.01, grid, -grid, mids, -mids,
                        np.nextafter(mids, 0), np.nextafter(mids, 1e9)]).astype(np.float32)
    x = x[np.abs(x) <= 448]
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(orc.encode_e4m3(x), want)


def test_e2m1_rounding_ties_and_saturation():
    x = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 7.0, 1e9, 0.2499, 0.2501, 5.0001, 4.9999, -0.25, -5.0, -7.0])
    want = np.array([0.0, 1.0, 1.0, 2.0, 2.0, 4.0, 4.0, 6.0, 6.0, 0.0, 0.5, 6.0, 4.0, -0.0, -4.0, -6.0])
    got = orc.decode_e2m1(orc.encode_e2m1(x))
    assert np.array_equal(got, want.astype(np.float32))
    # nearest-grid property on a dense sweep, by brute force over the 8 magnitudes
    xs = np.linspace(0, 6.5, 5001)
    got = orc.decode_e2m1(orc.encode_e2m1(xs)).astype(np.float64)
    grid = orc.E2M1_MAGNITUDES.astype(np.float64)
    best = np.abs(xs[:, None] - grid[None, :]).min(axis=1)
    assert np.allclose(np.abs(xs - got), best, atol=0)


def test_pack_is_low_nibble_first_and_round_trips():
    codes = np.arange(16, dtype=np.uint8).reshape(1, 16)
    packed = orc.pack_fp4(codes)
    assert packed.tolist() == [[0x10, 0x32, 0x54, 0x76, 0x98, 0xBA, 0xDC, 0xFE]]
    assert np.array_equal(orc.unpack_fp4(packed), codes)
    if hasattr(torch, "float4_e2m1fn_x2"):
        # torch's packed fp4 dtype uses the same byte layout (view only; no arithmetic needed)
        assert torch.from_numpy(packed).view(torch.float4_e2m1fn_x2).view(torch.uint8).numpy().tolist() == packed.tolist()


def test_mxfp4_quantiser_scale_rule_and_invariants():
    x = orc.activations_with_outliers(64, 256, seed=3)
    x[3, 32:64] = 0.0                                   # an all-zero block
    packed, scales = orc.quantize_mxfp4(x)
    xb = x.reshape(64, 8, 32).astype(np.float64)
    amax = np.abs(xb).max(-1)
    for r in range(64):
        for blk in range(8):
            if amax[r, blk] == 0:
                assert scales[r, blk] == 127 and not packed[r, blk * 16:(blk + 1) * 16].any()
            else:
                assert int(scales[r, blk]) - 127 == math.floor(math.log2(amax[r, blk])) - 2
    dq = orc.dequantize_mxfp4(packed, scales, np.float64)
    # the block's largest element lands on magnitude 4 or 6 (amax / scale is in [4, 8))
    top = np.abs(dq.reshape(64, 8, 32)).max(-1) / orc.decode_e8m0(scales)
    assert set(np.unique(top[amax > 0])) <= {4.0, 6.0}
    # idempotence: quantising the dequantised tensor changes nothing
    p2, s2 = orc.quantize_mxfp4(dq.astype(np.float32))
    assert np.array_equal(orc.dequantize_mxfp4(p2, s2, np.float64), dq)
    # error bound: half a grid step (<= 1 at the top of the range) times the scale, or saturation
    err = np.abs(dq - x.astype(np.float64)).reshape(64, 8, 32)
    assert (err <= 2.0 * orc.decode_e8m0(scales)[..., None] + 1e-30).all()
    # monotone: sorting a block before quantising gives sorted dequantised values
    blk = np.sort(x[0, :32])[None, :]
    q, s = orc.quantize_mxfp4(blk)
    assert (np.diff(orc.dequantize_mxfp4(q, s)[0]) >= 0).all()


def test_nvfp4_quantiser_scale_rule_and_exact_products():
    x = orc.randn((32, 128), seed=4)
    packed, sb, g = orc.quantize_nvfp4(x)
    assert g == np.float32(np.abs(x).max() / np.float32(448 * 6))
    amax = np.abs(x.reshape(32, 8, 16)).max(-1).astype(np.float64)
    want = torch.from_numpy(((amax / 6.0) / np.float64(g)).astype(np.float32)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(sb, want)
    # code x scale is exact in bf16, f16 and fp32 for every (code, finite scale byte)
    codes = np.repeat(np.arange(16, dtype=np.uint8), 16)[None, :]            # 256 elements: 16 blocks
    for s in range(256):
        if (s & 0x7F) == 0x7F:
            continue
        v64 = orc.dequantize_nvfp4_block(orc.pack_fp4(codes), np.full((1, 16), s, np.uint8), np.float64)
        t = torch.from_numpy(v64)
        assert torch.equal(t.to(torch.bfloat16).double(), t) and torch.equal(t.to(torch.float16).double(), t)
    dq = orc.dequantize_nvfp4(packed, sb, g)
    assert np.linalg.norm(dq - x) / np.linalg.norm(x) < 0.15


def test_mx_dequant_is_exact_product_of_table_and_power_of_two():
    codes = np.tile(np.arange(16, dtype=np.uint8), 2)[None, :]
    for s in range(255):
        v = orc.dequantize_mxfp4(orc.pack_fp4(codes), np.array([[s]], np.uint8), np.float64)[0]
        for c in range(16):
            assert Fraction(float(v[c])) == e2m1_from_fields(c) * Fraction(2) ** (s - 127)


def test_bf16_rounding_against_torch_and_single_rounding_from_f64():
    rng = np.random.default_rng(5)
    x = np.concatenate([rng.standard_normal(50000) * 10.0 ** rng.integers(-20, 20, 50000),
                        [1.00390625, 1.01171875, -1.00390625, 3.3895313892515355e38, 0.0, -0.0]]).astype(np.float32)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.uint16).numpy()
    assert np.array_equal(orc.f32_to_bf16_bits(x), want)
    # 1 + 2^-8 + 2^-30: fp32 rounding lands on the bf16 tie 1 + 2^-8 (would go to even = 1.0),
    # the correctly rounded bf16 of the fp64 value is 1 + 2^-7.
    v = np.array([1.0 + 2.0 ** -8 + 2.0 ** -30, 1.0 + 2.0 ** -8 - 2.0 ** -30, -(1.0 + 2.0 ** -8 + 2.0 ** -30)])
    got = orc.bf16_bits_to_f32(orc.f64_to_bf16_bits(v))
    assert got.tolist() == [1.0078125, 1.0, -1.0078125]
    assert orc.bf16_ulp(np.array([1.0, 1.5, 2.0, 0.75]))[[0, 1, 2, 3]].tolist() == [2.0 ** -7, 2.0 ** -7, 2.0 ** -6, 2.0 ** -8]


def brute_gemm_fraction(a, a_s, b, b_s, block, scale_decode):
    """Exact rational C = A . B^T straight from the bytes (independent of the oracle's numpy path)."""
    m, n, k = a.shape[0], b.shape[0], a.shape[1] * 2

    def elem(mat, sc, r, kk):
        byte = int(mat[r, kk // 2])
        code = (byte >> 4) if (kk & 1) else (byte & 0xF)
        return e2m1_from_fields(code) * scale_decode(int(sc[r, kk // block]))

    out = [[sum(elem(a, a_s, i, kk) * elem(b, b_s, j, kk) for kk in range(k)) for j in range(n)] for i in range(m)]
    return out


def e8m0_frac(byte):
    return Fraction(2) ** (byte - 127)


def e4m3_frac(byte):
    s, e, m = byte >> 7, (byte >> 3) & 0xF, byte & 7
    v = Fraction(m, 8) * Fraction(2) ** -6 if e == 0 else (1 + Fraction(m, 8)) * Fraction(2) ** (e - 7)
    return -v if s else v


def test_gemm_oracle_against_exact_rational_brute_force():
    a, a_s = orc.quantize_mxfp4(orc.randn((5, 64), seed=6))
    b, b_s = orc.quantize_mxfp4(orc.randn((7, 64), seed=7, std=0.02))
    exact = brute_gemm_fraction(a, a_s, b, b_s, 32, e8m0_frac)
    ref = orc.gemm_mxfp4_fp64(a, a_s, b, b_s)
    for i in range(5):
        for j in range(7):
            assert abs(Fraction(float(ref[i, j])) - exact[i][j]) <= abs(exact[i][j]) * Fraction(1, 2 ** 45)
    # a transposed or swapped operand would fail here: C is 5x7, not symmetric
    assert ref.shape == (5, 7)
    na, na_s, na_g = orc.quantize_nvfp4(orc.randn((4, 32), seed=8))
    nb, nb_s, nb_g = orc.quantize_nvfp4(orc.randn((6, 32), seed=9, std=0.02))
    exact = brute_gemm_fraction(na, na_s, nb, nb_s, 16, e4m3_frac)
    ref = orc.gemm_nvfp4_fp64(na, na_s, na_g, nb, nb_s, nb_g)
    gg = Fraction(float(np.float32(na_g))) * Fraction(float(np.float32(nb_g)))
    for i in range(4):
        for j in range(6):
            want = exact[i][j] * gg
            assert abs(Fraction(float(ref[i, j])) - want) <= abs(want) * Fraction(1, 2 ** 45)


def test_fp32_recipe_within_stated_tolerance_of_fp64():
    a, a_s = orc.quantize_mxfp4(orc.activations_with_outliers(256, 256, seed=0))
    b, b_s = orc.quantize_mxfp4(orc.randn((256, 256), seed=1))
    adq, bdq = orc.dequantize_mxfp4(a, a_s, np.float64), orc.dequantize_mxfp4(b, b_s, np.float64)
    ok, rep = orc.check_bf16_against_fp64(orc.gemm_mxfp4_fp32_bf16(a, a_s, b, b_s), adq @ bdq.T,
                                          np.abs(adq) @ np.abs(bdq).T, 256)
    assert ok, rep
    # the checker rejects a result that is off by two bf16 ulps in one element
    c = orc.f64_to_bf16_bits(adq @ bdq.T)
    c[10, 20] += 2
    assert not orc.check_bf16_against_fp64(c, adq @ bdq.T, np.abs(adq) @ np.abs(bdq).T, 256)[0]


def test_grouped_oracle_is_concatenation_of_plain_gemms():
    ro = np.array([0, 5, 5, 12], dtype=np.int32)
    a, a_s = orc.quantize_mxfp4(orc.randn((12, 64), seed=1))
    ws = [orc.quantize_mxfp4(orc.randn((8, 64), seed=2 + i)) for i in range(3)]
    b, b_s = np.stack([w[0] for w in ws]), np.stack([w[1] for w in ws])
    c = orc.grouped_gemm_mxfp4_fp64(a, a_s, b, b_s, ro)
    assert np.array_equal(c[0:5], orc.gemm_mxfp4_fp64(a[0:5], a_s[0:5], b[0], b_s[0]))
    assert np.array_equal(c[5:12], orc.gemm_mxfp4_fp64(a[5:12], a_s[5:12], b[2], b_s[2]))


def test_moe_routing_offsets():
    tok, ro = orc.moe_routing(1000, 8, 2, seed=5)
    assert ro[0] == 0 and ro[-1] == 2000 and (np.diff(ro) >= 0).all() and len(tok) == 2000
    # every token appears exactly twice, in two different experts
    assert (np.bincount(tok, minlength=1000) == 2).all()
    expert = np.searchsorted(ro, np.arange(2000), side="right") - 1
    for t in range(0, 1000, 97):
        assert len(set(expert[tok == t])) == 2


@pytest.mark.parametrize("name", ["mxfp4_32x48x64", "nvfp4_32x48x64", "grouped_mxfp4_45x32x64", "mxfp4_72x40x512",
                                  "nvfp4_24x40x512", "mxfp4_72x40x736", "nvfp4_72x40x320"])
def test_golden_fixtures_reproduce_and_match_exact_arithmetic(name):
    z = np.load(os.path.join(GOLDEN, name + ".npz"))
    if name.startswith("mxfp4"):
        ref = orc.gemm_mxfp4_fp64(z["a"], z["a_scale"], z["b"], z["b_scale"])
        exact = brute_gemm_fraction(z["a"][:4], z["a_scale"][:4], z["b"][:6], z["b_scale"][:6], 32, e8m0_frac)
        g = Fraction(1)
    elif name.startswith("nvfp4"):
        ref = orc.gemm_nvfp4_fp64(z["a"], z["a_scale"], z["a_global"], z["b"], z["b_scale"], z["b_global"])
        exact = brute_gemm_fraction(z["a"][:4], z["a_scale"][:4], z["b"][:6], z["b_scale"][:6], 16, e4m3_frac)
        g = Fraction(float(z["a_global"])) * Fraction(float(z["b_global"]))
    else:
        ref = orc.grouped_gemm_mxfp4_fp64(z["a"], z["a_scale"], z["b"], z["b_scale"], z["row_offsets"])
        exact = brute_gemm_fraction(z["a"][:4], z["a_scale"][:4], z["b"][0][:6], z["b_scale"][0][:6], 32, e8m0_frac)
        g = Fraction(1)
    assert np.array_equal(orc.f64_to_bf16_bits(ref), z["c_bf16_bits"])
    got = orc.bf16_bits_to_f32(z["c_bf16_bits"]).astype(np.float64)
    for i in range(4):
        for j in range(6):
            want = exact[i][j] * g
            # the stored bf16 is within half a bf16 ulp of the exact value
            assert abs(Fraction(float(got[i, j])) - want) <= Fraction(float(orc.bf16_ulp(np.array(float(want)))))/2


def _route_top2_brute(logits):
    """Pure-Python restatement: per token pick the two largest scores (ties to the lower index), list the
    (expert, token, rank) triples and sort them."""
    t, e = logits.shape
    rows = []
    for tok in range(t):
        order = sorted(range(e), key=lambda j: (-float(logits[tok, j]), j))
        z = [math.exp(float(logits[tok, j]) - float(max(logits[tok]))) for j in range(e)]
        for rank in range(2):
            rows.append((order[rank], tok, rank, z[order[rank]] / sum(z)))
    rows.sort(key=lambda r: (r[0], r[1], r[2]))
    offsets = [0] * (e + 1)
    for r in rows:
        offsets[r[0] + 1] += 1
    for j in range(e):
        offsets[j + 1] += offsets[j]
    return [r[1] for r in rows], offsets, [r[3] for r in rows]


@pytest.mark.parametrize("t,e,seed", [(1, 2, 0), (37, 8, 1), (200, 5, 2), (64, 32, 3)])
def test_route_top2_equals_brute_force(t, e, seed):
    logits = orc.randn((t, e), seed)
    if t > 10:
        logits[3] = logits[3, 0]          # all scores equal: experts 0 and 1
        logits[7, 1:] = logits[7, 0]
        logits[9, -1] = logits[9].max()   # a tie for first place
    tok, off, w = orc.route_top2(logits)
    btok, boff, bw = _route_top2_brute(logits)
    assert tok.dtype == np.int32 and off.dtype == np.int32
    assert tok.tolist() == btok and off.tolist() == boff
    assert np.allclose(w, bw, rtol=1e-12, atol=0)
    if t > 10:
        expert = np.searchsorted(off, np.arange(2 * t), side="right") - 1
        assert sorted(expert[tok == 3]) == [0, 1]


def test_route_top2_agrees_with_the_benchmark_routing_and_handles_no_tokens():
    tok, off, _ = orc.route_top2(orc.randn((1000, 8), 5))
    tok2, off2 = orc.moe_routing(1000, 8, 2, seed=5)
    assert np.array_equal(tok, tok2) and np.array_equal(off, off2)
    tok, off, w = orc.route_top2(np.zeros((0, 4), np.float32))
    assert len(tok) == 0 and off.tolist() == [0, 0, 0, 0, 0] and len(w) == 0


def test_gather_rows_is_plain_indexing_with_zero_rows_for_bad_indices():
    a, a_s = orc.quantize_mxfp4(orc.randn((6, 64), seed=9))
    idx = np.array([5, 0, 0, -1, 6, 3], dtype=np.int32)
    out, out_s = orc.gather_rows(a, a_s, idx)
    for i, j in enumerate(idx):
        if 0 <= j < 6:
            assert out[i].tolist() == a[j].tolist() and out_s[i].tolist() == a_s[j].tolist()
        else:
            assert not out[i].any() and not out_s[i].any()


@pytest.mark.parametrize("rows,cols", [(1, 1), (128, 4), (130, 5), (300, 128), (256, 896)])
def test_blocked_scale_layout_equals_the_index_formula_and_round_trips(rows, cols):
    """Independent restatement by byte offsets: tile (r//128, c//4) in row-major tile order, 512 bytes
    each; inside a tile, byte (r%32)*16 + ((r%128)//32)*4 + c%4."""
    rng = np.random.default_rng(rows * 1000 + cols)
    s = rng.integers(1, 256, size=(rows, cols), dtype=np.uint8)
    blocked = orc.scales_to_blocked(s)
    ct = (cols + 3) // 4
    assert blocked.shape == (((rows + 127) // 128) * 128 * ct * 4,)
    want = np.zeros_like(blocked)
    for r in range(rows):
        for c in range(cols):
            want[((r // 128) * ct + c // 4) * 512 + (r % 32) * 16 + ((r % 128) // 32) * 4 + c % 4] = s[r, c]
    assert np.array_equal(blocked, want)
    assert np.array_equal(orc.scales_from_blocked(blocked, rows, cols), s)


def test_swiglu_oracle_matches_torch_silu_and_a_hand_case():
    x = np.linspace(-30, 30, 241)
    assert np.allclose(orc.silu64(x), torch.nn.functional.silu(torch.from_numpy(x)).numpy(), rtol=1e-14, atol=1e-300)
    assert orc.silu64(np.array([0.0]))[0] == 0.0 and abs(orc.silu64(np.array([1.0]))[0] - 1 / (1 + math.exp(-1))) < 1e-16
    # one-hot activations: gate and up are single dequantised weights
    a = np.zeros((1, 32), np.float32)
    a[0, 0] = 2.0
    w = np.zeros((4, 32), np.float32)
    w[:, 0] = [1.0, -3.0, 0.5, 4.0]     # gate rows 0-1, up rows 2-3
    ap, asc = orc.quantize_mxfp4(a)
    wp, wsc = orc.quantize_mxfp4(w)
    h, gate, up = orc.gemm_mxfp4_swiglu_fp64(ap, asc, wp, wsc)
    assert gate.tolist() == [[2.0, -6.0]] and up.tolist() == [[1.0, 8.0]]
    assert abs(h[0, 0] - 2 / (1 + math.exp(-2))) < 1e-15 and abs(h[0, 1] + 48 / (1 + math.exp(6))) < 1e-14


def _round_f32(x):
    """A Python float (exact double) rounded once to float32, by the struct module (independent of numpy)."""
    import struct
    return struct.unpack("<f", struct.pack("<f", x))[0]


def _bf16_bits_of_f32(x):
    """Round-to-nearest-even of a float32 value onto bf16, on its bit pattern."""
    import struct
    u = struct.unpack("<I", struct.pack("<f", x))[0]
    if (u & 0x7FFFFFFF) > 0x7F800000:
        return (u >> 16) | 0x40
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF


@pytest.mark.parametrize("renormalize", [False, True])
def test_combine_top2_equals_a_scalar_restatement(renormalize):
    """rows_of_token inverts the routing, and the combine is two float32 products and one float32 sum per
    element, then one rounding to bf16 -- restated here element by element with Python doubles rounded through
    struct (a product or sum of two float32 values rounded once from its exact double is the IEEE result)."""
    t, e, h = 23, 6, 16
    logits = orc.randn((t, e), 11)
    tok, off, w = orc.route_top2(logits)
    inv = orc.rows_of_token(tok, logits)
    for tt in range(t):
        r0, r1 = inv[tt]
        assert tok[r0] == tt and tok[r1] == tt and r0 != r1
        e0 = np.searchsorted(off, r0, side="right") - 1
        e1 = np.searchsorted(off, r1, side="right") - 1
        assert (logits[tt, e0], -e0) >= (logits[tt, e1], -e1)          # first choice first
    rows = orc.f64_to_bf16_bits(orc.randn((2 * t, h), 12).astype(np.float64) * 3.0)
    w32 = w.astype(np.float32)
    inv_bad = inv.copy()
    inv_bad[5, 1] = 2 * t + 3                                           # out of range: contributes zeros
    got = orc.combine_top2(rows, inv_bad, w32, renormalize=renormalize)
    x = orc.bf16_bits_to_f32(rows)
    for tt in range(t):
        r0, r1 = int(inv_bad[tt, 0]), int(inv_bad[tt, 1])
        ok1 = r1 < 2 * t
        w0, w1 = float(w32[r0]), float(w32[r1]) if ok1 else 0.0
        if renormalize:
            total = _round_f32(w0 + w1)
            w0, w1 = _round_f32(w0 / total), _round_f32(w1 / total)
        for c in range(h):
            p0 = _round_f32(w0 * float(x[r0, c]))
            p1 = _round_f32(w1 * (float(x[r1, c]) if ok1 else 0.0))
            assert int(got[tt, c]) == _bf16_bits_of_f32(_round_f32(p0 + p1)), (tt, c)


def test_nvfp4_fp32_quantiser_equals_a_scalar_restatement():
    """quantize_nvfp4_fp32 (the device quantiser's recipe) block by block: float32 quotients formed as doubles and
    rounded once (innocuous for a quotient of two float32 values: 53 >= 2 * 24 + 2 bits), the scale byte by
    torch's float8_e4m3fn cast, the codes by a nearest-with-ties-to-even search over the E2M1 table in exact
    rationals."""
    x = orc.activations_with_outliers(6, 128, seed=31)
    x[1, 16:32] = 0.0                                  # an all-zero block
    x[2] *= 1e-6                                       # scales in the subnormal range of E4M3, some rounding to zero
    x[3, :16] = [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 7.0, -0.25, -5.0, 0.0, -0.0, 6.0, 4.0, 3.0, 2.0]
    g = np.float32(np.abs(x).max() / np.float32(448 * 6)) * np.float32(0.5)   # half the calibrated scale: some blocks saturate at 448
    packed, sb = orc.quantize_nvfp4_fp32(x, g)
    codes = orc.unpack_fp4(packed)
    grid = [Fraction(v) for v in (0, 0.5, 1, 1.5, 2, 3, 4, 6)]
    saturated = zero_scale = 0
    for r in range(x.shape[0]):
        for b in range(x.shape[1] // 16):
            blk = x[r, 16 * b:16 * b + 16]
            amax = float(np.abs(blk).max())
            u = _round_f32(_round_f32(amax / 6.0) / float(g))
            saturated += u > 448.0
            u = min(u, 448.0)
            byte = int(torch.tensor([u], dtype=torch.float32).to(torch.float8_e4m3fn).view(torch.uint8)[0])
            assert int(sb[r, b]) == byte, (r, b)
            d = _round_f32(float(torch.tensor([byte], dtype=torch.uint8).view(torch.float8_e4m3fn).float()[0]) * float(g))
            zero_scale += d == 0.0
            for j in range(16):
                q = Fraction(_round_f32(float(blk[j]) / d)) if d > 0 else Fraction(0)
                dist = [abs(abs(q) - v) for v in grid]
                best = min(dist)
                cands = [i for i, dv in enumerate(dist) if dv == best]
                mag = cands[0] if len(cands) == 1 else [i for i in cands if i % 2 == 0][0]   # tie: even code
                got = int(codes[r, 16 * b + j])
                assert (got & 7) == mag, (r, b, j)
                if mag:
                    assert (got >> 3) == int(blk[j] < 0), (r, b, j)
    assert saturated > 0 and zero_scale > 0              # both branches were exercised
    # with the calibrated global scale it is the fp64 recipe except next to rounding boundaries
    y = orc.randn((64, 256), seed=32)
    p64, s64, g64 = orc.quantize_nvfp4(y)
    p32, s32 = orc.quantize_nvfp4_fp32(y, g64)
    assert np.mean(s32 != s64) < 1e-3 and np.mean(orc.unpack_fp4(p32) != orc.unpack_fp4(p64)) < 2e-3


def test_golden_nvfp4_quantiser_fixture_reproduces():
    z = np.load(os.path.join(GOLDEN, "quantize_nvfp4_8x64.npz"))
    packed, sb = orc.quantize_nvfp4_fp32(z["x"], z["global_scale"])
    assert np.array_equal(packed, z["packed"]) and np.array_equal(sb, z["scales"])
    # decoded, it is the input to within half a grid step of every block (or the clamp at 6 steps)
    dq = orc.dequantize_nvfp4(z["packed"], z["scales"], z["global_scale"])
    step = orc.decode_e4m3(z["scales"]).astype(np.float64) * float(z["global_scale"])
    err = np.abs(dq - z["x"]).reshape(8, 4, 16)
    inside = np.abs(z["x"]).reshape(8, 4, 16) <= 6 * step[..., None]
    assert (err[inside] <= (step[..., None] * np.ones((1, 1, 16)))[inside] + 1e-12).all()



def test_quantisers_mark_blocks_with_non_finite_values():
    """A block that holds an infinity or a NaN gets the NaN scale byte of its format (0xFF in E8M0, 0x7F in E4M3, both
    NaN under the library decoders pinned above) and zero codes; it dequantises to NaN, and the other blocks of the
    row are what they are without the non-finite values."""
    rng = np.random.default_rng(9)
    x = rng.standard_normal((6, 128)).astype(np.float32)
    clean = x.copy()
    x[0, 5] = np.inf
    x[1, 40] = -np.inf
    x[2, 64] = np.nan
    x[3, 96:128] = np.nan
    x[4, 31], x[4, 32] = np.inf, np.nan          # neighbouring blocks
    bad_mx = np.zeros((6, 4), dtype=bool)
    bad_mx[0, 0] = bad_mx[1, 1] = bad_mx[2, 2] = bad_mx[3, 3] = bad_mx[4, 0] = bad_mx[4, 1] = True
    p, s = orc.quantize_mxfp4(x)
    cp, cs = orc.quantize_mxfp4(clean)
    assert np.array_equal(s == 0xFF, bad_mx)
    assert np.array_equal(s[~bad_mx], cs[~bad_mx])
    codes, ccodes = orc.unpack_fp4(p).reshape(6, 4, 32), orc.unpack_fp4(cp).reshape(6, 4, 32)
    assert not codes[bad_mx].any() and np.array_equal(codes[~bad_mx], ccodes[~bad_mx])
    dq = orc.dequantize_mxfp4(p, s).reshape(6, 4, 32)
    assert np.isnan(dq[bad_mx]).all() and np.isfinite(dq[~bad_mx]).all()
    assert torch.isnan(torch.tensor([0xFF], dtype=torch.uint8).view(torch.float8_e8m0fnu).float()).all()
    # NVFP4, blocks of 16
    g = np.float32(np.abs(clean).max() / (448 * 6))
    bad_nv = np.zeros((6, 8), dtype=bool)
    bad_nv[0, 0] = bad_nv[1, 2] = bad_nv[2, 4] = bad_nv[3, 6] = bad_nv[3, 7] = bad_nv[4, 1] = bad_nv[4, 2] = True
    p, s = orc.quantize_nvfp4_fp32(x, g)
    cp, cs = orc.quantize_nvfp4_fp32(clean, g)
    assert np.array_equal(s == 0x7F, bad_nv) and np.array_equal(s[~bad_nv], cs[~bad_nv])
    codes, ccodes = orc.unpack_fp4(p).reshape(6, 8, 16), orc.unpack_fp4(cp).reshape(6, 8, 16)
    assert not codes[bad_nv].any() and np.array_equal(codes[~bad_nv], ccodes[~bad_nv])
    assert np.isnan(orc.dequantize_nvfp4_block(p, s).reshape(6, 8, 16)[bad_nv]).all()
    assert torch.isnan(torch.tensor([0x7F], dtype=torch.uint8).view(torch.float8_e4m3fn).float()).all()
