"""Decoded FP4 x scale values, bit for bit, on every hot kernel (through the C ABI).

One operand ("varied") carries all 16 E2M1 codes under EVERY finite scale byte -- E8M0 0..254 for MXFP4, E4M3
0x00..0x7E and 0x80..0xFE for NVFP4 -- the other is one-hot (code 1.0 at one k per row), so every output element is
a single product: C[i][j] = dq(varied)[., k*] * dq(onehot)[., k*], which the fp32 accumulator and the bf16 store
hold exactly.  Expected bits come from the oracle's dequantisers (the reference's recipe: upcast, matmul, round to
bf16, compare on the CPU -- test/examples/gemm/amdgpu/test_amdgpu_gemm.py:24-38).

MXFP4: 2^-127 and 2^127 times a code leave the range of normal bf16 numbers, so the one-hot operand's scale of a
k-block is 2^64, 1 or 2^-64 according to the bytes that the varied operand holds in that block (blocks 0-3: bytes
0..63, blocks 4-11: 64..191, blocks 12-15: 192..254): every product is a normal number, and a wrong decode of any
byte still shows.  Both operand sides are varied in turn: they reach the matrix cores through different scale
operands, different LDS rows and (NVFP4) different conversion code.
"""
import numpy as np
import pytest
import torch

from avelang_amd import _lib
from tests import helpers as H
from tests.onehot_patterns import (E4M3_FINITE, mx_expect, mx_onehot, mx_varied, nv_expect, nv_onehot, nv_varied,
                                   same_bits as _same_bits)

pytestmark = pytest.mark.gpu
AUTO, GENERIC, TILE, DECODE, NARROW = 0, 1, 2, 3, 4


# ---------------------------------------------------------------- MXFP4
def _mx_split(device, a, a_s, b, b_s, slice_pairs, narrow):
    lib = _lib.load()
    m, k = a.shape[0], a.shape[1] * 2
    n = b.shape[0]
    slices = -(-(k // 512) // slice_pairs)
    ws = torch.full((slices * m * n,), float("nan"), dtype=torch.float32, device=device)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=device)
    da, das, db, dbs = (H.to_dev(x, device) for x in (a, a_s, b, b_s))
    _lib.check(lib.ave_fp4_debug_gemm_mxfp4_splitk(da.data_ptr(), das.data_ptr(), db.data_ptr(), dbs.data_ptr(),
                                                   out.data_ptr(), m, n, k, ws.data_ptr(), ws.numel() * 4, slice_pairs,
                                                   narrow, torch.cuda.current_stream(device).cuda_stream))
    torch.cuda.synchronize(device)
    return H.bits(out)


# (label, variant, K, rows of the one-hot operand per call when it is A, rows of the varied operand when it is A)
#  TILE K=512: pair scales, persistent form; K=768: scales per stage, one workgroup per tile
#  TILE K=992: one pair of stages from LDS, then 15 blocks straight from global memory (31-byte scale rows)
#  NARROW 256 rows: 256 x 128 tiles, three stage buffers; 128 rows: 128 x 128 tiles, four stage buffers
MX_TILE_LIKE = [("tile_pair_scales", TILE, 512, 512, 272), ("tile_stage_scales", TILE, 768, 768, 272),
                ("tile_k_tail", TILE, 992, 496, 272),
                ("narrow_256x128", NARROW, 512, 256, 272), ("narrow_128x128", NARROW, 512, 128, 112),
                ("narrow_long_k", NARROW, 2048, 256, 144), ("generic", GENERIC, 512, 512, 48)]


@pytest.mark.parametrize("label,variant,k,onehot_rows,varied_rows", MX_TILE_LIKE, ids=[c[0] for c in MX_TILE_LIKE])
def test_mx_weight_side_every_scale_byte(gpu, label, variant, k, onehot_rows, varied_rows):
    """B varied (528 rows: every byte at 33 row positions, ragged last tile), A one-hot over windows of K."""
    b, b_s = mx_varied(528, k)
    for first in range(0, k, onehot_rows):
        a, a_s = mx_onehot(first, onehot_rows, k)
        _same_bits(H.run_mx(gpu, a, a_s, b, b_s, variant=variant), mx_expect(a, a_s, b, b_s))


@pytest.mark.parametrize("label,variant,k,onehot_rows,varied_rows", MX_TILE_LIKE, ids=[c[0] for c in MX_TILE_LIKE])
def test_mx_activation_side_every_scale_byte(gpu, label, variant, k, onehot_rows, varied_rows):
    """A varied, B one-hot with one row per k."""
    a, a_s = mx_varied(varied_rows, k)
    b, b_s = mx_onehot(0, k, k)
    _same_bits(H.run_mx(gpu, a, a_s, b, b_s, variant=variant), mx_expect(a, a_s, b, b_s))


# weight-streaming kernels: rows of A, K.  16/32/64 rows = one, two, four row blocks on the LDS rings (K % 512 == 0,
# K % 1024 == 0 above 32 rows; K = 2048 and 4096 take wider panels); K = 640 with 16 rows is the register kernel,
# (K below 512 only), K = 672 through the rings with five more blocks behind the first 512 elements
# K = 992, 1568, 2144: whole units of 512 on the rings (one, two, four row blocks), 15 / 1 / 3 more blocks from
# global memory behind them
MX_DECODE = [(16, 512), (32, 512), (64, 1024), (16, 2048), (16, 4096), (16, 640), (9, 1024), (16, 672), (16, 992), (32, 1568),
             (64, 2144)]


@pytest.mark.parametrize("m,k", MX_DECODE)
def test_mx_decode_activation_side_every_scale_byte(gpu, m, k):
    a, a_s = mx_varied(m, k)
    if m < 16:   # fewer than 16 rows do not hold every byte: shift the pattern over two calls
        a2, a2_s = mx_varied(16 + m, k)
        a, a_s = np.concatenate([a, a2[16:]]), np.concatenate([a_s, a2_s[16:]])
    b, b_s = mx_onehot(0, k, k)
    for r0 in range(0, a.shape[0], m):
        _same_bits(H.run_mx(gpu, a[r0:r0 + m], a_s[r0:r0 + m], b, b_s, variant=DECODE),
                   mx_expect(a[r0:r0 + m], a_s[r0:r0 + m], b, b_s))


@pytest.mark.parametrize("m,k", MX_DECODE)
def test_mx_decode_weight_side_every_scale_byte(gpu, m, k):
    b, b_s = mx_varied(7 * 16 * 3 + 24, k)   # more than one workgroup's tiles, ragged last tile
    for first in range(0, k, m * (k // 512 if k >= 2048 else 1)):   # long K: a sample of the windows
        if first + m > k:
            break
        a, a_s = mx_onehot(first, m, k)
        _same_bits(H.run_mx(gpu, a, a_s, b, b_s, variant=DECODE), mx_expect(a, a_s, b, b_s))


@pytest.mark.parametrize("narrow", [0, 1, 2])
def test_mx_split_k_every_scale_byte(gpu, narrow):
    """K = 1024 in two slices: the one-hot product sits in one slice, the other adds an exact zero."""
    k = 1024
    b, b_s = mx_varied(528, k)
    rows = 128 if narrow == 2 else 256
    for first in range(0, k, rows):
        a, a_s = mx_onehot(first, rows, k)
        _same_bits(_mx_split(gpu, a, a_s, b, b_s, 1, narrow), mx_expect(a, a_s, b, b_s))
    a, a_s = mx_varied(112 if narrow == 2 else 272, k)
    b, b_s = mx_onehot(0, k, k)
    _same_bits(_mx_split(gpu, a, a_s, b, b_s, 1, narrow), mx_expect(a, a_s, b, b_s))


@pytest.mark.parametrize("variant", [TILE, NARROW])
def test_mx_grouped_every_scale_byte(gpu, variant):
    """Three experts with weights of their own (the varied pattern shifted by the expert index), ragged row ranges."""
    k, n = 512, 272
    row_offsets = np.array([0, 200, 200, 512], dtype=np.int32)
    a, a_s = mx_onehot(0, 512, k)
    ws = [mx_varied(n + 16 * e, k) for e in range(3)]
    b = np.stack([w[0][16 * e:] for e, w in enumerate(ws)])
    b_s = np.stack([w[1][16 * e:] for e, w in enumerate(ws)])
    got = H.run_grouped(gpu, a, a_s, b, b_s, row_offsets, variant=variant)
    for e in range(3):
        r0, r1 = row_offsets[e], row_offsets[e + 1]
        if r1 > r0:
            _same_bits(got[r0:r1], mx_expect(a[r0:r1], a_s[r0:r1], b[e], b_s[e]))


# ---------------------------------------------------------------- NVFP4
def _nv_ws(device, a, a_s, a_g, b, b_s, b_g):
    """ave_fp4_gemm_nvfp4_ws with the workspace it asks for (K split over the compute units)."""
    lib = _lib.load()
    m, k = a.shape[0], a.shape[1] * 2
    n = b.shape[0]
    need = lib.ave_fp4_gemm_nvfp4_workspace_bytes(m, n, k)
    assert need > 0, "shape chosen so that K is split"
    ws = torch.full((need // 4,), float("nan"), dtype=torch.float32, device=device)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=device)
    ag = torch.tensor([a_g], dtype=torch.float32, device=device)
    bg = torch.tensor([b_g], dtype=torch.float32, device=device)
    da, das, db, dbs = (H.to_dev(x, device) for x in (a, a_s, b, b_s))
    _lib.check(lib.ave_fp4_gemm_nvfp4_ws(da.data_ptr(), das.data_ptr(), ag.data_ptr(), db.data_ptr(), dbs.data_ptr(),
                                         bg.data_ptr(), out.data_ptr(), m, n, k, ws.data_ptr(), need,
                                         torch.cuda.current_stream(device).cuda_stream))
    torch.cuda.synchronize(device)
    return H.bits(out)


NV_G = (0.5, 4.0)   # per-tensor scales: powers of two, so the product stays exact


@pytest.mark.parametrize("variant,k", [(TILE, 512), (TILE, 768), (GENERIC, 512)])
def test_nv_tile_every_scale_byte_both_sides(gpu, variant, k):
    b, b_s = nv_varied(528, k)
    a, a_s = nv_onehot(0, k, k)
    _same_bits(H.run_nv(gpu, a, a_s, NV_G[0], b, b_s, NV_G[1], variant=variant), nv_expect(a, a_s, NV_G[0], b, b_s, NV_G[1]))
    # 272 rows: four waves of 128 x 128; 100 rows: eight waves of 64 x 128 (the tile kernel's form for at most 128 rows)
    for rows in (272, 100):
        a, a_s = nv_varied(rows, k)
        b, b_s = nv_onehot(0, k, k)
        _same_bits(H.run_nv(gpu, a, a_s, NV_G[0], b, b_s, NV_G[1], variant=variant), nv_expect(a, a_s, NV_G[0], b, b_s, NV_G[1]))


# rows of A, K: up to 32 rows with K % 512 == 0 run on the LDS rings, everything else on the register kernel
NV_DECODE = [(16, 512), (32, 512), (16, 2048), (48, 512), (64, 1024), (16, 640), (8, 1024), (16, 992), (32, 1056)]   # the last two: rings with a K tail


@pytest.mark.parametrize("m,k", NV_DECODE)
def test_nv_decode_every_scale_byte_both_sides(gpu, m, k):
    a, a_s = nv_varied(max(m, 8), k)
    b, b_s = nv_onehot(0, k, k)
    _same_bits(H.run_nv(gpu, a[:m], a_s[:m], NV_G[0], b, b_s, NV_G[1], variant=DECODE),
               nv_expect(a[:m], a_s[:m], NV_G[0], b, b_s, NV_G[1]))
    b, b_s = nv_varied(7 * 16 * 3 + 24, k)
    step = m * (k // 512 if k >= 2048 else 1)
    for first in range(0, k - m + 1, step):
        a, a_s = nv_onehot(first, m, k)
        _same_bits(H.run_nv(gpu, a, a_s, NV_G[0], b, b_s, NV_G[1], variant=DECODE),
                   nv_expect(a, a_s, NV_G[0], b, b_s, NV_G[1]))


def test_nv_split_k_every_scale_byte(gpu):
    k = 2048   # eight stages: the planner cuts them into slices for these few tiles
    b, b_s = nv_varied(528, k)
    for first in (0, 768, k - 256):
        a, a_s = nv_onehot(first, 256, k)
        _same_bits(_nv_ws(gpu, a, a_s, NV_G[0], b, b_s, NV_G[1]), nv_expect(a, a_s, NV_G[0], b, b_s, NV_G[1]))
    a, a_s = nv_varied(144, k)
    for first in range(0, k, 512):
        b, b_s = nv_onehot(first, 512, k)
        _same_bits(_nv_ws(gpu, a, a_s, NV_G[0], b, b_s, NV_G[1]), nv_expect(a, a_s, NV_G[0], b, b_s, NV_G[1]))


# ---------------------------------------------------------------- random operands, scale bytes over the whole range
def _mx_full_range_scales(rng, m, n, k):
    """Per k-block a base exponent anywhere in the E8M0 range; A takes base + jitter, B the mirror image, so that
    every byte 0..254 occurs while the products stay within 2^+-24 of one."""
    base = rng.integers(0, 255, size=k // 32)
    base[0], base[1] = 0, 254   # both ends of the range on both operands, whatever the draw
    a_s = np.clip(base[None, :] + rng.integers(-6, 7, size=(m, k // 32)), 0, 254).astype(np.uint8)
    b_s = np.clip(254 - base[None, :] + rng.integers(-6, 7, size=(n, k // 32)), 0, 254).astype(np.uint8)
    return a_s, b_s


MX_RANDOM = [("tile", TILE, 256, 520, 2048), ("tile_stage_scales", TILE, 300, 256, 768), ("narrow", NARROW, 200, 392, 3584),
             ("narrow_half", NARROW, 100, 392, 2048), ("ring16", DECODE, 16, 640, 4096), ("ring64", DECODE, 64, 336, 2048),
             ("register", DECODE, 16, 336, 1664)]


@pytest.mark.parametrize("label,variant,m,n,k", MX_RANDOM, ids=[c[0] for c in MX_RANDOM])
def test_mx_random_codes_scale_bytes_over_the_whole_range(gpu, label, variant, m, n, k):
    rng = np.random.default_rng(11)
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    a_s, b_s = _mx_full_range_scales(rng, m, n, k)
    assert a_s.min() == 0 and a_s.max() == 254 and b_s.min() == 0 and b_s.max() == 254
    H.assert_mx_close(H.run_mx(gpu, a, a_s, b, b_s, variant=variant), a, a_s, b, b_s)


NV_RANDOM = [("tile", TILE, 256, 264, 1024), ("tile_up_to_128_rows", TILE, 100, 264, 1024), ("ring", DECODE, 32, 336, 2048), ("register", DECODE, 64, 336, 1152)]


@pytest.mark.parametrize("label,variant,m,n,k", NV_RANDOM, ids=[c[0] for c in NV_RANDOM])
def test_nv_random_codes_every_finite_scale_byte(gpu, label, variant, m, n, k):
    """E4M3 bytes drawn from all 254 finite ones (both signs, subnormals, the top binade): |a||b| <= 448^2 * 36
    per product, far inside fp32 and bf16 range."""
    rng = np.random.default_rng(12)
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    a_s = E4M3_FINITE[rng.integers(0, 254, size=(m, k // 16))]
    b_s = E4M3_FINITE[rng.integers(0, 254, size=(n, k // 16))]
    c = H.run_nv(gpu, a, a_s, 2.0 ** -9, b, b_s, 2.0 ** -8, variant=variant)
    H.assert_nv_close(c, a, a_s, 2.0 ** -9, b, b_s, 2.0 ** -8)
