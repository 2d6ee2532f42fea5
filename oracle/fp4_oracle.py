"""CPU oracle for the block-scaled FP4 GEMM path.  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the benchmark's CPU-baseline leg may import this
module; the shipped library never does.

What it restates
----------------
The reference has no FP4 code.  The numerical recipe it does define for a GEMM
``C[M,N] = A[M,K] . B[N,K]^T`` is "upcast operands to fp32, matmul, round to
bf16, compare on the CPU":

* reference ``test/examples/gemm/amdgpu/test_amdgpu_gemm.py:24-38``
* reference ``benchmark/gemm/bench_amdgpu_gemm.py:62-68``
* operand convention (B stored ``[N, K]``, bf16 output, ``out=`` semantics):
  reference ``python/avelang_kernels/amdgpu_gemm.py:458-494``

:func:`gemm_dequant_fp32` follows that recipe with a dequantise step in front.
:func:`gemm_dequant_fp64` is the exact-arithmetic checker the tolerance is stated
against.

Beyond the GEMM it also restates the steps either side of it that the library
runs on the device: MoE top-2 routing, the row gather in front of the grouped GEMM
(:func:`route_top2`, :func:`gather_rows`) and the blocked scale layout
(:func:`scales_to_blocked`), and the device NVFP4 quantiser's fp32-step recipe
(:func:`quantize_nvfp4_fp32`).  The reference has none of these; each is pinned in
``tests/test_oracle_formats.py`` by an independent pure-Python brute force.

Parity status
-------------
PARITY UNPINNED by the reference for every format function below (E2M1, E8M0,
E4M3 decode, both quantisers, nibble packing): the reference holds no golden
vector, fixture or test for them.  They are pinned instead by closed forms and
library routines in ``tests/test_oracle_formats.py``: the 16-entry E2M1 table and
``ldexp`` for E8M0 (OCP Microscaling v1.0), ``torch.float8_e4m3fn`` casts for
E4M3 in both directions, the round-to-nearest-even tie table, idempotence and
monotonicity of the quantisers, and a pure-Python ``fractions`` brute force for
the GEMM.  The GEMM recipe itself (fp32 upcast, matmul, bf16 round) is pinned by
the reference lines above.
"""
from __future__ import annotations

import numpy as np

# --------------------------------------------------------------------------
# Element and scale formats
# --------------------------------------------------------------------------

#: magnitudes of the eight E2M1 codes 0..7 (bit 3 of the code is the sign)
E2M1_MAGNITUDES = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=np.float32)
#: all sixteen codes -> value
E2M1_TABLE = np.concatenate([E2M1_MAGNITUDES, -E2M1_MAGNITUDES]).astype(np.float32)

MX_BLOCK = 32   # K elements per E8M0 scale
NV_BLOCK = 16   # K elements per E4M3 scale
E4M3_MAX = 448.0
E2M1_MAX = 6.0


def decode_e2m1(codes: np.ndarray) -> np.ndarray:
    """4-bit codes (uint8, values 0..15) -> float32 values."""
    return E2M1_TABLE[np.asarray(codes, dtype=np.uint8) & 0xF]


def decode_e8m0(b: np.ndarray) -> np.ndarray:
    """E8M0 bytes -> float64 ``2**(b-127)``; byte 0xFF is NaN (OCP MX v1.0)."""
    b = np.asarray(b, dtype=np.uint8)
    out = np.ldexp(1.0, b.astype(np.int32) - 127)
    return np.where(b == 0xFF, np.nan, out)


def decode_e4m3(b: np.ndarray) -> np.ndarray:
    """E4M3 ("fn": no infinities, S.1111.111 is NaN) bytes -> float32."""
    b = np.asarray(b, dtype=np.uint8).astype(np.int32)
    sign = np.where(b & 0x80, -1.0, 1.0)
    e = (b >> 3) & 0xF
    m = b & 0x7
    normal = np.ldexp(1.0 + m / 8.0, e - 7)
    sub = np.ldexp(m / 8.0, -6)
    v = np.where(e == 0, sub, normal)
    v = np.where((e == 15) & (m == 7), np.nan, v)
    return (sign * v).astype(np.float32)


def _rne_to_grid(x: np.ndarray, grid: np.ndarray) -> np.ndarray:
    """Index of the nearest entry of an ascending ``grid`` for non-negative ``x``;
    ties go to the even index; values above the top saturate."""
    x = np.asarray(x, dtype=np.float64)
    hi = np.searchsorted(grid, x, side="left")          # first grid >= x
    hi = np.clip(hi, 0, len(grid) - 1)
    lo = np.clip(hi - 1, 0, len(grid) - 1)
    dlo = np.abs(x - grid[lo])
    dhi = np.abs(grid[hi] - x)
    pick_hi = (dhi < dlo) | ((dhi == dlo) & (hi % 2 == 0))
    idx = np.where(pick_hi, hi, lo)
    return np.where(x >= grid[-1], len(grid) - 1, idx).astype(np.uint8)


def encode_e2m1(x: np.ndarray) -> np.ndarray:
    """float -> E2M1 code, round-to-nearest-even on the grid, saturating at +-6.
    Negative zero and values rounding to zero keep their sign bit."""
    x = np.asarray(x, dtype=np.float64)
    mag = _rne_to_grid(np.abs(x), E2M1_MAGNITUDES.astype(np.float64))
    return (mag | np.where(np.signbit(x), 8, 0)).astype(np.uint8)


_E4M3_POS = None


def _e4m3_positive_grid() -> np.ndarray:
    global _E4M3_POS
    if _E4M3_POS is None:
        _E4M3_POS = decode_e4m3(np.arange(0, 0x7F, dtype=np.uint8)).astype(np.float64)  # 0 .. 448
    return _E4M3_POS


def encode_e4m3(x: np.ndarray) -> np.ndarray:
    """float -> E4M3 byte, round-to-nearest-even, saturating at +-448 (finite input)."""
    x = np.asarray(x, dtype=np.float64)
    grid = _e4m3_positive_grid()
    # consecutive codes are consecutive grid points and code parity == mantissa parity
    mag = _rne_to_grid(np.abs(x), grid)
    return (mag | np.where(np.signbit(x), 0x80, 0)).astype(np.uint8)


# --------------------------------------------------------------------------
# Packing: two codes per byte, LOW nibble = even k
# --------------------------------------------------------------------------

def pack_fp4(codes: np.ndarray) -> np.ndarray:
    codes = np.asarray(codes, dtype=np.uint8)
    assert codes.shape[-1] % 2 == 0
    return (codes[..., 0::2] & 0xF) | ((codes[..., 1::2] & 0xF) << 4)


def unpack_fp4(packed: np.ndarray) -> np.ndarray:
    packed = np.asarray(packed, dtype=np.uint8)
    out = np.empty(packed.shape[:-1] + (packed.shape[-1] * 2,), dtype=np.uint8)
    out[..., 0::2] = packed & 0xF
    out[..., 1::2] = packed >> 4
    return out


# --------------------------------------------------------------------------
# Quantisers (the synthetic-input recipe of the benchmark configurations)
# --------------------------------------------------------------------------

def quantize_mxfp4(x: np.ndarray):
    """fp32 ``[R, K]`` -> (packed ``uint8 [R, K/2]``, scales ``uint8 [R, K/32]``).

    Per 32-element K block: shared scale ``2**(floor(log2(amax)) - 2)`` stored as an
    E8M0 byte (exponent clamped to [-127, 127]); elements are divided by it and
    rounded to nearest-even onto the E2M1 grid, saturating at +-6.  An all-zero
    block gets scale byte 127 (1.0) and zero codes.  A block that holds an infinity
    or a NaN gets scale byte 0xFF (the E8M0 NaN) and zero codes, so that it
    dequantises to NaN and every GEMM result that uses it is NaN: a non-finite
    input stays visible instead of turning into a saturated finite block.
    """
    x = np.asarray(x, dtype=np.float32)
    R, K = x.shape
    assert K % MX_BLOCK == 0
    xb = x.reshape(R, K // MX_BLOCK, MX_BLOCK).astype(np.float64)
    bad = ~np.isfinite(xb).all(axis=-1)
    xb = np.where(bad[..., None], 0.0, xb)
    amax = np.abs(xb).max(axis=-1)
    # floor(log2(amax)) via frexp: exact, where log2 may round across an integer
    _, ex = np.frexp(amax)
    e = np.where(amax > 0, ex - 1, 0).astype(np.int64)
    e = np.clip(e - 2, -127, 127)
    e = np.where(amax > 0, e, 0)
    scale_bytes = np.where(bad, 0xFF, e + 127).astype(np.uint8)
    q = xb / np.ldexp(1.0, e)[..., None]
    codes = encode_e2m1(q).reshape(R, K)
    return pack_fp4(codes), scale_bytes


def quantize_nvfp4(x: np.ndarray):
    """fp32 ``[R, K]`` -> (packed ``[R, K/2]``, E4M3 scales ``[R, K/16]``, fp32 global scale).

    Global scale ``amax(x) / (448 * 6)``; block scale ``(amax_block / 6) / global``
    rounded to E4M3 (RNE, saturating); elements divided by ``decoded_scale * global``
    and rounded to nearest-even onto the E2M1 grid.
    """
    x = np.asarray(x, dtype=np.float32)
    R, K = x.shape
    assert K % NV_BLOCK == 0
    g = np.float32(np.abs(x).max() / np.float32(E4M3_MAX * E2M1_MAX))
    if g == 0:
        g = np.float32(1.0)
    xb = x.reshape(R, K // NV_BLOCK, NV_BLOCK).astype(np.float64)
    amax = np.abs(xb).max(axis=-1)
    sb = encode_e4m3((amax / E2M1_MAX) / np.float64(g))
    sdec = decode_e4m3(sb).astype(np.float64) * np.float64(g)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.where(sdec[..., None] > 0, xb / sdec[..., None], 0.0)
    codes = encode_e2m1(q).reshape(R, K)
    return pack_fp4(codes), sb, g


def quantize_nvfp4_fp32(x: np.ndarray, g) -> tuple:
    """fp32 ``[R, K]`` and a given per-tensor scale ``g`` -> (packed ``[R, K/2]``, E4M3 scales ``[R, K/16]``): the
    recipe of the device quantiser, every step one IEEE fp32 operation:
    ``u = min((amax / 6) / g, 448)``; scale byte ``E4M3(u)`` (RNE); ``d = decode(byte) * g``;
    codes ``E2M1(x / d)`` (RNE, saturating), zero codes where ``d == 0``.  A block that holds an infinity or a NaN
    gets scale byte 0x7F (the E4M3 NaN) and zero codes.
    Differs from :func:`quantize_nvfp4` (fp64 quotients, its own ``g``) only next to rounding boundaries."""
    x = np.asarray(x, dtype=np.float32)
    g = np.float32(g)
    R, K = x.shape
    assert K % NV_BLOCK == 0 and g > 0
    xb = x.reshape(R, K // NV_BLOCK, NV_BLOCK)
    bad = ~np.isfinite(xb).all(axis=-1)
    xb = np.where(bad[..., None], np.float32(0), xb)
    amax = np.abs(xb).max(axis=-1).astype(np.float32)
    with np.errstate(over="ignore", under="ignore"):
        u = np.minimum((amax / np.float32(E2M1_MAX)) / g, np.float32(E4M3_MAX)).astype(np.float32)
        sb = encode_e4m3(u)
        d = (decode_e4m3(sb).astype(np.float32) * g).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore", over="ignore", under="ignore"):
        q = np.where(d[..., None] > 0, xb / d[..., None], np.float32(0)).astype(np.float32)
    codes = encode_e2m1(q).reshape(R, K)
    return pack_fp4(codes), np.where(bad, 0x7F, sb).astype(np.uint8)


# --------------------------------------------------------------------------
# Dequantise
# --------------------------------------------------------------------------

def dequantize_mxfp4(packed: np.ndarray, scales: np.ndarray, dtype=np.float32) -> np.ndarray:
    """value = E2M1(code) * 2**(scale-127); exact in fp32 (and in fp64)."""
    v = decode_e2m1(unpack_fp4(packed)).astype(np.float64)
    R, K = v.shape
    s = decode_e8m0(scales)
    out = v.reshape(R, K // MX_BLOCK, MX_BLOCK) * s[..., None]
    return out.reshape(R, K).astype(dtype)


def dequantize_nvfp4_block(packed: np.ndarray, scales: np.ndarray, dtype=np.float32) -> np.ndarray:
    """value = E2M1(code) * E4M3(scale): at most 6 significant bits, exact in
    bf16/f16/fp32.  The per-tensor fp32 scale is NOT applied here."""
    v = decode_e2m1(unpack_fp4(packed)).astype(np.float64)
    R, K = v.shape
    s = decode_e4m3(scales).astype(np.float64)
    out = v.reshape(R, K // NV_BLOCK, NV_BLOCK) * s[..., None]
    return out.reshape(R, K).astype(dtype)


def dequantize_nvfp4(packed, scales, global_scale, dtype=np.float64) -> np.ndarray:
    return (dequantize_nvfp4_block(packed, scales, np.float64) * np.float64(global_scale)).astype(dtype)


# --------------------------------------------------------------------------
# bf16 helpers
# --------------------------------------------------------------------------

def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bit pattern (uint16), round-to-nearest-even, NaN stays NaN."""
    x = np.asarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    rounded = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    nan = np.isnan(x)
    return np.where(nan, np.uint16(0x7FC0), rounded).astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f64_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """fp64 -> bf16 with a single rounding (no double rounding through fp32)."""
    x = np.asarray(x, dtype=np.float64)
    f = x.astype(np.float32)                     # RNE to fp32
    # detect double-rounding hazard: fp32 value sits exactly on a bf16 tie but x did not
    u = f.view(np.uint32)
    tie = (u & 0xFFFF) == 0x8000
    fx = f.astype(np.float64)
    adj = np.where(tie & (np.abs(x) > np.abs(fx)), 1, 0) - np.where(tie & (np.abs(x) < np.abs(fx)), 1, 0)
    u2 = (u.astype(np.int64) + adj).astype(np.uint32)
    return f32_to_bf16_bits(u2.view(np.float32))


def bf16_ulp(x: np.ndarray) -> np.ndarray:
    """Spacing of bf16 numbers at magnitude |x| (fp64), with the subnormal floor."""
    x = np.abs(np.asarray(x, dtype=np.float64))
    _, ex = np.frexp(np.maximum(x, 2.0 ** -126))
    return np.ldexp(1.0, np.maximum(ex - 1, -126) - 7)


# --------------------------------------------------------------------------
# GEMM oracles
# --------------------------------------------------------------------------

def gemm_dequant_fp64(a_dq: np.ndarray, b_dq: np.ndarray) -> np.ndarray:
    """Exact-arithmetic checker: fp64 ``A . B^T`` of already dequantised operands."""
    return np.asarray(a_dq, dtype=np.float64) @ np.asarray(b_dq, dtype=np.float64).T


def gemm_dequant_fp32(a_dq: np.ndarray, b_dq: np.ndarray) -> np.ndarray:
    """The reference's validation recipe (test_amdgpu_gemm.py:27): fp32 operands,
    fp32 matmul, round to bf16.  Returns bf16 bit patterns (uint16)."""
    c = np.asarray(a_dq, dtype=np.float32) @ np.asarray(b_dq, dtype=np.float32).T
    return f32_to_bf16_bits(c)


def gemm_mxfp4_fp64(a, a_scale, b, b_scale) -> np.ndarray:
    return gemm_dequant_fp64(dequantize_mxfp4(a, a_scale, np.float64), dequantize_mxfp4(b, b_scale, np.float64))


def gemm_mxfp4_fp32_bf16(a, a_scale, b, b_scale) -> np.ndarray:
    return gemm_dequant_fp32(dequantize_mxfp4(a, a_scale), dequantize_mxfp4(b, b_scale))


def gemm_nvfp4_fp64(a, a_scale, a_global, b, b_scale, b_global) -> np.ndarray:
    c = gemm_dequant_fp64(dequantize_nvfp4_block(a, a_scale, np.float64), dequantize_nvfp4_block(b, b_scale, np.float64))
    return c * (np.float64(np.float32(a_global)) * np.float64(np.float32(b_global)))


def gemm_nvfp4_fp32_bf16(a, a_scale, a_global, b, b_scale, b_global) -> np.ndarray:
    c = np.asarray(dequantize_nvfp4_block(a, a_scale), dtype=np.float32) @ dequantize_nvfp4_block(b, b_scale).T
    return f32_to_bf16_bits(c * (np.float32(a_global) * np.float32(b_global)))


def grouped_gemm_mxfp4_fp64(a, a_scale, b, b_scale, row_offsets) -> np.ndarray:
    """Expert ``e`` owns rows ``row_offsets[e]:row_offsets[e+1]`` of ``a`` and uses
    weights ``b[e]`` (``[E, N, K/2]``) / ``b_scale[e]``."""
    E, N = b.shape[0], b.shape[1]
    out = np.zeros((a.shape[0], N), dtype=np.float64)
    for e in range(E):
        r0, r1 = int(row_offsets[e]), int(row_offsets[e + 1])
        if r1 > r0:
            out[r0:r1] = gemm_mxfp4_fp64(a[r0:r1], a_scale[r0:r1], b[e], b_scale[e])
    return out


# --------------------------------------------------------------------------
# Tolerance: 1 bf16 ulp + fp32 accumulation-order bound; 2**-7 per row
# --------------------------------------------------------------------------

def check_bf16_against_fp64(c_bits: np.ndarray, ref64: np.ndarray, abs_prod_sum: np.ndarray | None, k: int):
    """Returns (ok, report).  ``c_bits``: uint16 bf16 patterns from the device.

    Element bound: ``|c - ref| <= ulp_bf16(ref) + k * 2**-24 * S`` where ``S`` is
    ``sum_k |a||b|`` (fp64) -- the classical bound for any fp32 summation order; when
    ``abs_prod_sum`` is None only the row bound is applied.
    Row bound: ``max_j |c_ij - ref_ij| <= 2**-7 * max_j |ref_ij|`` for rows whose
    reference is not identically zero; all-zero reference rows must be exactly zero.
    """
    c = bf16_bits_to_f32(c_bits).astype(np.float64)
    err = np.abs(c - ref64)
    rep = {}
    ok = bool(np.isfinite(c).all())
    rowmax = np.abs(ref64).max(axis=1)
    nz = rowmax > 0
    rel = np.zeros_like(rowmax)
    rel[nz] = err[nz].max(axis=1) / rowmax[nz]
    rep["max_row_rel"] = float(rel.max()) if rel.size else 0.0
    ok &= bool((rel <= 2.0 ** -7).all())
    if (~nz).any():
        ok &= bool((c[~nz] == 0).all())
    if abs_prod_sum is not None:
        bound = bf16_ulp(ref64) + k * 2.0 ** -24 * abs_prod_sum
        viol = err > bound
        rep["elem_violations"] = int(viol.sum())
        rep["max_err_over_bound"] = float((err / bound).max()) if err.size else 0.0
        ok &= not bool(viol.any())
    return ok, rep


# --------------------------------------------------------------------------
# Seeded synthetic inputs of the benchmark configurations
# --------------------------------------------------------------------------

def randn(shape, seed: int, std: float = 1.0) -> np.ndarray:
    rng = np.random.Generator(np.random.PCG64(seed))
    return (rng.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(np.float32)


def activations_with_outliers(m: int, k: int, seed: int, frac: float = 0.01, mult: float = 20.0) -> np.ndarray:
    """N(0,1) with ``frac`` of the K channels (seeded choice) scaled by ``mult``."""
    x = randn((m, k), seed)
    rng = np.random.Generator(np.random.PCG64(seed + 7919))
    ch = rng.choice(k, size=max(1, int(round(frac * k))), replace=False)
    x[:, ch] *= np.float32(mult)
    return x


def moe_routing(tokens: int, experts: int, top_k: int, seed: int):
    """Seeded N(0,1) logits -> softmax -> top-k -> stable sort by expert.
    Returns (token index per routed row ``[tokens*top_k]``, row_offsets ``[experts+1]`` int32)."""
    logits = randn((tokens, experts), seed).astype(np.float64)
    p = np.exp(logits - logits.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    top = np.argsort(-p, axis=1, kind="stable")[:, :top_k]            # [tokens, top_k]
    expert_of_row = top.reshape(-1)
    token_of_row = np.repeat(np.arange(tokens), top_k)
    order = np.argsort(expert_of_row, kind="stable")
    counts = np.bincount(expert_of_row, minlength=experts)
    row_offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    return token_of_row[order], row_offsets


# --------------------------------------------------------------------------
# MoE routing and gather (the steps in front of the grouped GEMM)
# --------------------------------------------------------------------------

def route_top2(logits: np.ndarray):
    """Top-2 routing of ``logits`` ``[T, E]``: every token goes to its two highest-scoring experts
    (equal scores: lower expert index first); the ``2T`` routed rows are stably sorted by expert
    (inside an expert by token, then by rank).

    Returns ``(token_of_row int32 [2T], row_offsets int32 [E+1], row_weight float64 [2T])`` where
    ``row_weight`` is the full-softmax probability of the row's expert for its token."""
    logits = np.asarray(logits)
    t, e = logits.shape
    l64 = logits.astype(np.float64)
    top = np.argsort(-l64, axis=1, kind="stable")[:, :2]                  # [T, 2]
    p = np.exp(l64 - l64.max(axis=1, keepdims=True)) if t else l64
    if t:
        p = p / p.sum(axis=1, keepdims=True)
    expert_of_row = top.reshape(-1)
    token_of_row = np.repeat(np.arange(t), 2)
    order = np.argsort(expert_of_row, kind="stable")
    counts = np.bincount(expert_of_row, minlength=e)
    row_offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    tok = token_of_row[order].astype(np.int32)
    weight = p[tok, expert_of_row[order]] if t else np.zeros(0)
    return tok, row_offsets, weight


def rows_of_token(token_of_row: np.ndarray, logits: np.ndarray) -> np.ndarray:
    """Inverse of the routing permutation: ``[T, 2]`` int32, the routed row of every token's first and second
    choice (the order of :func:`route_top2`: higher score first, equal scores: lower expert index first)."""
    logits = np.asarray(logits)
    t, _ = logits.shape
    top = np.argsort(-logits.astype(np.float64), axis=1, kind="stable")[:, :2]
    order = np.argsort(top.reshape(-1), kind="stable")
    inv = np.empty(2 * t, dtype=np.int64)
    inv[order] = np.arange(2 * t)
    assert np.array_equal(np.asarray(token_of_row), (order // 2).astype(np.int32))
    return inv.reshape(t, 2).astype(np.int32)


def combine_top2(rows_bf16_bits: np.ndarray, rows_of_tok: np.ndarray, row_weight: np.ndarray,
                 renormalize: bool = False) -> np.ndarray:
    """``out[t] = w0 * rows[r0] + w1 * rows[r1]`` in float32, one IEEE operation each (two products, one sum),
    then rounded to bf16 (round to nearest even); returns bf16 bit patterns ``uint16 [T, H]``.  With
    ``renormalize`` the two weights are first divided by their float32 sum.  A row index outside the matrix
    contributes zeros."""
    rows = bf16_bits_to_f32(np.asarray(rows_bf16_bits))
    n_rows = rows.shape[0]
    idx = np.asarray(rows_of_tok).astype(np.int64)
    w = np.asarray(row_weight, dtype=np.float32)
    ok = (idx >= 0) & (idx < n_rows)
    safe = np.where(ok, idx, 0)
    w2 = np.where(ok, w[safe], np.float32(0)).astype(np.float32)              # [T, 2]
    if renormalize:
        total = (w2[:, 0] + w2[:, 1]).astype(np.float32)
        with np.errstate(invalid="ignore", divide="ignore"):
            w2 = (w2 / total[:, None]).astype(np.float32)
    x0 = np.where(ok[:, :1], rows[safe[:, 0]], np.float32(0)).astype(np.float32)
    x1 = np.where(ok[:, 1:], rows[safe[:, 1]], np.float32(0)).astype(np.float32)
    p0 = (w2[:, :1] * x0).astype(np.float32)
    p1 = (w2[:, 1:] * x1).astype(np.float32)
    return f64_to_bf16_bits((p0 + p1).astype(np.float32).astype(np.float64))


def gather_rows(a: np.ndarray, a_scale: np.ndarray, index: np.ndarray):
    """``out[i] = a[index[i]]`` (and the same for the scale rows); an index outside ``[0, rows)``
    gives a row of zero bytes."""
    index = np.asarray(index).astype(np.int64)
    ok = (index >= 0) & (index < a.shape[0])
    safe = np.where(ok, index, 0)
    out = np.where(ok[:, None], a[safe], 0).astype(a.dtype) if a.shape[0] else np.zeros((len(index), a.shape[1]), a.dtype)
    out_s = (np.where(ok[:, None], a_scale[safe], 0).astype(a_scale.dtype) if a.shape[0]
             else np.zeros((len(index), a_scale.shape[1]), a_scale.dtype))
    return out, out_s


# --------------------------------------------------------------------------
# Blocked scale layout
# --------------------------------------------------------------------------

def scales_to_blocked(scales: np.ndarray) -> np.ndarray:
    """Row-major ``[rows, cols]`` scale bytes -> the 128 x 4 blocked image (flat): pad to multiples of
    128 rows and 4 columns with zeros, cut into 128 x 4 tiles kept in row-major tile order, and store
    each tile as 32 rows of 16 bytes where row ``r % 32`` holds, for ``r // 32`` = 0..3, the four
    scales of tile row ``r``."""
    rows, cols = scales.shape
    rt, ct = (rows + 127) // 128, (cols + 3) // 4
    padded = np.zeros((rt * 128, ct * 4), dtype=scales.dtype)
    padded[:rows, :cols] = scales
    tiles = padded.reshape(rt, 128, ct, 4).transpose(0, 2, 1, 3)        # [rt, ct, 128, 4]
    inner = tiles.reshape(rt, ct, 4, 32, 4).transpose(0, 1, 3, 2, 4)    # [rt, ct, r%32, r//32, c]
    return np.ascontiguousarray(inner).reshape(-1)


def scales_from_blocked(blocked: np.ndarray, rows: int, cols: int) -> np.ndarray:
    rt, ct = (rows + 127) // 128, (cols + 3) // 4
    inner = np.asarray(blocked).reshape(rt, ct, 32, 4, 4).transpose(0, 1, 3, 2, 4)   # [rt, ct, r//32, r%32, c]
    padded = inner.reshape(rt, ct, 128, 4).transpose(0, 2, 1, 3).reshape(rt * 128, ct * 4)
    return np.ascontiguousarray(padded[:rows, :cols])


# --------------------------------------------------------------------------
# SwiGLU-fused gate+up GEMM
# --------------------------------------------------------------------------

def silu64(x: np.ndarray) -> np.ndarray:
    x = np.asarray(x, dtype=np.float64)
    return x / (1.0 + np.exp(-x))


def gemm_mxfp4_swiglu_fp64(a, a_scale, b, b_scale):
    """``b`` holds N gate rows followed by N up rows.  Returns ``(h, gate, up)`` in float64 with
    ``h = silu(gate) * up``, ``gate = A . B[:N]^T``, ``up = A . B[N:]^T``."""
    n = b.shape[0] // 2
    gate = gemm_mxfp4_fp64(a, a_scale, b[:n], b_scale[:n])
    up = gemm_mxfp4_fp64(a, a_scale, b[n:], b_scale[n:])
    return silu64(gate) * up, gate, up


def check_swiglu_bf16(c_bits, a, a_scale, b, b_scale):
    """bf16 result of the fused GEMM against exact arithmetic.  Stated tolerance per element:
    one bf16 ulp of the exact value, plus the fp32 accumulation bound ``K * 2^-24 * sum|a||b|`` of each
    projection pushed through the product (``d silu/dx <= 1.1``), plus ``2^-20 |h|`` for the fp32
    evaluation of exp, the division and the multiply."""
    n = b.shape[0] // 2
    k = a.shape[1] * 2
    h, gate, up = gemm_mxfp4_swiglu_fp64(a, a_scale, b, b_scale)
    adq = np.abs(dequantize_mxfp4(a, a_scale, np.float64))
    bdq = np.abs(dequantize_mxfp4(b, b_scale, np.float64))
    eg = k * 2.0 ** -24 * (adq @ bdq[:n].T)
    eu = k * 2.0 ** -24 * (adq @ bdq[n:].T)
    bound = bf16_ulp(h) + 1.1 * np.abs(up) * eg + np.abs(silu64(gate)) * eu + 1.1 * eg * eu + 2.0 ** -20 * np.abs(h)
    got = bf16_bits_to_f32(np.asarray(c_bits)).astype(np.float64)
    err = np.abs(got - h)
    bad = err > bound
    return not bad.any(), {"violations": int(bad.sum()), "max_err_over_bound": float((err / np.maximum(bound, 1e-300)).max())}
