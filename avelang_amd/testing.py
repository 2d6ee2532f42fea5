"""Synthetic-input helpers for the benchmark and the tests (the reference keeps its test
helpers in ``python/avelang/testing.py``).  Nothing here is on the GEMM path: these are the
quantisers that turn seeded fp32 tensors into the packed operands the kernels consume,
written with torch ops so they run where the data lives (GPU or CPU).

They implement the same recipe as the CPU oracle's quantisers and are tested against them.
"""
from __future__ import annotations

import torch

E2M1_MAX = 6.0
E4M3_MAX = 448.0


def has_rocm() -> bool:
    """Same gate as the reference's ``avelang.testing.has_rocm`` (python/avelang/testing.py:21-26)."""
    return torch.cuda.is_available() and getattr(torch.version, "hip", None) is not None


def _e2m1_codes(q: torch.Tensor) -> torch.Tensor:
    """Round-to-nearest-even onto {0,.5,1,1.5,2,3,4,6}, saturating; returns uint8 codes with
    the sign in bit 3.  Ties go to the even code: 0.25->0, 0.75->1, 1.25->1, 1.75->2, 2.5->2,
    3.5->4, 5->4."""
    a = q.abs()
    idx = ((a > 0.25).to(torch.uint8) + (a >= 0.75).to(torch.uint8) + (a > 1.25).to(torch.uint8)
           + (a >= 1.75).to(torch.uint8) + (a > 2.5).to(torch.uint8) + (a >= 3.5).to(torch.uint8)
           + (a > 5.0).to(torch.uint8))
    return idx | (torch.signbit(q).to(torch.uint8) << 3)


def _pack(codes: torch.Tensor) -> torch.Tensor:
    return (codes[..., 0::2] | (codes[..., 1::2] << 4)).contiguous()


def quantize_mxfp4(x: torch.Tensor):
    """fp32 ``[R, K]`` -> (packed uint8 ``[R, K/2]``, E8M0 uint8 ``[R, K/32]``)."""
    r, k = x.shape
    xb = x.float().reshape(r, k // 32, 32)
    amax = xb.abs().amax(dim=-1)
    _, ex = torch.frexp(amax)                       # amax = m * 2**ex, m in [0.5, 1)
    e = torch.where(amax > 0, ex - 1 - 2, torch.zeros_like(ex)).clamp(-127, 127)
    scale = torch.ldexp(torch.ones_like(amax), e)
    codes = _e2m1_codes(xb / scale[..., None]).reshape(r, k)
    return _pack(codes), (e + 127).to(torch.uint8).contiguous()


def quantize_nvfp4(x: torch.Tensor):
    """fp32 ``[R, K]`` -> (packed ``[R, K/2]``, E4M3 uint8 ``[R, K/16]``, fp32 global scale ``[1]``)."""
    r, k = x.shape
    x = x.float()
    g = (x.abs().amax() / (E4M3_MAX * E2M1_MAX)).reshape(1)
    g = torch.where(g == 0, torch.ones_like(g), g)
    xb = x.reshape(r, k // 16, 16)
    amax = xb.abs().amax(dim=-1)
    # the oracle divides in fp64; do the same so the E4M3 rounding sees identical inputs
    sb = ((amax.double() / E2M1_MAX) / g.double()).to(torch.float32).to(torch.float8_e4m3fn)
    sdec = sb.float().double() * g.double()
    q = torch.where(sdec[..., None] > 0, xb.double() / sdec[..., None], torch.zeros_like(xb, dtype=torch.float64))
    codes = _e2m1_codes(q).reshape(r, k)
    return _pack(codes), sb.view(torch.uint8).contiguous(), g


def activations_with_outliers(m: int, k: int, generator: torch.Generator, device, frac: float = 0.01,
                              mult: float = 20.0) -> torch.Tensor:
    """N(0,1) activations with ``frac`` of the K channels (seeded choice) scaled by ``mult``."""
    x = torch.randn((m, k), generator=generator, device=device, dtype=torch.float32)
    n_out = max(1, int(round(frac * k)))
    ch = torch.randperm(k, generator=generator, device=device)[:n_out]
    x[:, ch] *= mult
    return x


def moe_routing(tokens: int, experts: int, top_k: int, generator: torch.Generator, device):
    """Seeded N(0,1) logits -> softmax -> top-k -> stable sort by expert.
    Returns (token index of every routed row, int32 row_offsets ``[experts+1]``)."""
    logits = torch.randn((tokens, experts), generator=generator, device=device, dtype=torch.float32)
    top = torch.softmax(logits, dim=-1).topk(top_k, dim=-1).indices.reshape(-1)
    token = torch.arange(tokens, device=device).repeat_interleave(top_k)
    order = torch.sort(top, stable=True).indices
    counts = torch.bincount(top, minlength=experts)
    row_offsets = torch.cat([torch.zeros(1, dtype=torch.int64, device=device), counts.cumsum(0)]).to(torch.int32)
    return token[order], row_offsets
