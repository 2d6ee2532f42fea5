"""Scale-layout adapters: row-major ``[rows, cols]`` block scales (what the GEMM entry points take)
to and from the 128 x 4 blocked layout other FP4 stacks store them in.  Conventions as in
:mod:`avelang_amd.amdgpu_gemm_fp4` (reference ``python/avelang_kernels/amdgpu_gemm.py:458-494``):
``ValueError`` before launch, current stream, optional preallocated output."""
from __future__ import annotations

import torch

from . import _lib
from .amdgpu_gemm_fp4 import _as_bytes, _check_matrix, _stream_ptr


def blocked_numel(rows: int, cols: int) -> int:
    """Bytes of the blocked image of a ``[rows, cols]`` scale tensor."""
    return ((rows + 127) // 128) * 128 * ((cols + 3) // 4) * 4


def _gpu_matrix(t, name):
    t = _as_bytes(t, name)
    if t.device.type != "cuda":
        raise ValueError(f"{name} must be on a ROCm GPU device, got {t.device}.")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous (row-major).")
    return t


def scales_to_blocked(scales, out=None):
    """``scales`` uint8 ``[rows, cols]`` -> flat uint8 ``[blocked_numel(rows, cols)]`` (padding zero)."""
    scales = _gpu_matrix(scales, "scales")
    if scales.dim() != 2:
        raise ValueError(f"scales must be 2-D, got {scales.dim()}-D.")
    rows, cols = scales.shape
    dev = scales.device
    n = blocked_numel(rows, cols)
    if out is None:
        out = torch.empty((n,), dtype=torch.uint8, device=dev)
    out = _as_bytes(out, "out")
    _check_matrix(out, "out", (n,), dev)
    with torch.cuda.device(dev):
        rc = _lib.load().ave_fp4_scales_to_blocked(scales.data_ptr(), rows, cols, out.data_ptr(), _stream_ptr(dev))
    _lib.check(rc)
    return out


def scales_from_blocked(blocked, rows: int, cols: int, out=None):
    """Flat blocked image -> uint8 ``[rows, cols]`` row-major scales."""
    blocked = _gpu_matrix(blocked, "blocked")
    dev = blocked.device
    if rows < 0 or cols < 0:
        raise ValueError(f"rows and cols must be non-negative, got {rows} and {cols}.")
    if blocked.numel() != blocked_numel(rows, cols):
        raise ValueError(f"blocked must hold {blocked_numel(rows, cols)} bytes for a {rows} x {cols} scale tensor, "
                         f"got {blocked.numel()}.")
    if out is None:
        out = torch.empty((rows, cols), dtype=torch.uint8, device=dev)
    out = _as_bytes(out, "out")
    _check_matrix(out, "out", (rows, cols), dev)
    with torch.cuda.device(dev):
        rc = _lib.load().ave_fp4_scales_from_blocked(blocked.data_ptr(), rows, cols, out.data_ptr(), _stream_ptr(dev))
    _lib.check(rc)
    return out
