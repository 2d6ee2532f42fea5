"""Host entry points of the two steps in front of the grouped (MoE) GEMM: top-2 routing and the row
gather that builds its ``A`` operand.  Same conventions as :mod:`avelang_amd.amdgpu_gemm_fp4`
(reference ``python/avelang_kernels/amdgpu_gemm.py:458-494``): ``ValueError`` before anything is
launched, asynchronous launch on torch's current stream, optional preallocated outputs, no
synchronisation, so that routing, gather and :func:`grouped_gemm_mxfp4_transposed_b` can be captured
in one graph.  The reference has no MoE code; these are additions."""
from __future__ import annotations

import torch

from . import _lib
from .amdgpu_gemm_fp4 import GROUP_K_MXFP4, _as_bytes, _check_matrix, _stream_ptr

MAX_EXPERTS = 256


def _out_tensor(t, name, shape, dtype, device):
    if t is None:
        return torch.empty(shape, dtype=dtype, device=device)
    if t.dtype != dtype:
        raise ValueError(f"{name} must have dtype {dtype}, got {t.dtype}.")
    _check_matrix(t, name, shape, device)
    return t


def moe_route_top2(logits, token_of_row=None, row_offsets=None, row_weight=None, rows_of_token=None):
    """Route every token to its two highest-scoring experts.

    ``logits`` ``[T, E]`` fp32 on the GPU.  Returns ``(token_of_row int32 [2T], row_offsets int32
    [E+1], row_weight fp32 [2T])``: routed rows sorted by expert (stable: by token, then by rank), the
    offsets :func:`grouped_gemm_mxfp4_transposed_b` takes, and the softmax probability of each row.
    ``rows_of_token`` (int32 ``[T, 2]``, optional) is filled with the inverse map that
    :func:`moe_combine_top2` reads: the routed row of every token's first and second choice."""
    if not isinstance(logits, torch.Tensor):
        raise TypeError(f"logits must be a torch.Tensor, got {type(logits).__name__}.")
    if logits.dtype != torch.float32:
        raise ValueError(f"logits must have dtype torch.float32, got {logits.dtype}.")
    if logits.dim() != 2:
        raise ValueError(f"logits must be 2-D, got {logits.dim()}-D.")
    if logits.device.type != "cuda":
        raise ValueError(f"logits must be on a ROCm GPU device, got {logits.device}.")
    if not logits.is_contiguous():
        raise ValueError("logits must be contiguous (row-major).")
    t, e = logits.shape
    if e < 2 or e > MAX_EXPERTS:
        raise ValueError(f"E must be between 2 and {MAX_EXPERTS}, got {e}.")
    dev = logits.device
    token_of_row = _out_tensor(token_of_row, "token_of_row", (2 * t,), torch.int32, dev)
    row_offsets = _out_tensor(row_offsets, "row_offsets", (e + 1,), torch.int32, dev)
    row_weight = _out_tensor(row_weight, "row_weight", (2 * t,), torch.float32, dev)
    if rows_of_token is not None:
        rows_of_token = _out_tensor(rows_of_token, "rows_of_token", (t, 2), torch.int32, dev)
    lib = _lib.load()
    with torch.cuda.device(dev):
        rc = lib.ave_fp4_moe_route_top2_ex(logits.data_ptr(), t, e, token_of_row.data_ptr(), row_offsets.data_ptr(),
                                           row_weight.data_ptr(),
                                           rows_of_token.data_ptr() if rows_of_token is not None else None,
                                           _stream_ptr(dev))
    _lib.check(rc)
    return token_of_row, row_offsets, row_weight


def moe_combine_top2(rows, rows_of_token, row_weight, out=None, *, renormalize=False):
    """``out[t] = w0 * rows[r0] + w1 * rows[r1]`` with ``(r0, r1) = rows_of_token[t]`` and ``w`` the routing
    probabilities of those rows (divided by their sum when ``renormalize``): the expert outputs back in token
    order.  ``rows`` bf16 ``[2T, H]`` (``H % 8 == 0``), ``rows_of_token`` int32 ``[T, 2]``, ``row_weight`` fp32
    ``[2T]``; returns bf16 ``[T, H]``."""
    if not isinstance(rows, torch.Tensor) or rows.dtype != torch.bfloat16:
        raise ValueError("rows must be a torch.bfloat16 tensor.")
    if rows.dim() != 2 or rows.shape[0] % 2 != 0:
        raise ValueError(f"rows must be 2-D with an even number of rows, got shape {tuple(rows.shape)}.")
    if rows.device.type != "cuda":
        raise ValueError(f"rows must be on a ROCm GPU device, got {rows.device}.")
    if not rows.is_contiguous():
        raise ValueError("rows must be contiguous (row-major).")
    t, h = rows.shape[0] // 2, rows.shape[1]
    if h % 8 != 0 or h == 0:
        raise ValueError(f"H must be a positive multiple of 8, got {h}.")
    dev = rows.device
    if rows_of_token is None or row_weight is None:
        raise ValueError("rows_of_token and row_weight (outputs of moe_route_top2) are required.")
    rows_of_token = _out_tensor(rows_of_token, "rows_of_token", (t, 2), torch.int32, dev)
    row_weight = _out_tensor(row_weight, "row_weight", (2 * t,), torch.float32, dev)
    out = _out_tensor(out, "out", (t, h), torch.bfloat16, dev)
    lib = _lib.load()
    with torch.cuda.device(dev):
        rc = lib.ave_fp4_moe_combine_top2(rows.data_ptr(), rows_of_token.data_ptr(), row_weight.data_ptr(), t, h,
                                          1 if renormalize else 0, out.data_ptr(), _stream_ptr(dev))
    _lib.check(rc)
    return out


def gather_rows_mxfp4(A, A_scale, index, out=None, out_scale=None):
    """``out[i] = A[index[i]]``, ``out_scale[i] = A_scale[index[i]]``: ``A`` ``[R, K/2]`` packed E2M1,
    ``A_scale`` ``[R, K/32]`` E8M0 bytes, ``index`` int32 ``[rows]``.  An index outside ``[0, R)`` gives
    a row of zero bytes.  Returns ``(out uint8 [rows, K/2], out_scale uint8 [rows, K/32])``."""
    A = _as_bytes(A, "A")
    A_scale = _as_bytes(A_scale, "A_scale")
    if A.dim() != 2:
        raise ValueError(f"A must be 2-D, got {A.dim()}-D.")
    r, kb = A.shape
    k = kb * 2
    if k % GROUP_K_MXFP4 != 0 or k == 0:
        raise ValueError(f"K must be a multiple of {GROUP_K_MXFP4}, got {k}.")
    if A.device.type != "cuda":
        raise ValueError(f"A must be on a ROCm GPU device, got {A.device}.")
    dev = A.device
    _check_matrix(A, "A", (r, kb), dev)
    _check_matrix(A_scale, "A_scale", (r, k // GROUP_K_MXFP4), dev)
    if not isinstance(index, torch.Tensor) or index.dtype != torch.int32 or index.dim() != 1:
        raise ValueError("index must be a 1-D torch.int32 tensor.")
    rows = index.shape[0]
    _check_matrix(index, "index", (rows,), dev)
    out = _out_tensor(out, "out", (rows, kb), torch.uint8, dev)
    out_scale = _out_tensor(out_scale, "out_scale", (rows, k // GROUP_K_MXFP4), torch.uint8, dev)
    lib = _lib.load()
    with torch.cuda.device(dev):
        rc = lib.ave_fp4_gather_rows_mxfp4(A.data_ptr(), A_scale.data_ptr(), index.data_ptr(), rows, r, k,
                                           out.data_ptr(), out_scale.data_ptr(), _stream_ptr(dev))
    _lib.check(rc)
    return out, out_scale
