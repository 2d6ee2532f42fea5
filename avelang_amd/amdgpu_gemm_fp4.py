"""Host entry points of the block-scaled FP4 GEMM, mirroring the reference's
``avelang_kernels.amdgpu_gemm.gemm_pipeline_transposed_b``
(reference ``python/avelang_kernels/amdgpu_gemm.py:458-494``):

* ``C[M, N] (bf16) = A[M, K] . B[N, K]^T`` with ``B`` stored ``[N, K]``;
* operands are validated with ``ValueError`` before anything is launched;
* ``out=None`` allocates ``torch.empty((M, N), bfloat16, device=A.device)``, otherwise
  ``out`` is checked for shape, dtype and device and written in place; ``out`` is returned;
* the launch is asynchronous on torch's current stream of ``A``'s device and performs no
  allocation or synchronisation, so it can be captured in a graph (the reference benchmark
  relies on that, ``benchmark/gemm/bench_amdgpu_gemm.py:37-41``).

What differs from the bf16 reference: ``A``/``B`` hold packed E2M1 codes (two per byte,
low nibble = even k) and each comes with a block-scale tensor; the reference's
``M % 128 == N % 128 == 0`` restriction is dropped.
"""
from __future__ import annotations

import torch

from . import _lib

GROUP_K_MXFP4 = 32  # K elements per E8M0 scale
GROUP_K_NVFP4 = 16  # K elements per E4M3 scale

_BYTE_DTYPES = {torch.uint8}
for _name in ("float4_e2m1fn_x2", "float8_e8m0fnu", "float8_e4m3fn"):
    if hasattr(torch, _name):
        _BYTE_DTYPES.add(getattr(torch, _name))


def _as_bytes(t: torch.Tensor, name: str) -> torch.Tensor:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor, got {type(t).__name__}.")
    if t.dtype not in _BYTE_DTYPES:
        raise ValueError(f"{name} must have dtype torch.uint8 (or a 1-byte FP4/FP8 dtype), got {t.dtype}.")
    if t.dtype != torch.uint8:
        t = t.view(torch.uint8)
    return t


def _check_matrix(t: torch.Tensor, name: str, shape, device) -> None:
    if tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}.")
    if t.device != device:
        raise ValueError(f"{name} must be on device {device}, got {t.device}.")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous (row-major).")


def _prepare_out(out, out_shape, device):
    if out is None:
        return torch.empty(out_shape, dtype=torch.bfloat16, device=device)
    if tuple(out.shape) != tuple(out_shape):
        raise ValueError(f"out must have shape {tuple(out_shape)}, got {tuple(out.shape)}.")
    if out.dtype != torch.bfloat16:
        raise ValueError(f"out must have dtype torch.bfloat16, got {out.dtype}.")
    if out.device != device:
        raise ValueError(f"out must be on device {device}, got {out.device}.")
    if not out.is_contiguous():
        raise ValueError("out must be contiguous (row-major).")
    return out


def _require_gpu(t: torch.Tensor) -> None:
    if t.device.type != "cuda":
        raise ValueError(f"A must be on a ROCm GPU device, got {t.device}.")


def _stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _gemm_operands(A, A_scale, B, B_scale, group_k, *, grouped=False, gate_up=False, row_offsets=None, quantised_out=False):
    """The checks every GEMM wrapper makes before anything is launched (the reference's ``ValueError`` block,
    ``python/avelang_kernels/amdgpu_gemm.py:463-486``): byte views of the operands, dimensions, ``K`` against the scale
    block, device, shapes, contiguity.  ``grouped``: ``B`` is ``[E, rows, K/2]`` and ``row_offsets`` int32 ``[E+1]``;
    ``gate_up``: the rows of ``B`` (of every expert) are ``N`` gate rows followed by ``N`` up rows;
    ``quantised_out``: the result is quantised per 32 outputs, so ``N`` must be a multiple of 32.
    Returns ``(A, A_scale, B, B_scale, m, n, k, e, device)`` with ``e = 0`` for a plain GEMM."""
    A = _as_bytes(A, "A")
    B = _as_bytes(B, "B")
    A_scale = _as_bytes(A_scale, "A_scale")
    B_scale = _as_bytes(B_scale, "B_scale")
    if grouped:
        if A.dim() != 2 or B.dim() != 3:
            raise ValueError(f"A must be 2-D and B 3-D, got {A.dim()}-D and {B.dim()}-D.")
    elif A.dim() != 2 or B.dim() != 2:
        raise ValueError(f"A and B must be 2-D, got {A.dim()}-D and {B.dim()}-D.")
    m, k = A.shape[0], A.shape[1] * 2
    e = B.shape[0] if grouped else 0
    b_rows = B.shape[1] if grouped else B.shape[0]
    if gate_up and b_rows % 2 != 0:
        who = "every expert of B" if grouped else "B"
        raise ValueError(f"{who} must hold gate rows followed by as many up rows, got {b_rows} rows.")
    n = b_rows // 2 if gate_up else b_rows
    if k % group_k != 0 or k == 0:
        raise ValueError(f"K must be a multiple of {group_k}, got {k}.")
    if quantised_out and n % GROUP_K_MXFP4 != 0:
        raise ValueError(f"N must be a multiple of {GROUP_K_MXFP4} (whole scale blocks per row), got {n}.")
    _require_gpu(A)
    dev = A.device
    lead = (e,) if grouped else ()
    _check_matrix(A, "A", (m, k // 2), dev)
    _check_matrix(B, "B", lead + (b_rows, k // 2), dev)
    _check_matrix(A_scale, "A_scale", (m, k // group_k), dev)
    _check_matrix(B_scale, "B_scale", lead + (b_rows, k // group_k), dev)
    if grouped:
        if not isinstance(row_offsets, torch.Tensor) or row_offsets.dtype != torch.int32:
            raise ValueError("row_offsets must be a torch.int32 tensor.")
        _check_matrix(row_offsets, "row_offsets", (e + 1,), dev)
    return A, A_scale, B, B_scale, m, n, k, e, dev


def _padded_columns(n, n_pad, what):
    """``n_pad`` checked against ``n`` (``None``: no padding)."""
    if n_pad is None:
        return n
    if not isinstance(n_pad, int) or n_pad < n or n_pad % GROUP_K_MXFP4 != 0:
        raise ValueError(f"{what} must be a multiple of {GROUP_K_MXFP4} and at least {n}, got {n_pad}.")
    return n_pad


def _quantised_outputs(out, out_scale, m, n, dev, n_pad=None):
    """``(codes [m, n_pad/2], scales [m, n_pad/32])`` of the fused quantiser: checked when given, allocated when not
    (zero-filled when padded: the kernels leave the columns from ``n`` on alone)."""
    n_pad = _padded_columns(n, n_pad, "n_pad")
    alloc = torch.zeros if n_pad != n else torch.empty
    if out is None:
        out = alloc((m, n_pad // 2), dtype=torch.uint8, device=dev)
    if out_scale is None:
        out_scale = alloc((m, n_pad // GROUP_K_MXFP4), dtype=torch.uint8, device=dev)
    _check_matrix(_as_bytes(out, "out"), "out", (m, n_pad // 2), dev)
    _check_matrix(_as_bytes(out_scale, "out_scale"), "out_scale", (m, n_pad // GROUP_K_MXFP4), dev)
    return out, out_scale, n_pad


def gemm_mxfp4_transposed_b(A, A_scale, B, B_scale, out=None, *, variant: int = _lib.AUTO, split_k: bool = True, lib=None):
    """MXFP4 GEMM. ``A`` ``[M, K/2]`` and ``B`` ``[N, K/2]`` packed E2M1; ``A_scale``
    ``[M, K/32]`` and ``B_scale`` ``[N, K/32]`` E8M0 bytes. Returns bf16 ``[M, N]``.
    ``split_k=False`` keeps every shape on the one-launch kernels (bit-identical to ``ave_fp4_gemm_mxfp4``).
    ``lib``: the binding to call through -- the ctypes binding of ``libave_fp4.so`` unless given (the pybind11
    extension built from ``python/src`` offers the same functions)."""
    A, A_scale, B, B_scale, m, n, k, _, dev = _gemm_operands(A, A_scale, B, B_scale, GROUP_K_MXFP4)
    out = _prepare_out(out, (m, n), dev)
    lib = lib or _lib.load()
    with torch.cuda.device(dev):
        # shapes with few output tiles and a long K are split along K through a workspace from torch's allocator
        # (stream-ordered like `out`, and part of the graph's pool under capture); the library never allocates
        ws_bytes = lib.ave_fp4_gemm_mxfp4_workspace_bytes(m, n, k) if int(variant) == _lib.AUTO and split_k else 0
        if ws_bytes:
            workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
            rc = lib.ave_fp4_gemm_mxfp4_ws(
                A.data_ptr(), A_scale.data_ptr(), B.data_ptr(), B_scale.data_ptr(), out.data_ptr(),
                m, n, k, workspace.data_ptr(), ws_bytes, _stream_ptr(dev),
            )
        else:
            rc = lib.ave_fp4_gemm_mxfp4_ex(
                A.data_ptr(), A_scale.data_ptr(), B.data_ptr(), B_scale.data_ptr(), out.data_ptr(),
                m, n, k, _stream_ptr(dev), int(variant),
            )
    _lib.check(rc)
    return out


def gemm_mxfp4_blocked_scales_transposed_b(A, A_scale_blocked, B, B_scale_blocked, out=None, *, lib=None):
    """MXFP4 GEMM on scale tensors in the 128 x 4 blocked layout (what :func:`avelang_amd.scales_to_blocked` writes and
    other FP4 stacks' quantisers emit), read by the kernels as they are.  ``A_scale_blocked`` and ``B_scale_blocked`` are
    flat uint8 tensors of ``ceil(rows / 128) * 128 * K / 32`` bytes; ``K`` must be a multiple of 512 (``ValueError``
    otherwise: convert with :func:`avelang_amd.scales_from_blocked`).  Bit-identical to
    :func:`gemm_mxfp4_transposed_b` on the row-major scales with ``variant`` DECODE (up to 64 rows) or TILE."""
    A = _as_bytes(A, "A")
    B = _as_bytes(B, "B")
    A_scale_blocked = _as_bytes(A_scale_blocked, "A_scale_blocked")
    B_scale_blocked = _as_bytes(B_scale_blocked, "B_scale_blocked")
    if A.dim() != 2 or B.dim() != 2:
        raise ValueError(f"A and B must be 2-D, got {A.dim()}-D and {B.dim()}-D.")
    m, k, n = A.shape[0], A.shape[1] * 2, B.shape[0]
    if k % GROUP_K_MXFP4 != 0 or k == 0:
        raise ValueError(f"K must be a multiple of {GROUP_K_MXFP4}, got {k}.")
    _require_gpu(A)
    dev = A.device
    _check_matrix(A, "A", (m, k // 2), dev)
    _check_matrix(B, "B", (n, k // 2), dev)
    for name, t, rows in (("A_scale_blocked", A_scale_blocked, m), ("B_scale_blocked", B_scale_blocked, n)):
        want = -(-rows // 128) * 128 * (-(-(k // GROUP_K_MXFP4) // 4) * 4)
        _check_matrix(t.reshape(-1) if t.is_contiguous() else t, name, (want,), dev)
    out = _prepare_out(out, (m, n), dev)
    with torch.cuda.device(dev):
        rc = (lib or _lib.load()).ave_fp4_gemm_mxfp4_blocked_scales(A.data_ptr(), A_scale_blocked.data_ptr(), B.data_ptr(),
                                                                    B_scale_blocked.data_ptr(), out.data_ptr(), m, n, k, _stream_ptr(dev))
    _lib.check(rc)
    return out


def gemm_mxfp4_swiglu_transposed_b(A, A_scale, B, B_scale, out=None, *, variant: int = _lib.AUTO):
    """MXFP4 gate+up GEMM with SwiGLU fused: ``B`` ``[2N, K/2]`` holds the ``N`` gate rows followed by the
    ``N`` up rows (``B_scale`` ``[2N, K/32]`` likewise); returns bf16 ``[M, N]`` with
    ``out[m, n] = silu(A[m] . B[n]) * (A[m] . B[N + n])``, evaluated in fp32."""
    A, A_scale, B, B_scale, m, n, k, _, dev = _gemm_operands(A, A_scale, B, B_scale, GROUP_K_MXFP4, gate_up=True)
    out = _prepare_out(out, (m, n), dev)
    lib = _lib.load()
    with torch.cuda.device(dev):
        rc = lib.ave_fp4_gemm_mxfp4_swiglu_ex(
            A.data_ptr(), A_scale.data_ptr(), B.data_ptr(), B_scale.data_ptr(), out.data_ptr(),
            m, n, k, _stream_ptr(dev), int(variant),
        )
    _lib.check(rc)
    return out


def gemm_mxfp4_swiglu_quant_transposed_b(A, A_scale, B, B_scale, out=None, out_scale=None, *, n_pad=None):
    """Gate+up GEMM, SwiGLU and the MXFP4 quantiser of the next GEMM's activations in one launch: returns
    ``(codes, scales)``, uint8 ``[M, N/2]`` and ``[M, N/32]``, bit-identical to
    ``quantize_mxfp4`` applied to the bf16 result of :func:`gemm_mxfp4_swiglu_transposed_b`.  ``N % 32 == 0``;
    needs ``K`` to be a multiple of 32 from 512 up (the LDS-staged kernels; multiples of 512 are fastest) and raises
    ``ValueError`` otherwise.  ``n_pad`` (a multiple of 32, at least N): the rows of both results are laid out for
    ``n_pad`` columns, for a consumer that runs over a padded K (see :func:`quantize_mxfp4`); the columns from N on are
    not written -- tensors allocated here are zero-filled, tensors passed in must hold zero bytes there."""
    A, A_scale, B, B_scale, m, n, k, _, dev = _gemm_operands(A, A_scale, B, B_scale, GROUP_K_MXFP4, gate_up=True,
                                                             quantised_out=True)
    out, out_scale, n_pad = _quantised_outputs(out, out_scale, m, n, dev, n_pad)
    if m == 0 or n == 0:
        return out, out_scale
    lib = _lib.load()
    with torch.cuda.device(dev):
        rc = lib.ave_fp4_gemm_mxfp4_swiglu_quant_padded(
            A.data_ptr(), A_scale.data_ptr(), B.data_ptr(), B_scale.data_ptr(), out.data_ptr(), out_scale.data_ptr(),
            m, n, n_pad, k, _stream_ptr(dev),
        )
    _lib.check(rc)
    return out, out_scale


def gemm_nvfp4_transposed_b(A, A_scale, A_global, B, B_scale, B_global, out=None, *, variant: int = _lib.AUTO,
                            split_k: bool = True, lib=None):
    """NVFP4 GEMM. Scales are E4M3 bytes per 16 k (``[M, K/16]``, ``[N, K/16]``);
    ``A_global`` / ``B_global`` are one-element fp32 tensors on the same device."""
    A, A_scale, B, B_scale, m, n, k, _, dev = _gemm_operands(A, A_scale, B, B_scale, GROUP_K_NVFP4)
    for name, g in (("A_global", A_global), ("B_global", B_global)):
        if not isinstance(g, torch.Tensor) or g.dtype != torch.float32 or g.numel() != 1:
            raise ValueError(f"{name} must be a one-element torch.float32 tensor.")
        if g.device != dev:
            raise ValueError(f"{name} must be on device {dev}, got {g.device}.")
    out = _prepare_out(out, (m, n), dev)
    lib = lib or _lib.load()
    with torch.cuda.device(dev):
        # few output tiles over a long K: split along K through a workspace from torch's allocator (see gemm_mxfp4_transposed_b)
        ws_bytes = lib.ave_fp4_gemm_nvfp4_workspace_bytes(m, n, k) if int(variant) == _lib.AUTO and split_k else 0
        if ws_bytes:
            workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
            rc = lib.ave_fp4_gemm_nvfp4_ws(
                A.data_ptr(), A_scale.data_ptr(), A_global.data_ptr(), B.data_ptr(), B_scale.data_ptr(),
                B_global.data_ptr(), out.data_ptr(), m, n, k, workspace.data_ptr(), ws_bytes, _stream_ptr(dev),
            )
        else:
            rc = lib.ave_fp4_gemm_nvfp4_ex(
                A.data_ptr(), A_scale.data_ptr(), A_global.data_ptr(), B.data_ptr(), B_scale.data_ptr(),
                B_global.data_ptr(), out.data_ptr(), m, n, k, _stream_ptr(dev), int(variant),
            )
    _lib.check(rc)
    return out


def grouped_gemm_mxfp4_transposed_b(A, A_scale, B, B_scale, row_offsets, out=None, *, variant: int = _lib.AUTO, lib=None):
    """Grouped (MoE) MXFP4 GEMM in one launch. ``A`` ``[total_M, K/2]`` holds the rows of
    all experts back to back; ``B`` ``[E, N, K/2]``; ``row_offsets`` int32 ``[E+1]`` on the
    device (rows ``row_offsets[e]:row_offsets[e+1]`` use ``B[e]``). Returns bf16 ``[total_M, N]``."""
    A, A_scale, B, B_scale, m, n, k, e, dev = _gemm_operands(A, A_scale, B, B_scale, GROUP_K_MXFP4, grouped=True,
                                                             row_offsets=row_offsets)
    out = _prepare_out(out, (m, n), dev)
    lib = lib or _lib.load()
    with torch.cuda.device(dev):
        rc = lib.ave_fp4_grouped_gemm_mxfp4_ex(
            A.data_ptr(), A_scale.data_ptr(), B.data_ptr(), B_scale.data_ptr(), row_offsets.data_ptr(),
            out.data_ptr(), m, e, n, k, _stream_ptr(dev), int(variant),
        )
    _lib.check(rc)
    return out


def grouped_gemm_mxfp4_swiglu_transposed_b(A, A_scale, B, B_scale, row_offsets, out=None):
    """Grouped (MoE) gate+up GEMM with SwiGLU in one launch: ``B`` ``[E, 2N, K/2]`` holds, per expert, the ``N`` gate
    rows followed by the ``N`` up rows; rows ``row_offsets[e]:row_offsets[e+1]`` of ``A`` use ``B[e]``.  Returns bf16
    ``[total_M, N]``, every expert's rows equal to :func:`gemm_mxfp4_swiglu_transposed_b` on that expert alone."""
    A, A_scale, B, B_scale, m, n, k, e, dev = _gemm_operands(A, A_scale, B, B_scale, GROUP_K_MXFP4, grouped=True,
                                                             gate_up=True, row_offsets=row_offsets)
    out = _prepare_out(out, (m, n), dev)
    lib = _lib.load()
    with torch.cuda.device(dev):
        rc = lib.ave_fp4_grouped_gemm_mxfp4_swiglu(
            A.data_ptr(), A_scale.data_ptr(), B.data_ptr(), B_scale.data_ptr(), row_offsets.data_ptr(),
            out.data_ptr(), m, e, n, k, _stream_ptr(dev),
        )
    _lib.check(rc)
    return out


def grouped_gemm_mxfp4_swiglu_quant_transposed_b(A, A_scale, B, B_scale, row_offsets, out=None, out_scale=None, *,
                                                 n_pad=None):
    """:func:`grouped_gemm_mxfp4_swiglu_transposed_b` with the MXFP4 quantiser of the down projection's input fused
    behind it: returns ``(codes [total_M, N/2], scales [total_M, N/32])``, bit-identical to ``quantize_mxfp4`` of the
    bf16 result.  ``N % 32 == 0``; needs ``K`` to be a multiple of 32 from 512 up and raises ``ValueError`` otherwise.
    ``n_pad``: as in :func:`gemm_mxfp4_swiglu_quant_transposed_b`."""
    A, A_scale, B, B_scale, m, n, k, e, dev = _gemm_operands(A, A_scale, B, B_scale, GROUP_K_MXFP4, grouped=True,
                                                             gate_up=True, row_offsets=row_offsets, quantised_out=True)
    out, out_scale, n_pad = _quantised_outputs(out, out_scale, m, n, dev, n_pad)
    if m == 0 or n == 0:
        return out, out_scale
    lib = _lib.load()
    with torch.cuda.device(dev):
        rc = lib.ave_fp4_grouped_gemm_mxfp4_swiglu_quant_padded(
            A.data_ptr(), A_scale.data_ptr(), B.data_ptr(), B_scale.data_ptr(), row_offsets.data_ptr(),
            out.data_ptr(), out_scale.data_ptr(), m, e, n, n_pad, k, _stream_ptr(dev),
        )
    _lib.check(rc)
    return out, out_scale


def _quantiser_operands(x, group_k, packed, scales, k_pad=None):
    """Checks shared by the two quantiser wrappers; returns ``(rows, k, device, packed, scales)``; the results are laid
    out for ``k_pad`` columns when that is given."""
    if not isinstance(x, torch.Tensor):
        raise TypeError(f"x must be a torch.Tensor, got {type(x).__name__}.")
    if x.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError(f"x must have dtype torch.float32 or torch.bfloat16, got {x.dtype}.")
    if x.dim() != 2:
        raise ValueError(f"x must be 2-D, got {x.dim()}-D.")
    r, k = x.shape
    if k % group_k != 0 or k == 0:
        raise ValueError(f"K must be a multiple of {group_k}, got {k}.")
    if x.device.type != "cuda":
        raise ValueError(f"x must be on a ROCm GPU device, got {x.device}.")
    if not x.is_contiguous():
        raise ValueError("x must be contiguous (row-major).")
    dev = x.device
    kp = k if k_pad is None else k_pad
    if packed is None:
        packed = torch.empty((r, kp // 2), dtype=torch.uint8, device=dev)
    if scales is None:
        scales = torch.empty((r, kp // group_k), dtype=torch.uint8, device=dev)
    if packed.dtype != torch.uint8 or scales.dtype != torch.uint8:
        raise ValueError("packed and scales must have dtype torch.uint8.")
    _check_matrix(packed, "packed", (r, kp // 2), dev)
    _check_matrix(scales, "scales", (r, kp // group_k), dev)
    return r, k, dev, packed, scales


def quantize_mxfp4(x, packed=None, scales=None, *, k_pad=None):
    """Quantise ``x`` ``[R, K]`` (fp32 or bf16, contiguous, on the GPU) to MXFP4 on the device: returns
    ``(packed uint8 [R, K/2], scales uint8 [R, K/32])`` in the layout :func:`gemm_mxfp4_transposed_b`
    takes.  ``packed`` / ``scales`` may be passed to write in place (same ``out=`` convention).  A block that holds
    an infinity or a NaN gets scale byte 0xFF (the E8M0 NaN) and zero codes.

    ``k_pad`` (a multiple of 32, at least K): the results are ``[R, k_pad/2]`` and ``[R, k_pad/32]``, the columns from K
    on written as zero blocks.  A GEMM over ``k_pad`` with weights padded the same way (:func:`pad_k_mxfp4`) gives the
    same sums, and the tuned kernels run faster on a K that is a multiple of 512 than on one whose packed rows are no
    multiple of 128 bytes (2880 -> 3072: 14 % less time at 8192 x 2880 x 2880)."""
    if k_pad is not None and isinstance(x, torch.Tensor) and x.dim() == 2:
        k_pad = _padded_columns(x.shape[1], k_pad, "k_pad")
    r, k, dev, packed, scales = _quantiser_operands(x, GROUP_K_MXFP4, packed, scales, k_pad)
    lib = _lib.load()
    fn = lib.ave_fp4_quantize_mxfp4_bf16_padded if x.dtype == torch.bfloat16 else lib.ave_fp4_quantize_mxfp4_f32_padded
    with torch.cuda.device(dev):
        rc = fn(x.data_ptr(), packed.data_ptr(), scales.data_ptr(), r, k, k if k_pad is None else k_pad, _stream_ptr(dev))
    _lib.check(rc)
    return packed, scales


def pad_k_mxfp4(packed, scales, k_pad):
    """Pads MXFP4 operands (``packed [..., R, K/2]``, ``scales [..., R, K/32]``, e.g. weights, once, when they are loaded)
    with zero blocks to ``k_pad`` columns: zero codes under the scale byte 127.  Plain torch ops on whatever device the
    tensors are on; returns new contiguous tensors (the arguments themselves when ``k_pad == K``)."""
    k = scales.shape[-1] * GROUP_K_MXFP4
    if packed.shape[-1] * 2 != k:
        raise ValueError(f"packed has {packed.shape[-1]} bytes per row and scales {scales.shape[-1]}: not the same K.")
    k_pad = _padded_columns(k, k_pad, "k_pad")
    if k_pad == k:
        return packed, scales
    pb, sb = _as_bytes(packed, "packed"), _as_bytes(scales, "scales")
    return (torch.nn.functional.pad(pb, (0, (k_pad - k) // 2), value=0).contiguous(),
            torch.nn.functional.pad(sb, (0, (k_pad - k) // GROUP_K_MXFP4), value=127).contiguous())


def quantize_nvfp4(x, global_scale, packed=None, scales=None):
    """Quantise ``x`` ``[R, K]`` (fp32 or bf16, contiguous, on the GPU) to NVFP4 on the device for a given
    per-tensor scale ``global_scale`` (fp32 tensor with one positive element, on the same device; calibrated by
    the caller, e.g. ``amax / (448 * 6)``): returns ``(packed uint8 [R, K/2], scales uint8 [R, K/16])`` in the
    layout :func:`gemm_nvfp4_transposed_b` takes together with the same ``global_scale``.  A block that holds an
    infinity or a NaN gets scale byte 0x7F (the E4M3 NaN) and zero codes."""
    r, k, dev, packed, scales = _quantiser_operands(x, GROUP_K_NVFP4, packed, scales)
    if not isinstance(global_scale, torch.Tensor) or global_scale.dtype != torch.float32 or global_scale.numel() != 1:
        raise ValueError("global_scale must be a torch.float32 tensor with one element.")
    if global_scale.device != dev:
        raise ValueError(f"global_scale must be on {dev}, got {global_scale.device}.")
    lib = _lib.load()
    fn = lib.ave_fp4_quantize_nvfp4_bf16 if x.dtype == torch.bfloat16 else lib.ave_fp4_quantize_nvfp4_f32
    with torch.cuda.device(dev):
        rc = fn(x.data_ptr(), global_scale.data_ptr(), packed.data_ptr(), scales.data_ptr(), r, k, _stream_ptr(dev))
    _lib.check(rc)
    return packed, scales
