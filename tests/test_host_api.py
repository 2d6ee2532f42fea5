"""Host-side checks that need no GPU: the C-ABI library loads and exports every symbol the
header declares, argument validation (C and Python level), the workgroup->tile map, and the
torch quantisers used to make synthetic inputs."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from avelang_amd import (_lib, blocked_numel, gather_rows_mxfp4, gemm_mxfp4_swiglu_quant_transposed_b,
                         gemm_mxfp4_swiglu_transposed_b, gemm_mxfp4_transposed_b, gemm_nvfp4_transposed_b,
                         grouped_gemm_mxfp4_swiglu_quant_transposed_b, grouped_gemm_mxfp4_swiglu_transposed_b,
                         grouped_gemm_mxfp4_transposed_b, moe_combine_top2, moe_route_top2, quantize_mxfp4,
                         scales_to_blocked)
from avelang_amd import testing as synth
from oracle import fp4_oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols(headers=("ave_fp4.h", "ave_fp4_debug.h")):
    text = "".join(open(os.path.join(ROOT, "include", h)).read() for h in headers)
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ave_fp4_\w+)\s*\(", text)))


def test_product_header_declares_no_diagnostics():
    """A binding written from ave_fp4.h sees entry points only; probes and test hooks are in ave_fp4_debug.h."""
    product, debug = declared_symbols(("ave_fp4.h",)), declared_symbols(("ave_fp4_debug.h",))
    assert product and not [n for n in product if "_debug_" in n]
    assert debug and all("_debug_" in n for n in debug)


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = declared_symbols()
    assert len(names) >= 9
    for name in names:
        assert hasattr(lib, name), name
    assert sorted(_lib.SIGNATURES) == names
    assert lib.ave_fp4_abi_version() == 1


def test_plain_c_caller_links_against_declared_symbols_only():
    """The C program the GPU tests run is built with the library and imports nothing the header lacks."""
    import subprocess
    binary = os.path.join(ROOT, "avelang_amd", "abi_check")
    assert os.path.exists(binary), "run `make -C avelang_amd/csrc`"
    undefined = subprocess.run(["nm", "-D", "--undefined-only", binary], capture_output=True, text=True, check=True).stdout
    used = sorted(set(re.findall(r"\b(ave_fp4_\w+)", undefined)))
    assert used and set(used) <= set(declared_symbols(("ave_fp4.h",))), used   # the product header alone


def test_c_abi_rejects_bad_arguments_before_touching_the_gpu():
    lib = _lib.load()
    one = ctypes.c_void_p(16)
    assert lib.ave_fp4_gemm_mxfp4(one, one, one, one, one, 4, 4, 33, None) == -1
    assert "K must be a positive multiple of 32, got 33" in _lib.last_error()
    assert lib.ave_fp4_gemm_nvfp4(one, one, one, one, one, one, one, 4, 4, 8, None) == -1
    assert "multiple of 16" in _lib.last_error()
    assert lib.ave_fp4_gemm_mxfp4(one, one, one, one, one, -1, 4, 32, None) == -1
    assert lib.ave_fp4_gemm_mxfp4(None, one, one, one, one, 4, 4, 32, None) == -1
    assert "null" in _lib.last_error()
    assert lib.ave_fp4_gemm_mxfp4(ctypes.c_void_p(8), one, one, one, one, 4, 4, 32, None) == -1
    assert "aligned" in _lib.last_error()
    assert lib.ave_fp4_grouped_gemm_mxfp4(one, one, one, one, one, one, 4, 0, 4, 32, None) == -1
    assert lib.ave_fp4_gemm_mxfp4_ex(one, one, one, one, one, 4, 4, 32, None, 99) == -1
    assert lib.ave_fp4_gemm_mxfp4_ex(one, one, one, one, one, 64, 64, 32, None, 2) == -1      # K % 256 for the tile kernel
    assert lib.ave_fp4_gemm_mxfp4_ex(one, one, one, one, one, 17, 64, 256, None, 3) == -1     # M > 16 for decode
    assert lib.ave_fp4_gemm_mxfp4_ex(one, one, one, one, one, 65, 64, 512, None, 3) == -1     # M > 64 for decode
    assert lib.ave_fp4_gemm_mxfp4_swiglu_ex(one, one, one, one, one, 4, 4, 64, None, 3) == -1   # K % 512 for decode
    assert "swiglu decode kernel does not support" in _lib.last_error()
    assert lib.ave_fp4_gemm_mxfp4_swiglu_ex(one, one, one, one, one, 4, 4, 64, None, 2) == -1   # no tile variant
    # blocked scale tensors: whole 512-element units of K only, 16-byte aligned tensors
    assert lib.ave_fp4_gemm_mxfp4_blocked_scales(one, one, one, one, one, 4, 4, 544, None) == -1
    assert "whole 512-element units of K" in _lib.last_error()
    assert lib.ave_fp4_gemm_mxfp4_blocked_scales(one, ctypes.c_void_p(8), one, one, one, 4, 4, 512, None) == -1
    assert "16-byte aligned" in _lib.last_error()
    assert lib.ave_fp4_gemm_mxfp4_blocked_scales(one, one, one, one, one, 0, 4, 512, None) == 0
    # the GEMM with a workspace (K split over idle compute units)
    assert lib.ave_fp4_gemm_mxfp4_ws(one, one, one, one, one, 4, 4, 33, one, 64, None) == -1
    assert lib.ave_fp4_gemm_mxfp4_ws(one, one, one, one, one, 128, 128, 1024, None, 64, None) == -1
    assert "null workspace" in _lib.last_error()
    assert lib.ave_fp4_gemm_mxfp4_ws(one, one, one, one, one, 128, 128, 1024, ctypes.c_void_p(8), 64, None) == -1
    assert "16-byte aligned" in _lib.last_error()
    # the plan depends on the compute units of the current device (none: no split), so the hook that takes the
    # count as an argument is asked; the device-dependent queries can only be a whole number of [M, N] fp32 slices
    sl, per, tiles, ws = ctypes.c_int(), ctypes.c_int(), ctypes.c_int(), ctypes.c_size_t()
    assert lib.ave_fp4_debug_split_plan(128, 4096, 14336, 256, ctypes.byref(sl), ctypes.byref(per), ctypes.byref(tiles),
                                        ctypes.byref(ws)) == 0
    assert sl.value > 1 and ws.value == sl.value * 128 * 4096 * 4
    assert lib.ave_fp4_gemm_mxfp4_workspace_bytes(128, 4096, 14336) % (128 * 4096 * 4) == 0
    assert lib.ave_fp4_gemm_nvfp4_workspace_bytes(128, 4096, 14336) % (128 * 4096 * 4) == 0
    assert lib.ave_fp4_gemm_nvfp4_ws(one, one, one, one, one, one, one, 128, 128, 1024, None, 64, None) == -1
    assert "null workspace" in _lib.last_error()
    assert lib.ave_fp4_gemm_nvfp4_ws(one, one, None, one, one, one, one, 128, 128, 1024, one, 64, None) == -1
    assert lib.ave_fp4_gemm_nvfp4_ex(one, one, one, one, one, one, one, 65, 64, 256, None, 3) == -1     # M > 64 for decode
    assert "nvfp4 decode kernel does not support" in _lib.last_error()
    assert lib.ave_fp4_debug_gemm_mxfp4_splitk(one, one, one, one, one, 128, 128, 768, one, 1 << 20, 1, 0, None) == -1
    assert "K % 512" in _lib.last_error()
    assert lib.ave_fp4_debug_gemm_mxfp4_splitk(one, one, one, one, one, 128, 128, 1024, one, 1 << 20, 3, 1, None) == -1
    assert "slice_pairs must be in 1..2, got 3" in _lib.last_error()
    assert lib.ave_fp4_debug_gemm_mxfp4_splitk(one, one, one, one, one, 128, 128, 1024, one, 2 * 128 * 128 * 4 - 1, 1, 0, None) == -1
    assert "hold 131072 bytes" in _lib.last_error()
    assert lib.ave_fp4_debug_gemm_mxfp4_splitk(one, ctypes.c_void_p(8), one, one, one, 128, 128, 1024, one, 1 << 20, 1, 1, None) == -1
    # the steps either side of the GEMM
    assert lib.ave_fp4_quantize_mxfp4_f32(one, one, one, 4, 48, None) == -1
    assert lib.ave_fp4_quantize_nvfp4_f32(one, one, one, one, 4, 24, None) == -1
    assert "multiple of 16" in _lib.last_error()
    assert lib.ave_fp4_quantize_nvfp4_bf16(one, None, one, one, 4, 32, None) == -1
    assert lib.ave_fp4_quantize_nvfp4_bf16(ctypes.c_void_p(8), one, one, one, 4, 32, None) == -1
    assert "aligned" in _lib.last_error()
    assert lib.ave_fp4_moe_route_top2(one, 4, 1, one, one, one, None) == -1
    assert "E must be between 2 and 256, got 1" in _lib.last_error()
    assert lib.ave_fp4_moe_route_top2(one, 4, 8, one, None, one, None) == -1
    assert lib.ave_fp4_gather_rows_mxfp4(one, one, one, 4, 4, 40, one, one, None) == -1
    assert lib.ave_fp4_gather_rows_mxfp4(one, one, ctypes.c_void_p(2), 4, 4, 64, one, one, None) == -1
    assert lib.ave_fp4_scales_to_blocked(one, -1, 4, one, None) == -1
    assert lib.ave_fp4_scales_from_blocked(ctypes.c_void_p(2), 4, 4, one, None) == -1
    assert "4-byte aligned" in _lib.last_error()
    # SwiGLU with the fused quantiser
    assert lib.ave_fp4_gemm_mxfp4_swiglu_quant(one, one, one, one, one, one, 4, 48, 512, None) == -1
    assert "multiple of 32" in _lib.last_error()
    assert lib.ave_fp4_gemm_mxfp4_swiglu_quant(one, one, one, one, one, None, 4, 64, 512, None) == -1
    assert lib.ave_fp4_gemm_mxfp4_swiglu_quant(one, one, one, one, one, one, 4, 64, 256, None) == -1
    assert "LDS-staged kernels only" in _lib.last_error()
    assert lib.ave_fp4_gemm_mxfp4_swiglu_quant(None, None, None, None, None, None, 0, 64, 512, None) == 0
    assert lib.ave_fp4_grouped_gemm_mxfp4_swiglu(one, one, one, one, one, one, 4, 0, 64, 512, None) == -1
    assert "E must be positive" in _lib.last_error()
    assert lib.ave_fp4_grouped_gemm_mxfp4_swiglu(one, one, one, one, None, one, 4, 2, 64, 512, None) == -1
    assert "row_offsets" in _lib.last_error()
    assert lib.ave_fp4_grouped_gemm_mxfp4_swiglu_quant(one, one, one, one, one, one, one, 4, 2, 48, 512, None) == -1
    assert "multiple of 32" in _lib.last_error()
    assert lib.ave_fp4_grouped_gemm_mxfp4_swiglu_quant(one, one, one, one, one, one, one, 4, 2, 64, 256, None) == -1
    assert "LDS-staged kernels only" in _lib.last_error()
    assert lib.ave_fp4_moe_route_top2_ex(one, 4, 1, one, one, one, one, None) == -1
    assert lib.ave_fp4_moe_combine_top2(one, one, one, 4, 12, 0, one, None) == -1
    assert "multiple of 8" in _lib.last_error()
    assert lib.ave_fp4_moe_combine_top2(one, None, one, 4, 16, 0, one, None) == -1
    assert lib.ave_fp4_moe_combine_top2(ctypes.c_void_p(8), one, one, 4, 16, 0, one, None) == -1
    assert "16-byte aligned" in _lib.last_error()
    assert lib.ave_fp4_moe_combine_top2(None, None, None, 0, 16, 0, None, None) == 0
    # the matrix-core rate probe
    flop = ctypes.c_double()
    assert lib.ave_fp4_debug_mfma_rate(one, 8, 4, 4, one, None, ctypes.byref(flop)) == -1
    assert "at least 16 bytes" in _lib.last_error()
    assert lib.ave_fp4_debug_mfma_rate(one, 64, 0, 4, one, None, ctypes.byref(flop)) == -1
    assert lib.ave_fp4_debug_mfma_rate(one, 64, 4, 4, None, None, ctypes.byref(flop)) == -1
    # empty problems are a no-op
    assert lib.ave_fp4_gemm_mxfp4(None, None, None, None, None, 0, 4, 32, None) == 0
    assert lib.ave_fp4_gather_rows_mxfp4(None, None, None, 0, 4, 64, None, None, None) == 0
    assert lib.ave_fp4_scales_to_blocked(None, 0, 4, None, None) == 0
    assert _lib.last_error() == ""
    with pytest.raises(ValueError):
        _lib.check(-1)


def test_last_error_is_per_thread():
    """ave_fp4_last_error holds the calling thread's text only: a failing call on another thread
    neither shows up here nor clears what this thread was told."""
    import threading

    lib = _lib.load()
    one = ctypes.c_void_p(16)
    assert lib.ave_fp4_gemm_mxfp4(one, one, one, one, one, 4, 4, 33, None) == -1
    mine = _lib.last_error()
    assert "got 33" in mine
    seen = {}

    def other():
        seen["before"] = _lib.last_error()
        seen["rc"] = lib.ave_fp4_gemm_nvfp4(one, one, one, one, one, one, one, 4, 4, 8, None)
        seen["after"] = _lib.last_error()

    t = threading.Thread(target=other)
    t.start()
    t.join()
    assert seen["before"] == "" and seen["rc"] == -1 and "multiple of 16" in seen["after"]
    assert _lib.last_error() == mine


def test_python_wrappers_validate_like_the_reference():
    a = torch.zeros((4, 16), dtype=torch.uint8)
    s = torch.zeros((4, 1), dtype=torch.uint8)
    with pytest.raises(ValueError, match="dtype"):
        gemm_mxfp4_transposed_b(a.float(), s, a, s)
    with pytest.raises(ValueError, match="K must be a multiple of 32, got 24"):
        gemm_mxfp4_transposed_b(a[:, :12], s, a[:, :12], s)
    with pytest.raises(ValueError, match="ROCm GPU"):
        gemm_mxfp4_transposed_b(a, s, a, s)
    with pytest.raises(ValueError, match="K must be a multiple of 16, got 8"):
        gemm_nvfp4_transposed_b(a[:, :4], s, torch.ones(1), a[:, :4], s, torch.ones(1))
    with pytest.raises(ValueError, match="3-D"):
        grouped_gemm_mxfp4_transposed_b(a, s, a, s, torch.zeros(2, dtype=torch.int32))
    with pytest.raises(TypeError):
        gemm_mxfp4_transposed_b(np.zeros((4, 16), np.uint8), s, a, s)
    with pytest.raises(ValueError, match="gate rows followed by as many up rows"):
        gemm_mxfp4_swiglu_transposed_b(a, s, a[:3], s[:3])
    with pytest.raises(ValueError, match="ROCm GPU"):
        gemm_mxfp4_swiglu_transposed_b(a, s, a, s)
    # the fused forms: shape rules first, the device check before anything is launched
    w = torch.zeros((6, 16), dtype=torch.uint8)      # 3 gate + 3 up rows: N = 3
    ws = torch.zeros((6, 1), dtype=torch.uint8)
    with pytest.raises(ValueError, match="multiple of 32"):
        gemm_mxfp4_swiglu_quant_transposed_b(a, s, w, ws)
    with pytest.raises(ValueError, match="gate rows followed by as many up rows"):
        gemm_mxfp4_swiglu_quant_transposed_b(a, s, w[:5], ws[:5])
    w64 = torch.zeros((64, 16), dtype=torch.uint8)   # N = 32
    with pytest.raises(ValueError, match="ROCm GPU"):
        gemm_mxfp4_swiglu_quant_transposed_b(a, s, w64, torch.zeros((64, 1), dtype=torch.uint8))
    ro = torch.zeros(3, dtype=torch.int32)
    with pytest.raises(ValueError, match="3-D"):
        grouped_gemm_mxfp4_swiglu_transposed_b(a, s, w, ws, ro)
    with pytest.raises(ValueError, match="gate rows followed by as many up rows"):
        grouped_gemm_mxfp4_swiglu_transposed_b(a, s, w[:5].reshape(1, 5, 16), ws[:5].reshape(1, 5, 1), ro[:2])
    with pytest.raises(ValueError, match="ROCm GPU"):
        grouped_gemm_mxfp4_swiglu_transposed_b(a, s, w.reshape(2, 3, 16)[:, :2], ws.reshape(2, 3, 1)[:, :2], ro)
    with pytest.raises(ValueError, match="multiple of 32"):     # one helper: the same order of checks as the plain form
        grouped_gemm_mxfp4_swiglu_quant_transposed_b(a, s, w.reshape(1, 6, 16), ws.reshape(1, 6, 1), ro[:2])
    with pytest.raises(ValueError, match="ROCm GPU"):
        grouped_gemm_mxfp4_swiglu_quant_transposed_b(a, s, w64.reshape(1, 64, 16), torch.zeros((1, 64, 1), dtype=torch.uint8),
                                                     ro[:2])
    with pytest.raises(ValueError, match="bfloat16"):
        moe_combine_top2(torch.zeros((8, 16)), torch.zeros((4, 2), dtype=torch.int32), torch.ones(8))
    with pytest.raises(ValueError, match="ROCm GPU"):
        moe_combine_top2(torch.zeros((8, 16), dtype=torch.bfloat16), torch.zeros((4, 2), dtype=torch.int32), torch.ones(8))
    with pytest.raises(ValueError, match="float32 or torch.bfloat16"):
        quantize_mxfp4(torch.zeros((4, 32), dtype=torch.float16))
    with pytest.raises(ValueError, match="ROCm GPU"):
        quantize_mxfp4(torch.zeros((4, 32)))
    from avelang_amd import quantize_nvfp4
    with pytest.raises(ValueError, match="multiple of 16"):
        quantize_nvfp4(torch.zeros((4, 24)), torch.ones(1))
    with pytest.raises(ValueError, match="float32 or torch.bfloat16"):
        quantize_nvfp4(torch.zeros((4, 32), dtype=torch.float16), torch.ones(1))
    with pytest.raises(ValueError, match="ROCm GPU"):
        quantize_nvfp4(torch.zeros((4, 32)), torch.ones(1))
    with pytest.raises(ValueError, match="ROCm GPU"):
        gemm_mxfp4_transposed_b(a, s, a, s, split_k=False)
    with pytest.raises(ValueError, match="ROCm GPU"):
        gemm_nvfp4_transposed_b(a, torch.zeros((4, 2), dtype=torch.uint8), torch.ones(1), a,
                                torch.zeros((4, 2), dtype=torch.uint8), torch.ones(1), split_k=False)
    with pytest.raises(ValueError, match="float32"):
        moe_route_top2(torch.zeros((4, 8), dtype=torch.float64))
    with pytest.raises(ValueError, match="ROCm GPU"):
        moe_route_top2(torch.zeros((4, 8)))
    with pytest.raises(ValueError, match="ROCm GPU"):
        gather_rows_mxfp4(a, s, torch.zeros(2, dtype=torch.int32))
    with pytest.raises(ValueError, match="ROCm GPU"):
        scales_to_blocked(s)
    assert blocked_numel(130, 5) == 256 * 8 and blocked_numel(0, 4) == 0


@pytest.mark.parametrize("m_tiles,n_tiles", [(32, 56), (1, 1), (3, 5), (129, 56), (8, 8), (7, 3), (40, 1), (1, 57),
                                             (136, 56), (64, 3), (33, 2), (31, 9)])
def test_tile_map_is_a_bijection(m_tiles, n_tiles):
    lib = _lib.load()
    tm, tn = ctypes.c_int(), ctypes.c_int()
    seen = set()
    total = m_tiles * n_tiles
    xcd_ranges = {}
    for pid in range(total):
        assert lib.ave_fp4_debug_map_tile(pid, m_tiles, n_tiles, ctypes.byref(tm), ctypes.byref(tn)) == 0
        assert 0 <= tm.value < m_tiles and 0 <= tn.value < n_tiles
        seen.add((tm.value, tn.value))
        xcd_ranges.setdefault(pid % 8, []).append(tm.value)
    assert len(seen) == total
    assert lib.ave_fp4_debug_map_tile(total, m_tiles, n_tiles, ctypes.byref(tm), ctypes.byref(tn)) == -1
    if (m_tiles, n_tiles) == (32, 56):
        # one band of 4 m-tiles per XCD: its concurrent tiles share panels in its own L2
        assert all(len(set(v)) == 4 for v in xcd_ranges.values())
    if (m_tiles, n_tiles) == (136, 56):
        # the 8 XCDs work on 8 neighbouring bands at any time: the first 224 workgroups of every XCD
        # together cover m-tiles 0..31 only
        first = [v[:224] for v in xcd_ranges.values()]
        assert set(t for v in first for t in v) == set(range(32)) and all(len(set(v)) == 4 for v in first)


def test_torch_quantisers_equal_the_oracle_quantisers():
    x = orc.activations_with_outliers(48, 256, seed=3)
    x[5, 32:64] = 0
    x[6] *= 1e-30
    x[7] *= 1e30
    p, s = orc.quantize_mxfp4(x)
    tp, ts = synth.quantize_mxfp4(torch.from_numpy(x))
    assert np.array_equal(p, tp.numpy()) and np.array_equal(s, ts.numpy())
    y = orc.randn((48, 256), seed=4, std=0.02)
    p, s, g = orc.quantize_nvfp4(y)
    tp, ts, tg = synth.quantize_nvfp4(torch.from_numpy(y))
    assert np.array_equal(p, tp.numpy()) and np.array_equal(s, ts.numpy()) and np.float32(g) == tg.item()
    ties = torch.tensor([[0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 7.0, -0.25, -5.0, 0.0, -0.0, 6.0, 4.0, 3.0, 2.0]])
    assert np.array_equal(orc.encode_e2m1(ties.numpy()), synth._e2m1_codes(ties).numpy())


def test_torch_moe_routing_shape_contract():
    g = torch.Generator().manual_seed(0)
    tok, ro = synth.moe_routing(512, 8, 2, g, "cpu")
    assert ro.dtype == torch.int32 and ro[0] == 0 and ro[-1] == 1024 and bool((ro[1:] >= ro[:-1]).all())
    assert bool((torch.bincount(tok, minlength=512) == 2).all())


def _split_plan(m, n, k, cus=256):
    lib = _lib.load()
    slices, per, narrow = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    ws = ctypes.c_size_t()
    assert lib.ave_fp4_debug_split_plan(m, n, k, cus, ctypes.byref(slices), ctypes.byref(per), ctypes.byref(narrow),
                                        ctypes.byref(ws)) == 0
    return slices.value, per.value, narrow.value, ws.value


def test_split_planner_arithmetic():
    """The K-split planner is host arithmetic: checked here for a device with 256 compute units."""
    # the down projection at decode batch sizes: split, on the narrow-tile kernel's tiles (its 128 x 128 tiles fit the
    # compute units up to 1024 rows, where they leave no room for a second slice), one work item per compute unit at most
    for m in (128, 256, 512):
        slices, per, tiling, ws = _split_plan(m, 4096, 14336)
        pairs = 14336 // 512
        assert slices > 1 and tiling in (1, 2)                                    # 256 x 128 or 128 x 128 tiles
        assert slices == -(-pairs // per) and (slices - 1) * per < pairs          # every slice holds work
        assert slices * -(-m // (256 if tiling == 1 else 128)) * (4096 // 128) <= 256
        assert ws == slices * m * 4096 * 4
    assert _split_plan(128, 4096, 14336)[2] == 2 and _split_plan(256, 4096, 14336)[2] == 2
    # 33..64 rows over a long K: the split as well (the weight-streaming kernel's four row blocks cost more there)
    assert _split_plan(33, 4096, 14336)[0] > 1 and _split_plan(64, 5120, 13824)[0] > 1
    # not split: the weight-streaming kernel's rows, K not in whole pairs of stages, enough tiles, too little K,
    # the gate/up shape (one row of 112 tiles gains nothing from two slices)
    # and 1024 or 2048 rows of the down projection (256 narrow tiles: one per compute unit without a split)
    for shape in ((32, 4096, 14336), (64, 4096, 8192), (128, 4096, 14336 + 256), (8192, 14336, 4096), (128, 4096, 512), (128, 28672, 4096),
                  (1024, 4096, 14336), (2048, 4096, 14336)):
        assert _split_plan(*shape) == (1, 0, 0, 0), shape
    # fewer compute units, fewer slices; a device too small for two slices does not split
    many = _split_plan(128, 4096, 14336, 256)[0]
    few = _split_plan(128, 4096, 14336, 64)[0]
    assert 1 < few < many and _split_plan(128, 4096, 14336, 16)[0] == 1
    lib = _lib.load()
    assert lib.ave_fp4_debug_split_plan(128, 128, 1024, 0, None, None, None, None) == -1


def test_split_plans_beyond_the_allocation_free_scratch_are_replanned_under_it():
    """On 256 compute units some planned splits want more than the 32 MiB of partial sums that the allocation-free
    entry point holds (a few hundred rows against a K of 30000 and more).  Planned under that cap, every such shape
    gets a split that fits or none, and a shape whose plan fits is planned the same with and without the cap."""
    lib = _lib.load()
    cap = 32 << 20
    sl, per, tiles, ws = ctypes.c_int(), ctypes.c_int(), ctypes.c_int(), ctypes.c_size_t()
    out = (ctypes.byref(sl), ctypes.byref(per), ctypes.byref(tiles), ctypes.byref(ws))
    over = 0
    for m in range(65, 2200, 64):
        for n in (1024, 4096):
            for k in range(2048, 53249, 2048):
                free = _split_plan(m, n, k)
                assert lib.ave_fp4_debug_split_plan_capped(m, n, k, 256, cap, *out) == 0
                capped = (sl.value, per.value, tiles.value, ws.value)
                assert capped[3] <= cap and capped[3] == (capped[0] * m * n * 4 if capped[0] > 1 else 0)
                if free[3] <= cap:
                    assert capped == free, (m, n, k)
                else:
                    over += 1
                    pairs = k // 512
                    assert capped[0] == 1 or (capped[0] == -(-pairs // capped[1]) and (capped[0] - 1) * capped[1] < pairs)
    assert over > 0 and _split_plan(513, 4096, 30720)[3] > cap   # such shapes exist: the cap is not vacuous



def _locate(table, total_m, tile_rows, tm):
    import ctypes
    lib = _lib.load()
    arr = (ctypes.c_int32 * len(table))(*table)
    e, b, t = ctypes.c_int(-1), ctypes.c_int(-1), ctypes.c_int(-1)
    rc = lib.ave_fp4_debug_locate_group_tile(arr, len(table) - 1, total_m, tile_rows, tm, ctypes.byref(e), ctypes.byref(b),
                                             ctypes.byref(t))
    assert rc in (0, 1), _lib.last_error()
    return (e.value, b.value, t.value) if rc == 1 else None


def _tiles(table, total_m, tile_rows):
    out, tm = [], 0
    while (hit := _locate(table, total_m, tile_rows, tm)) is not None:
        out.append(hit)
        tm += 1
        assert tm < 10000
    return out


@pytest.mark.parametrize("tile_rows", [32, 128, 256])
def test_grouped_tile_walk_covers_every_row_once(tile_rows):
    """The function the grouped kernels run on the device, on the host: a well-formed table yields, expert by
    expert, tiles that cover every row exactly once and end at the expert's last row."""
    table = [0, 300, 300, 811, 1000, 1000, 1001]
    tiles = _tiles(table, 1001, tile_rows)
    covered = np.zeros(1001, dtype=int)
    for e, b, t in tiles:
        assert table[e] <= b < t == table[e + 1] and (b - table[e]) % tile_rows == 0
        covered[b:min(b + tile_rows, t)] += 1
    assert (covered == 1).all()
    assert len(tiles) == sum(-(-(table[i + 1] - table[i]) // tile_rows) for i in range(6))
    assert len(tiles) <= -(-1001 // tile_rows) + 6        # the grid the launchers size: ceil(M / rows) + E


@pytest.mark.parametrize("table,total_m", [
    ([0, 100, 5000], 300),            # a table left over from a larger batch: end past total_M
    ([-50, 100, 300], 300),           # negative start
    ([0, 200, 100, 300], 300),        # decreasing pair
    ([0, 1 << 30, -(1 << 30), 7], 300),
    ([500, 600, 700], 300),           # everything past the end
    ([0, 0, 0], 0),                   # nothing at all
])
def test_grouped_tile_walk_stays_inside_the_matrix_for_a_malformed_table(table, total_m):
    """Entries are clamped to [0, total_M] and empty ranges have no tiles: rows may stay unwritten, but no tile
    starts or ends outside the matrix, whatever the table holds."""
    for tile_rows in (32, 128, 256):
        for e, b, t in _tiles(table, total_m, tile_rows):
            assert 0 <= e < len(table) - 1 and 0 <= b < t <= total_m
    for tm in (0, 1, 5, 10 ** 6):
        hit = _locate(table, total_m, 256, tm)
        assert hit is None or 0 <= hit[1] < hit[2] <= total_m


def test_generic_kernel_grid_has_room_for_millions_of_rows():
    """The m-tiles of the shape-agnostic kernels share one grid dimension with the n-blocks, so that M is not capped
    at 65535 tiles of 32 rows; what does not fit 2^31 - 1 workgroups is reported, not truncated."""
    import ctypes
    lib = _lib.load()
    wg = ctypes.c_uint(0)
    for m, n, e, want in [(1, 1, 0, 1), (33, 129, 0, 4), (1 << 22, 256, 0, 2 * (1 << 17)), (100, 128, 8, 12),
                          (1 << 30, 1 << 20, 0, 0), ((1 << 31) - 1, 128, 0, 1 << 26)]:
        assert lib.ave_fp4_debug_generic_grid(m, n, e, ctypes.byref(wg)) == 0
        assert wg.value == want, (m, n, e)
    assert lib.ave_fp4_debug_generic_grid(0, 5, 0, ctypes.byref(wg)) == -1


def test_weights_from_hbm_hint_models_the_last_level_cache():
    """The dispatch hint for the 256 x 256 kernel's look-ahead touches: a weight tensor is taken to be cache-resident
    when it is among the device's most recent weight tensors whose sizes add up to 192 MB at most."""
    lib = _lib.load()
    mb = 1 << 20

    def hint(addr, size):
        return lib.ave_fp4_debug_weights_from_hbm(ctypes.c_void_p(addr), size)

    base = 0x7000_0000_0000
    # one GEMM replayed on the same weights (the reference benchmark's protocol): cold once, then resident
    assert hint(base, 31 * mb) == 1
    assert [hint(base, 31 * mb) for _ in range(3)] == [0, 0, 0]
    # nine weight buffers in turn (a model's layers): each has left the window when its turn comes again
    for _ in range(3):
        assert [hint(base + (i + 1) * 64 * mb, 31 * mb) for i in range(9)] == [1] * 9
    # a small block replayed (gate/up 62 MB + down 31 MB): both resident from the second round on
    w1, w2 = base + 0x1000_0000_00, base + 0x2000_0000_00
    assert (hint(w1, 62 * mb), hint(w2, 31 * mb)) == (1, 1)
    assert [(hint(w1, 62 * mb), hint(w2, 31 * mb)) for _ in range(3)] == [(0, 0)] * 3
    # two large weight tensors in turn do not fit the window together
    big1, big2 = base + 0x3000_0000_00, base + 0x4000_0000_00
    assert [(hint(big1, 150 * mb), hint(big2, 150 * mb)) for _ in range(3)] == [(1, 1)] * 3


def test_tiles_per_workgroup_of_the_weight_streaming_kernels():
    """One round of workgroups while ceil(tiles / CUs) fits the most tiles a workgroup takes; beyond that balanced
    rounds instead of a full round and a nearly empty one.  Every choice covers all tiles."""
    lib = _lib.load()
    f = lib.ave_fp4_debug_tiles_per_workgroup
    assert f(1792, 256, 7, 1) == 7            # N = 28672: the decode benchmark, one round of 256 workgroups
    assert f(256, 256, 7, 1) == 1 and f(100, 256, 7, 1) == 1
    assert f(513, 256, 7, 1) == 3             # one round of 171 workgroups, not two of 2-tile workgroups
    assert f(2048, 256, 7, 1) == 4            # N = 32768: two rounds of 256 workgroups of 4 tiles
    assert f(1793, 256, 7, 1) == 4
    assert f(1792, 256, 8, 4) == 8 and f(1024, 256, 8, 4) == 4 and f(2560, 256, 8, 4) == 4   # fused quantiser: 4 or 8
    assert f(0, 256, 7, 1) == 0 and f(10, 256, 7, 8) == 0
    for n in list(range(1, 4000, 37)) + [1792, 1793, 2048, 3584, 3585]:
        for cus in (8, 104, 256, 304):
            t = f(n, cus, 7, 1)
            assert 1 <= t <= 7
            rounds = -(-(-(-n // t)) // cus)
            # never worse than the former rule (ceil(n / cus) clamped to 7) by the model the choice minimises
            t_old = min(7, max(1, -(-n // cus)))
            assert rounds * (t + 1) <= -(-(-(-n // t_old)) // cus) * (t_old + 1)
