"""GPU-side behaviour of the entry points that mirrors the reference wrapper
(python/avelang_kernels/amdgpu_gemm.py:458-494): `out=` semantics, validation, asynchronous launch on
the current stream, and graph capture (benchmark/gemm/bench_amdgpu_gemm.py:37-41)."""
import numpy as np
import pytest
import torch

from avelang_amd import gemm_mxfp4_transposed_b, gemm_nvfp4_transposed_b, grouped_gemm_mxfp4_transposed_b
from avelang_amd import testing as synth
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _mx(gpu, m, n, k, seed=0):
    g = torch.Generator(device=gpu).manual_seed(seed)
    a, a_s = synth.quantize_mxfp4(torch.randn((m, k), generator=g, device=gpu))
    b, b_s = synth.quantize_mxfp4(torch.randn((n, k), generator=g, device=gpu) * 0.02)
    return a, a_s, b, b_s


def test_out_semantics_and_validation(gpu):
    a, a_s, b, b_s = _mx(gpu, 64, 96, 256)
    c = gemm_mxfp4_transposed_b(a, a_s, b, b_s)
    assert c.shape == (64, 96) and c.dtype == torch.bfloat16 and c.device == a.device
    out = torch.full((64, 96), 7.0, dtype=torch.bfloat16, device=gpu)
    ret = gemm_mxfp4_transposed_b(a, a_s, b, b_s, out=out)
    assert ret is out and torch.equal(out, c)
    with pytest.raises(ValueError, match="out must have shape"):
        gemm_mxfp4_transposed_b(a, a_s, b, b_s, out=torch.empty((64, 95), dtype=torch.bfloat16, device=gpu))
    with pytest.raises(ValueError, match="out must have dtype"):
        gemm_mxfp4_transposed_b(a, a_s, b, b_s, out=torch.empty((64, 96), dtype=torch.float16, device=gpu))
    with pytest.raises(ValueError, match="out must be on device"):
        gemm_mxfp4_transposed_b(a, a_s, b, b_s, out=torch.empty((64, 96), dtype=torch.bfloat16))
    with pytest.raises(ValueError, match="A_scale must have shape"):
        gemm_mxfp4_transposed_b(a, a_s[:, :4], b, b_s)
    with pytest.raises(ValueError, match="contiguous"):
        gemm_mxfp4_transposed_b(a.t().contiguous().t(), a_s, b, b_s)
    # typed views of the same bytes are accepted
    if hasattr(torch, "float8_e8m0fnu") and hasattr(torch, "float4_e2m1fn_x2"):
        c2 = gemm_mxfp4_transposed_b(a.view(torch.float4_e2m1fn_x2), a_s.view(torch.float8_e8m0fnu),
                                     b.view(torch.float4_e2m1fn_x2), b_s.view(torch.float8_e8m0fnu))
        assert torch.equal(c2, c)
    # empty problems return an empty tensor without launching
    e = gemm_mxfp4_transposed_b(a[:0], a_s[:0], b, b_s)
    assert e.shape == (0, 96)


@pytest.mark.parametrize("shape", [(256, 512, 512), (16, 1024, 2048), (100, 72, 96), (4352, 4100, 512)])
def test_graph_capture_replays_match_eager(gpu, shape):
    """The launch allocates nothing and never synchronises, so it can be captured; every replay,
    with eager work in between, must reproduce the eager result bit for bit."""
    m, n, k = shape
    a, a_s, b, b_s = _mx(gpu, m, n, k, seed=1)
    out = torch.zeros((m, n), dtype=torch.bfloat16, device=gpu)
    eager = gemm_mxfp4_transposed_b(a, a_s, b, b_s).clone()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    stream = torch.cuda.Stream()
    with torch.cuda.graph(graph, stream=stream):
        gemm_mxfp4_transposed_b(a, a_s, b, b_s, out=out)
    for i in range(3):
        out.fill_(0)                      # eager kernel between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {i}"
    # new operand contents through the same captured pointers
    a2, a2_s, _, _ = _mx(gpu, m, n, k, seed=2)
    a.copy_(a2)
    a_s.copy_(a2_s)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, gemm_mxfp4_transposed_b(a, a_s, b, b_s))


def test_launch_is_on_the_current_stream(gpu):
    a, a_s, b, b_s = _mx(gpu, 512, 512, 1024, seed=3)
    ref = gemm_mxfp4_transposed_b(a, a_s, b, b_s).clone()
    side = torch.cuda.Stream()
    out = torch.empty_like(ref)
    with torch.cuda.stream(side):
        gemm_mxfp4_transposed_b(a, a_s, b, b_s, out=out)
        done = torch.cuda.Event()
        done.record()
    done.synchronize()
    assert torch.equal(out, ref)


def test_nvfp4_and_grouped_wrappers_validate(gpu):
    g = torch.Generator(device=gpu).manual_seed(4)
    a, a_s, a_g = synth.quantize_nvfp4(torch.randn((32, 64), generator=g, device=gpu))
    b, b_s, b_g = synth.quantize_nvfp4(torch.randn((48, 64), generator=g, device=gpu))
    c = gemm_nvfp4_transposed_b(a, a_s, a_g, b, b_s, b_g)
    assert c.shape == (32, 48)
    with pytest.raises(ValueError, match="A_global"):
        gemm_nvfp4_transposed_b(a, a_s, torch.ones(2, device=gpu), b, b_s, b_g)
    with pytest.raises(ValueError, match="B_global must be on device"):
        gemm_nvfp4_transposed_b(a, a_s, a_g, b, b_s, torch.ones(1))
    am, am_s, bm, bm_s = _mx(gpu, 40, 32, 64)
    ro = torch.tensor([0, 10, 40], dtype=torch.int32, device=gpu)
    bb, bb_s = torch.stack([bm, bm]), torch.stack([bm_s, bm_s])
    c = grouped_gemm_mxfp4_transposed_b(am, am_s, bb, bb_s, ro)
    assert torch.equal(c, gemm_mxfp4_transposed_b(am, am_s, bm, bm_s))
    with pytest.raises(ValueError, match="row_offsets must have shape"):
        grouped_gemm_mxfp4_transposed_b(am, am_s, bb, bb_s, ro[:2])
    with pytest.raises(ValueError, match="int32"):
        grouped_gemm_mxfp4_transposed_b(am, am_s, bb, bb_s, ro.long())


def test_mfma_rate_probe_runs_and_counts_its_flop(gpu):
    """The diagnostic launch completes, leaves its sink alone and reports 8 waves x iters x 8 MFMAs of
    2*32*32*64 flop per workgroup."""
    import ctypes
    from avelang_amd import _lib
    lib = _lib.load()
    codes = torch.randint(0, 256, (4096,), dtype=torch.uint8, device=gpu)
    sink = torch.zeros(1, dtype=torch.float32, device=gpu)
    flop = ctypes.c_double()
    rc = lib.ave_fp4_debug_mfma_rate(codes.data_ptr(), codes.numel(), 16, 10, sink.data_ptr(),
                                     torch.cuda.current_stream().cuda_stream, ctypes.byref(flop))
    assert rc == 0, _lib.last_error()
    torch.cuda.synchronize()
    assert flop.value == 16 * 8 * 10 * 8 * 2 * 32 * 32 * 64
    assert sink.item() == 0.0
