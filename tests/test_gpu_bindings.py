"""Calls through the pybind11 extension under the reference's import path
(``from avelang_kernels.amdgpu_gemm_fp4 import ...``; interface being mirrored: reference
python/avelang_kernels/amdgpu_gemm.py:458-494, python/src/avelang_bindings.cc:493-529) give the ctypes result bit for
bit, keep the ``out=`` semantics, and stay capturable in a graph."""
import numpy as np
import pytest
import torch

import avelang_amd
from avelang_kernels import _ave_fp4_bindings as ext
from avelang_kernels import amdgpu_gemm_fp4 as ak
from tests import helpers as H

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("m,n,k", [(256, 384, 512), (16, 640, 1024), (100, 200, 96), (200, 4096, 4096)])
def test_mxfp4_through_the_extension_equals_ctypes(gpu, m, n, k):
    a, a_s = H.mx_operand(m, k, seed=1, outliers=True)
    b, b_s = H.mx_operand(n, k, seed=2, std=0.02)
    ops = [H.to_dev(x, gpu) for x in (a, a_s, b, b_s)]
    got = ak.gemm_mxfp4_transposed_b(*ops)
    want = avelang_amd.gemm_mxfp4_transposed_b(*ops)
    assert got.dtype == torch.bfloat16 and got.shape == (m, n) and torch.equal(got, want)
    H.assert_mx_close(H.bits(got), a, a_s, b, b_s)
    out = torch.empty((m, n), dtype=torch.bfloat16, device=gpu)
    assert ak.gemm_mxfp4_transposed_b(*ops, out=out) is out and torch.equal(out, want)
    with pytest.raises(ValueError, match="out must have shape"):
        ak.gemm_mxfp4_transposed_b(*ops, out=torch.empty((m, n + 1), dtype=torch.bfloat16, device=gpu))


def test_nvfp4_and_grouped_through_the_extension_equal_ctypes(gpu):
    a, a_s, a_g = H.nv_operand(130, 1024, seed=3)
    b, b_s, b_g = H.nv_operand(264, 1024, seed=4, std=0.02)
    ag = torch.tensor([a_g], dtype=torch.float32, device=gpu)
    bg = torch.tensor([b_g], dtype=torch.float32, device=gpu)
    ops = (H.to_dev(a, gpu), H.to_dev(a_s, gpu), ag, H.to_dev(b, gpu), H.to_dev(b_s, gpu), bg)
    got = ak.gemm_nvfp4_transposed_b(*ops)
    assert torch.equal(got, avelang_amd.gemm_nvfp4_transposed_b(*ops))
    H.assert_nv_close(H.bits(got), a, a_s, a_g, b, b_s, b_g)
    ro = np.array([0, 100, 100, 356, 400], dtype=np.int32)
    ga, ga_s = H.mx_operand(400, 512, seed=5)
    gw = [H.mx_operand(272, 512, seed=6 + i, std=0.02) for i in range(4)]
    gops = (H.to_dev(ga, gpu), H.to_dev(ga_s, gpu), H.to_dev(np.stack([w[0] for w in gw]), gpu),
            H.to_dev(np.stack([w[1] for w in gw]), gpu), H.to_dev(ro, gpu))
    got = ak.grouped_gemm_mxfp4_transposed_b(*gops)
    assert torch.equal(got, avelang_amd.grouped_gemm_mxfp4_transposed_b(*gops))


def test_extension_takes_tensors_as_pointers_and_reports_errors(gpu):
    """Objects with data_ptr() are accepted where the C ABI takes a pointer, as the reference's launcher does; a
    variant that cannot run the shape raises ValueError with the library's text."""
    a, a_s = H.mx_operand(64, 512, seed=7)
    b, b_s = H.mx_operand(128, 512, seed=8, std=0.02)
    da, das, db, dbs = (H.to_dev(x, gpu) for x in (a, a_s, b, b_s))
    out = torch.empty((64, 128), dtype=torch.bfloat16, device=gpu)
    stream = torch.cuda.current_stream(gpu).cuda_stream
    assert ext.ave_fp4_gemm_mxfp4(da, das, db, dbs, out, 64, 128, 512, stream) == 0
    torch.cuda.synchronize()
    H.assert_mx_close(H.bits(out), a, a_s, b, b_s)
    with pytest.raises(ValueError, match="decode kernel does not support"):
        ext.ave_fp4_gemm_mxfp4_ex(da, das, db, dbs, out, 65, 128, 512, stream, 3)


def test_calls_through_the_extension_are_captured_in_a_graph(gpu):
    """No allocation, no synchronisation: the reference benchmark captures its launches
    (benchmark/gemm/bench_amdgpu_gemm.py:37-41), and so can a caller of this module."""
    m, n, k = 512, 768, 1024
    a, a_s = H.mx_operand(m, k, seed=9)
    b, b_s = H.mx_operand(n, k, seed=10, std=0.02)
    ops = [H.to_dev(x, gpu) for x in (a, a_s, b, b_s)]
    out = torch.zeros((m, n), dtype=torch.bfloat16, device=gpu)
    want = ak.gemm_mxfp4_transposed_b(*ops).clone()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=torch.cuda.Stream()):
        ak.gemm_mxfp4_transposed_b(*ops, out=out)
    for _ in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)
