"""GPU parity of the MXFP4 GEMM split along K (fp32 partial sums in a caller-provided workspace, added up by a
second kernel) against the oracle, and of the entry point that decides about the split by itself."""
import numpy as np
import pytest
import torch

from avelang_amd import _lib, gemm_mxfp4_transposed_b
from oracle import fp4_oracle as orc
from tests import helpers as H

pytestmark = pytest.mark.gpu


def run_forced(device, a, a_s, b, b_s, slice_pairs, narrow=0, poison=True):
    """ave_fp4_debug_gemm_mxfp4_splitk on a workspace of exactly the required size, pre-filled with NaNs."""
    lib = _lib.load()
    m, k = a.shape[0], a.shape[1] * 2
    n = b.shape[0]
    slices = -(-(k // 512) // slice_pairs)
    ws = torch.empty(slices * m * n, dtype=torch.float32, device=device)
    if poison:
        ws.fill_(float("nan"))
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=device)
    da, das, db, dbs = (H.to_dev(x, device) for x in (a, a_s, b, b_s))
    rc = lib.ave_fp4_debug_gemm_mxfp4_splitk(da.data_ptr(), das.data_ptr(), db.data_ptr(), dbs.data_ptr(), out.data_ptr(),
                                             m, n, k, ws.data_ptr(), ws.numel() * 4, slice_pairs, narrow,
                                             torch.cuda.current_stream(device).cuda_stream)
    _lib.check(rc)
    torch.cuda.synchronize(device)
    return H.bits(out)


# (M, N, K, pairs per slice): whole and ragged last slices, ragged tiles, more work items than compute units
CASES = [(100, 300, 1536, 1), (257, 256, 2560, 2), (128, 512, 4096, 3), (65, 8, 1024, 1), (300, 1000, 512, 1),
         (1100, 2300, 1024, 1)]


@pytest.mark.parametrize("narrow", [0, 1])
@pytest.mark.parametrize("m,n,k,per", CASES)
def test_split_k_matches_oracle(gpu, m, n, k, per, narrow):
    """On 256 x 256 tiles and on the 256 x 128 tiles of the three-buffer kernel; the two add up every slice in the
    same order, so they must agree bit for bit."""
    a, a_s = H.mx_operand(m, k, seed=0, outliers=True)
    b, b_s = H.mx_operand(n, k, seed=1, std=0.02)
    c = run_forced(gpu, a, a_s, b, b_s, per, narrow)
    H.assert_mx_close(c, a, a_s, b, b_s)
    if narrow:
        assert np.array_equal(c, run_forced(gpu, a, a_s, b, b_s, per, 0))


def test_split_k_unit_scales_integer_exact(gpu):
    """Every partial sum and every sum of partial sums is an integer multiple of 0.25 below 2^24: no rounding before
    the final one, so the split result must equal the correctly rounded exact sum bit for bit."""
    rng = np.random.default_rng(4)
    m, n, k = 200, 520, 2048
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    a_s = np.full((m, k // 32), 127, dtype=np.uint8)
    b_s = np.full((n, k // 32), 127, dtype=np.uint8)
    want = orc.f64_to_bf16_bits(orc.gemm_mxfp4_fp64(a, a_s, b, b_s))
    for per in (1, 3, 4):
        assert np.array_equal(run_forced(gpu, a, a_s, b, b_s, per), want), per
        assert np.array_equal(run_forced(gpu, a, a_s, b, b_s, per, narrow=1), want), per


def test_split_k_slices_see_their_own_scales(gpu):
    """Scale bytes differ per row and per 32-block, so a slice that read another slice's scale rows cannot pass."""
    rng = np.random.default_rng(5)
    m, n, k = 130, 260, 1536
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    a_s = rng.integers(117, 138, size=(m, k // 32), dtype=np.uint8)
    b_s = rng.integers(117, 138, size=(n, k // 32), dtype=np.uint8)
    H.assert_mx_close(run_forced(gpu, a, a_s, b, b_s, 1), a, a_s, b, b_s)
    H.assert_mx_close(run_forced(gpu, a, a_s, b, b_s, 2), a, a_s, b, b_s)
    H.assert_mx_close(run_forced(gpu, a, a_s, b, b_s, 1, narrow=1), a, a_s, b, b_s)
    H.assert_mx_close(run_forced(gpu, a, a_s, b, b_s, 2, narrow=1), a, a_s, b, b_s)


@pytest.mark.parametrize("m,n,k", [(33, 300, 12288), (64, 1000, 13824), (48, 4096, 14336)])
def test_33_to_64_rows_over_a_long_k_take_the_split_through_the_wrapper(gpu, m, n, k):
    """From K = 12288 the planner also splits 33..64 rows (the weight-streaming kernel pays for four blocks of
    activation rows per K panel there); up to 32 rows, and below that K, it does not.  The split result is within
    tolerance of the oracle; split_k=False gives the weight-streaming kernel's bits."""
    lib = _lib.load()
    with torch.cuda.device(gpu):
        assert lib.ave_fp4_gemm_mxfp4_workspace_bytes(m, n, k) > 0
        assert lib.ave_fp4_gemm_mxfp4_workspace_bytes(32, n, k) == 0
        assert lib.ave_fp4_gemm_mxfp4_workspace_bytes(m, n, 8192) == 0
    a, a_s = H.mx_operand(m, k, seed=m, outliers=True)
    b, b_s = H.mx_operand(n, k, seed=n, std=0.02)
    split = H.run_mx(gpu, a, a_s, b, b_s)
    H.assert_mx_close(split, a, a_s, b, b_s)
    da, das, db, dbs = (H.to_dev(x, gpu) for x in (a, a_s, b, b_s))
    whole = H.bits(gemm_mxfp4_transposed_b(da, das, db, dbs, split_k=False))
    H.assert_mx_close(whole, a, a_s, b, b_s)
    assert np.array_equal(whole, H.run_mx(gpu, a, a_s, b, b_s, variant=3))


def test_workspace_entry_point_splits_by_itself(gpu):
    lib = _lib.load()
    m, n, k = 128, 512, 8192
    with torch.cuda.device(gpu):
        need = lib.ave_fp4_gemm_mxfp4_workspace_bytes(m, n, k)
        assert need > 0 and need % (m * n * 4) == 0            # whole slices of fp32 partial sums
        assert lib.ave_fp4_gemm_mxfp4_workspace_bytes(64, n, k) == 0      # the weight-streaming kernel's shapes
        assert lib.ave_fp4_gemm_mxfp4_workspace_bytes(8192, 8192, k) == 0  # enough tiles for every compute unit
        assert lib.ave_fp4_gemm_mxfp4_workspace_bytes(m, n, 8192 + 256) == 0
    a, a_s = H.mx_operand(m, k, seed=2, outliers=True)
    b, b_s = H.mx_operand(n, k, seed=3, std=0.02)
    da, das, db, dbs = (H.to_dev(x, gpu) for x in (a, a_s, b, b_s))
    stream = torch.cuda.current_stream(gpu).cuda_stream

    def call(ws, ws_bytes):
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=gpu)
        _lib.check(lib.ave_fp4_gemm_mxfp4_ws(da.data_ptr(), das.data_ptr(), db.data_ptr(), dbs.data_ptr(), out.data_ptr(),
                                             m, n, k, ws, ws_bytes, stream))
        torch.cuda.synchronize(gpu)
        return H.bits(out)

    ws = torch.full((need // 4,), float("nan"), dtype=torch.float32, device=gpu)
    split = call(ws.data_ptr(), need)
    H.assert_mx_close(split, a, a_s, b, b_s)
    assert not torch.isnan(ws).any()                                       # every partial sum was written
    # too small a workspace, or none: the one-launch GEMM, bit for bit
    plain = H.bits(gemm_mxfp4_transposed_b(da, das, db, dbs, split_k=False))
    assert np.array_equal(call(ws.data_ptr(), need - 4), plain)
    assert np.array_equal(call(None, 0), plain)
    # the Python wrapper takes the split path by itself and gives the same bits as the C call
    assert np.array_equal(H.bits(gemm_mxfp4_transposed_b(da, das, db, dbs)), split)
    # bad arguments
    out = torch.empty((m, n), dtype=torch.bfloat16, device=gpu)
    rc = lib.ave_fp4_gemm_mxfp4_ws(da.data_ptr(), das.data_ptr(), db.data_ptr(), dbs.data_ptr(), out.data_ptr(),
                                   m, n, k, None, need, stream)
    assert rc == -1 and "workspace" in _lib.last_error()
    rc = lib.ave_fp4_gemm_mxfp4_ws(da.data_ptr(), das.data_ptr(), db.data_ptr(), dbs.data_ptr(), out.data_ptr(),
                                   m, n, k, ws.data_ptr() + 4, need, stream)
    assert rc == -1 and "aligned" in _lib.last_error()


def test_split_k_in_a_graph(gpu):
    """Captured with its workspace from the graph's pool and replayed with new activations."""
    m, n, k = 192, 256, 4096
    b, b_s = H.mx_operand(n, k, seed=7, std=0.02)
    db, dbs = H.to_dev(b, gpu), H.to_dev(b_s, gpu)
    a0, a0_s = H.mx_operand(m, k, seed=8)
    da, das = H.to_dev(a0, gpu), H.to_dev(a0_s, gpu)
    out = torch.empty((m, n), dtype=torch.bfloat16, device=gpu)
    gemm_mxfp4_transposed_b(da, das, db, dbs, out=out)
    torch.cuda.synchronize(gpu)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        gemm_mxfp4_transposed_b(da, das, db, dbs, out=out)
    for seed in (9, 10, 11):
        a, a_s = H.mx_operand(m, k, seed=seed)
        da.copy_(H.to_dev(a, gpu))
        das.copy_(H.to_dev(a_s, gpu))
        graph.replay()
        torch.cuda.synchronize(gpu)
        replayed = H.bits(out).copy()
        H.assert_mx_close(replayed, a, a_s, b, b_s)
        eager = H.bits(gemm_mxfp4_transposed_b(da, das, db, dbs))
        assert np.array_equal(replayed, eager)


# ---- the NVFP4 GEMM with a workspace --------------------------------------------------------------------------------

from avelang_amd import gemm_nvfp4_transposed_b  # noqa: E402


def _nv_dev(gpu, a, a_s, a_g, b, b_s, b_g):
    return (H.to_dev(a, gpu), H.to_dev(a_s, gpu), torch.tensor([a_g], dtype=torch.float32, device=gpu),
            H.to_dev(b, gpu), H.to_dev(b_s, gpu), torch.tensor([b_g], dtype=torch.float32, device=gpu))


@pytest.mark.parametrize("m,n,k", [(128, 512, 4096), (100, 300, 2560), (257, 256, 1024), (65, 8, 8192), (600, 1000, 1280)])
def test_nv_split_k_matches_oracle(gpu, m, n, k):
    """Whole and ragged last slices (10 and 5 stages), ragged tiles, one and several rows of tiles, tiles whose
    upper waves have no rows."""
    lib = _lib.load()
    with torch.cuda.device(gpu):
        assert lib.ave_fp4_gemm_nvfp4_workspace_bytes(m, n, k) > 0
    a, a_s, a_g = H.nv_operand(m, k, seed=m)
    b, b_s, b_g = H.nv_operand(n, k, seed=n, std=0.02)
    ops = _nv_dev(gpu, a, a_s, a_g, b, b_s, b_g)
    c = H.bits(gemm_nvfp4_transposed_b(*ops))
    H.assert_nv_close(c, a, a_s, a_g, b, b_s, b_g)
    H.assert_nv_close(H.bits(gemm_nvfp4_transposed_b(*ops, split_k=False)), a, a_s, a_g, b, b_s, b_g)


def test_nv_workspace_entry_point(gpu):
    lib = _lib.load()
    m, n, k = 192, 520, 3072
    with torch.cuda.device(gpu):
        need = lib.ave_fp4_gemm_nvfp4_workspace_bytes(m, n, k)
        assert need > 0 and need % (m * n * 4) == 0
        assert lib.ave_fp4_gemm_nvfp4_workspace_bytes(64, n, k) == 0          # the weight-streaming kernel's rows
        assert lib.ave_fp4_gemm_nvfp4_workspace_bytes(4096, 4096, k) == 0     # a tile for every compute unit
        assert lib.ave_fp4_gemm_nvfp4_workspace_bytes(m, n, 512) == 0         # two stages: nothing to split
    rng = np.random.default_rng(23)
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    a_s = np.full((m, k // 16), 0x38, dtype=np.uint8)                          # 1.0: integer-exact sums
    b_s = np.full((n, k // 16), 0x38, dtype=np.uint8)
    da, das, dag, db, dbs, dbg = _nv_dev(gpu, a, a_s, 1.0, b, b_s, 1.0)
    stream = torch.cuda.current_stream(gpu).cuda_stream

    def call(ws, ws_bytes):
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=gpu)
        _lib.check(lib.ave_fp4_gemm_nvfp4_ws(da.data_ptr(), das.data_ptr(), dag.data_ptr(), db.data_ptr(), dbs.data_ptr(),
                                             dbg.data_ptr(), out.data_ptr(), m, n, k, ws, ws_bytes, stream))
        torch.cuda.synchronize(gpu)
        return H.bits(out)

    want = orc.f64_to_bf16_bits(orc.gemm_nvfp4_fp64(a, a_s, 1.0, b, b_s, 1.0))
    ws = torch.full((need // 4,), float("nan"), dtype=torch.float32, device=gpu)
    assert np.array_equal(call(ws.data_ptr(), need), want)
    assert not torch.isnan(ws).any()                                           # every partial sum was written
    assert np.array_equal(call(ws.data_ptr(), need - 4), want)                 # too small: the one-launch GEMM
    assert np.array_equal(call(None, 0), want)
    out = torch.empty((m, n), dtype=torch.bfloat16, device=gpu)
    rc = lib.ave_fp4_gemm_nvfp4_ws(da.data_ptr(), das.data_ptr(), dag.data_ptr(), db.data_ptr(), dbs.data_ptr(),
                                   dbg.data_ptr(), out.data_ptr(), m, n, k, None, need, stream)
    assert rc == -1 and "workspace" in _lib.last_error()


def test_nv_split_k_in_a_graph(gpu):
    """Captured with its workspace from the graph's pool and replayed with new activations."""
    m, n, k = 160, 256, 4096
    b, b_s, b_g = H.nv_operand(n, k, seed=7, std=0.02)
    a0, a0_s, a0_g = H.nv_operand(m, k, seed=8)
    da, das, dag, db, dbs, dbg = _nv_dev(gpu, a0, a0_s, a0_g, b, b_s, b_g)
    out = torch.empty((m, n), dtype=torch.bfloat16, device=gpu)
    gemm_nvfp4_transposed_b(da, das, dag, db, dbs, dbg, out=out)
    torch.cuda.synchronize(gpu)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        gemm_nvfp4_transposed_b(da, das, dag, db, dbs, dbg, out=out)
    for seed in (9, 10, 11):
        a, a_s, a_g = H.nv_operand(m, k, seed=seed)
        da.copy_(H.to_dev(a, gpu))
        das.copy_(H.to_dev(a_s, gpu))
        dag.fill_(float(a_g))
        graph.replay()
        torch.cuda.synchronize(gpu)
        replayed = H.bits(out).copy()
        H.assert_nv_close(replayed, a, a_s, a_g, b, b_s, b_g)
        assert np.array_equal(replayed, H.bits(gemm_nvfp4_transposed_b(da, das, dag, db, dbs, dbg)))
