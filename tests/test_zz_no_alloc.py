"""The allocation-free entry point ave_fp4_gemm_mxfp4_noalloc (partial sums of the K split in the library's own
static device array) against ave_fp4_gemm_mxfp4_ws with a caller's workspace: same kernels, same split, so the
bf16 results must agree bit for bit -- on two calls in a row, the second on a smaller problem, so that the second
call finds the first one's partial sums in the shared array.  A shape whose planned split would not fit the array
runs on the best split that does, and is checked against exact arithmetic and the one-launch GEMM's tolerance."""
import numpy as np
import pytest
import torch

from avelang_amd import _lib
from tests import helpers as H

pytestmark = pytest.mark.gpu
SCRATCH_BYTES = 32 << 20   # AVE_FP4_NOALLOC_SCRATCH_BYTES


def _args(device, a, a_s, b, b_s):
    return tuple(H.to_dev(x, device) for x in (a, a_s, b, b_s))


def _noalloc(device, ops, m, n, k):
    """One call for the result; then the same call again between two readings of the device's free memory
    (hipMemGetInfo, which sees every allocation on the device, the library's own included -- torch's counters see
    only torch's).  The first call may load code objects and looks the scratch's address up; the second has nothing
    left to set up, so any byte it takes or returns is an allocation inside the entry point."""
    lib = _lib.load()
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=device)
    stream = torch.cuda.current_stream(device).cuda_stream
    _lib.check(lib.ave_fp4_gemm_mxfp4_noalloc(*(t.data_ptr() for t in ops), out.data_ptr(), m, n, k, stream))
    torch.cuda.synchronize(device)
    first = H.bits(out)
    out.fill_(float("nan"))
    torch.cuda.synchronize(device)
    before, allocated = torch.cuda.mem_get_info(device)[0], torch.cuda.memory_allocated(device)
    _lib.check(lib.ave_fp4_gemm_mxfp4_noalloc(*(t.data_ptr() for t in ops), out.data_ptr(), m, n, k, stream))
    torch.cuda.synchronize(device)
    assert torch.cuda.mem_get_info(device)[0] == before and torch.cuda.memory_allocated(device) == allocated
    assert np.array_equal(H.bits(out), first)
    return first


def _with_workspace(device, ops, m, n, k):
    lib = _lib.load()
    need = lib.ave_fp4_gemm_mxfp4_workspace_bytes(m, n, k)
    ws = torch.full((max(need, 4) // 4,), float("nan"), dtype=torch.float32, device=device)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=device)
    _lib.check(lib.ave_fp4_gemm_mxfp4_ws(*(t.data_ptr() for t in ops), out.data_ptr(), m, n, k, ws.data_ptr(), need,
                                         torch.cuda.current_stream(device).cuda_stream))
    torch.cuda.synchronize(device)
    return H.bits(out), need


def test_noalloc_equals_the_workspace_entry_point_on_two_calls_in_a_row(gpu):
    # a few hundred rows against the down projection's weights: few output tiles, a long K -> split along K
    shapes = [(512, 4096, 14336), (136, 1000, 14336)]   # the first fills the scratch to its last byte
    for i, (m, n, k) in enumerate(shapes):
        a, a_s = H.mx_operand(m, k, seed=60 + i, outliers=True)
        b, b_s = H.mx_operand(n, k, seed=70 + i, std=0.02)
        ops = _args(gpu, a, a_s, b, b_s)
        want, need = _with_workspace(gpu, ops, m, n, k)
        assert 0 < need <= SCRATCH_BYTES, "shape chosen so that K is split and the partial sums fit the scratch"
        got = _noalloc(gpu, ops, m, n, k)
        assert np.array_equal(got, want), (m, n, k)
        if i == 1:
            H.assert_mx_close(got, a, a_s, b, b_s)   # and the smaller problem against exact arithmetic
    # a third call, same operands as the second: the result does not depend on what the scratch held before
    assert np.array_equal(_noalloc(gpu, ops, m, n, k), want)


def test_noalloc_shapes_that_are_not_split_and_argument_checks(gpu):
    lib = _lib.load()
    # not split (many tiles): the one-launch GEMM, bit for bit
    m, n, k = 300, 2200, 512
    a, a_s = H.mx_operand(m, k, seed=80)
    b, b_s = H.mx_operand(n, k, seed=81, std=0.02)
    ops = _args(gpu, a, a_s, b, b_s)
    assert lib.ave_fp4_gemm_mxfp4_workspace_bytes(m, n, k) == 0
    assert np.array_equal(_noalloc(gpu, ops, m, n, k), H.run_mx(gpu, a, a_s, b, b_s))
    assert lib.ave_fp4_gemm_mxfp4_workspace_bytes(512, 4096, 14336) <= SCRATCH_BYTES
    # argument checks are those of the plain entry point
    rc = lib.ave_fp4_gemm_mxfp4_noalloc(ops[0].data_ptr(), ops[1].data_ptr(), ops[2].data_ptr(), ops[3].data_ptr(), 0,
                                        300, 2200, 500, torch.cuda.current_stream(gpu).cuda_stream)
    assert rc == -1 and "multiple of 32" in _lib.last_error()


def test_noalloc_takes_a_smaller_split_when_the_planned_one_does_not_fit_the_scratch(gpu):
    """513 x 4096 x 30720: with a workspace K is cut into 5 slices (40 MiB of partial sums on 256 compute units); the
    allocation-free call runs the best split under 32 MiB instead of refusing the shape.  Checked against exact
    arithmetic to the GEMM's tolerance, and the workspace call beside it."""
    import ctypes
    lib = _lib.load()
    m, n, k = 513, 4096, 30720
    cus = torch.cuda.get_device_properties(gpu).multi_processor_count // 8 * 8
    sl, per, tiles, ws = ctypes.c_int(), ctypes.c_int(), ctypes.c_int(), ctypes.c_size_t()
    assert lib.ave_fp4_debug_split_plan_capped(m, n, k, cus, SCRATCH_BYTES, ctypes.byref(sl), ctypes.byref(per), ctypes.byref(tiles),
                                               ctypes.byref(ws)) == 0
    assert ws.value <= SCRATCH_BYTES
    a, a_s = H.mx_operand(m, k, seed=90, outliers=True)
    b, b_s = H.mx_operand(n, k, seed=91, std=0.02)
    ops = _args(gpu, a, a_s, b, b_s)
    got = _noalloc(gpu, ops, m, n, k)
    H.assert_mx_close(got, a, a_s, b, b_s)
    want, need = _with_workspace(gpu, ops, m, n, k)
    if cus == 256:
        assert need > SCRATCH_BYTES and sl.value > 1, "shape chosen so that the uncapped plan does not fit and the capped one still splits"
    H.assert_mx_close(want, a, a_s, b, b_s)
    if need <= SCRATCH_BYTES:
        assert np.array_equal(got, want)
