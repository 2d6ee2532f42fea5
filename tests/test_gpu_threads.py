"""Two host threads, each launching on a stream of its own, through the same library handle: the
launch path (shape checks, the once-per-device LDS attribute, the thread-local error text) is shared
state of the library, the kernels share the compute units.  Every result must equal, bit for bit, what
the same call gives when it runs alone (the reference launches on the caller's current stream and
leaves concurrency to the caller: python/avelang/runtime/jit.py:791-831)."""
import threading

import numpy as np
import pytest
import torch

from avelang_amd import (_lib, gemm_mxfp4_transposed_b, gemm_nvfp4_transposed_b, quantize_mxfp4)
from tests.helpers import bits, mx_operand, nv_operand, to_dev

pytestmark = pytest.mark.gpu

# (M, N, K): the weight-streaming kernel, the narrow-tile kernel, the 256 x 256 tile kernel, the generic one
MX_SHAPES = [(16, 1024, 1024), (128, 2048, 1024), (512, 1024, 1024), (24, 40, 96)]


def _mx_case(gpu, shape, seed):
    m, n, k = shape
    a, a_s = mx_operand(m, k, seed)
    b, b_s = mx_operand(n, k, seed + 1, std=0.02)
    return [to_dev(x, gpu) for x in (a, a_s, b, b_s)]


def test_two_threads_on_their_own_streams_match_serial_results(gpu):
    mx = [_mx_case(gpu, s, 40 + 2 * i) for i, s in enumerate(MX_SHAPES)]
    na, nas, nag = nv_operand(96, 512, 71)
    nb, nbs, nbg = nv_operand(160, 512, 72, std=0.02)
    nv = [to_dev(na, gpu), to_dev(nas, gpu), torch.tensor([nag], dtype=torch.float32, device=gpu),
          to_dev(nb, gpu), to_dev(nbs, gpu), torch.tensor([nbg], dtype=torch.float32, device=gpu)]
    x = torch.randn(64, 1024, generator=torch.Generator().manual_seed(5)).to(gpu)

    def one_pass():
        res = [bits(gemm_mxfp4_transposed_b(*ops)) for ops in mx]
        res.append(bits(gemm_nvfp4_transposed_b(*nv)))
        q, qs = quantize_mxfp4(x)
        res += [q.cpu().numpy(), qs.cpu().numpy()]
        return res

    want = one_pass()
    torch.cuda.synchronize()
    failures = []
    start = threading.Barrier(2)

    def worker(tag, rounds):
        try:
            stream = torch.cuda.Stream(device=gpu)
            with torch.cuda.stream(stream):
                start.wait(timeout=60)
                for r in range(rounds):
                    got = one_pass()
                    for i, (g, w) in enumerate(zip(got, want)):
                        if not np.array_equal(g, w):
                            failures.append((tag, r, i))
                    assert _lib.last_error() == ""
                stream.synchronize()
        except Exception as exc:  # reported by the main thread
            failures.append((tag, repr(exc)))

    threads = [threading.Thread(target=worker, args=(t, 6)) for t in ("first", "second")]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
        assert not t.is_alive()
    assert not failures, failures
