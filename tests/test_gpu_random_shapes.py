"""Seeded sweep over shapes that shape-based dispatch sends to every kernel: each case is checked against the
oracle with the stated tolerance.  Shapes are drawn once from a fixed seed, so the list is the same on every
run; it covers ragged M and N, every K granularity each kernel accepts, and empty experts."""
import numpy as np
import pytest

from oracle import fp4_oracle as orc
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _mx_cases():
    rng = np.random.default_rng(20240611)
    cases = []
    for _ in range(10):   # weight-streaming kernel, LDS ring: M <= 64, K % 512 == 0 (K % 1024 above 32 rows)
        m = int(rng.integers(1, 65))
        k = int(rng.integers(1, 9)) * (1024 if m > 32 else 512)
        cases.append((m, int(rng.integers(1, 700)), k))
    for _ in range(5):    # weight-streaming kernel, register variant: M <= 16, K % 128 == 0 but not % 512
        cases.append((int(rng.integers(1, 17)), int(rng.integers(1, 400)), int(rng.choice([128, 384, 640, 896, 1152]))))
    for _ in range(8):    # LDS-staged kernel: K % 256 == 0, any M and N
        cases.append((int(rng.integers(65, 600)), int(rng.integers(1, 600)), int(rng.integers(1, 7)) * 256))
    for _ in range(7):    # shape-agnostic kernel: K % 32 == 0 only
        cases.append((int(rng.integers(17, 200)), int(rng.integers(1, 200)), int(rng.choice([32, 96, 160, 224, 288, 800]))))
    rng = np.random.default_rng(20240612)   # a stream of its own: the cases above stay what they were
    for _ in range(10):   # narrow-tile kernel (K % 512 == 0, few tiles), 128- and 256-row forms; long K: split along K
        cases.append((int(rng.integers(65, 520)), int(rng.integers(1, 1200)), int(rng.integers(1, 9)) * 512))
    rng = np.random.default_rng(20240613)
    for _ in range(10):   # LDS-staged kernel with a K tail: any multiple of 32 from 512 up, more than 64 rows
        k = int(rng.integers(16, 100)) * 32
        cases.append((int(rng.integers(65, 700)), int(rng.integers(1, 700)), k if k % 256 else k + 32))
    for _ in range(8):    # weight-streaming kernel on the rings with a K tail: whole units of 512 plus 1..15 blocks
        m = int(rng.integers(1, 65))
        units = int(rng.integers(1, 9)) * (2 if m > 32 else 1)
        cases.append((m, int(rng.integers(1, 900)), units * 512 + int(rng.integers(1, 16)) * 32))
    for _ in range(6):    # register variant of the weight-streaming kernel with a partial last step: M <= 16, K % 128 != 0
        k = int(rng.integers(1, 60)) * 32
        cases.append((int(rng.integers(1, 17)), int(rng.integers(1, 500)), k if k % 128 else k + 32))
    return cases


@pytest.mark.parametrize("m,n,k", _mx_cases())
def test_mxfp4_random_shape(gpu, m, n, k):
    a, a_s = H.mx_operand(m, k, seed=m * 7 + k)
    b, b_s = H.mx_operand(n, k, seed=n * 11 + k, std=0.05)
    H.assert_mx_close(H.run_mx(gpu, a, a_s, b, b_s), a, a_s, b, b_s)


def _nv_cases():
    rng = np.random.default_rng(77)
    cases = [(int(rng.integers(1, 500)), int(rng.integers(1, 500)), int(rng.integers(1, 6)) * 256) for _ in range(6)]
    cases += [(int(rng.integers(1, 150)), int(rng.integers(1, 150)), int(rng.choice([16, 48, 112, 272, 528]))) for _ in range(5)]
    rng = np.random.default_rng(78)
    # weight-streaming kernels: the LDS rings (M <= 32, K % 512 == 0) and the loads into registers (M <= 64, K % 128 == 0)
    cases += [(int(rng.integers(1, 33)), int(rng.integers(1, 900)), int(rng.integers(1, 9)) * 512) for _ in range(6)]
    cases += [(int(rng.integers(1, 65)), int(rng.integers(1, 900)), int(rng.choice([128, 384, 640, 1152, 2048]))) for _ in range(6)]
    # more than 64 rows over a long K: the tile kernel split along K through the wrapper's workspace
    cases += [(int(rng.integers(65, 400)), int(rng.integers(1, 700)), int(rng.integers(4, 17)) * 256) for _ in range(5)]
    return cases


@pytest.mark.parametrize("m,n,k", _nv_cases())
def test_nvfp4_random_shape(gpu, m, n, k):
    a, a_s, a_g = H.nv_operand(m, k, seed=m + k)
    b, b_s, b_g = H.nv_operand(n, k, seed=n + 3 * k, std=0.05)
    H.assert_nv_close(H.run_nv(gpu, a, a_s, a_g, b, b_s, b_g), a, a_s, a_g, b, b_s, b_g)


def _grouped_cases():
    rng = np.random.default_rng(5)
    cases = []
    for _ in range(8):
        e = int(rng.integers(1, 9))
        rows = rng.integers(0, 400, size=e)
        rows[rng.integers(0, e)] = 0                        # at least one expert without rows
        offsets = np.concatenate([[0], np.cumsum(rows)]).astype(np.int32)
        k = int(rng.choice([256, 512, 768, 96, 160]))       # LDS-staged and shape-agnostic kernels
        cases.append((offsets.tolist(), int(rng.integers(1, 400)), k))
    rng = np.random.default_rng(6)
    for _ in range(6):    # expert layers at decode batch sizes (at most 128 rows per expert on average): narrow tiles
        e = int(rng.integers(2, 9))
        rows = rng.integers(0, 150, size=e)
        rows[rng.integers(0, e)] = 0
        offsets = np.concatenate([[0], np.cumsum(rows)]).astype(np.int32)
        cases.append((offsets.tolist(), int(rng.integers(1, 400)), int(rng.integers(1, 5)) * 512))
    rng = np.random.default_rng(7)
    for _ in range(5):    # K tails in the grouped LDS-staged kernel (more than 128 rows per expert on average)
        e = int(rng.integers(1, 5))
        rows = rng.integers(130, 700, size=e)
        if e > 1:
            rows[rng.integers(0, e)] = 0
        offsets = np.concatenate([[0], np.cumsum(rows)]).astype(np.int32)
        k = int(rng.integers(16, 60)) * 32
        cases.append((offsets.tolist(), int(rng.integers(1, 500)), k if k % 256 else k + 32))
    return cases


# Long K of an odd number of 256-element stages (scales per stage, every wave loads its share of a stage), grouped:
# a stage barrier that waits only for the loads of the waves that issue them in the pair-scale forms let the other
# waves' data arrive late here, the more often the more stages there are.
_GROUPED_ODD_STAGES = [
    ([0, 292], 1167, 7936),
    ([0, 200, 350], 917, 6912),
    ([0, 103, 336, 502, 502, 769, 769, 769, 944], 1161, 7936),
    ([0, 293, 405, 546, 823, 980, 980, 1079, 1181], 12, 1792),
]


@pytest.mark.parametrize("offsets,n,k", _GROUPED_ODD_STAGES)
@pytest.mark.parametrize("variant", [0, 2])
def test_grouped_long_k_of_odd_stage_count(gpu, offsets, n, k, variant):
    total, e = offsets[-1], len(offsets) - 1
    ws = [H.mx_operand(n, k, seed=300 + i + n, std=0.05) for i in range(e)]
    b, b_s = np.stack([w[0] for w in ws]), np.stack([w[1] for w in ws])
    a, a_s = H.mx_operand(total, k, seed=total + k)
    for _ in range(3):   # the launch is cheap, the oracle is not: several launches against one reference
        c = H.run_grouped(gpu, a, a_s, b, b_s, offsets, variant=variant)
        for i in range(e):
            r0, r1 = offsets[i], offsets[i + 1]
            if r1 > r0:
                H.assert_mx_close(c[r0:r1], a[r0:r1], a_s[r0:r1], b[i], b_s[i])


@pytest.mark.parametrize("offsets,n,k", _grouped_cases())
def test_grouped_random_shape(gpu, offsets, n, k):
    total, e = offsets[-1], len(offsets) - 1
    ws = [H.mx_operand(n, k, seed=100 + i + n, std=0.05) for i in range(e)]
    b, b_s = np.stack([w[0] for w in ws]), np.stack([w[1] for w in ws])
    if total == 0:   # every expert empty: the call succeeds, launches nothing and returns an empty [0, N] result
        a, a_s = np.zeros((0, k // 2), np.uint8), np.zeros((0, k // 32), np.uint8)
        assert H.run_grouped(gpu, a, a_s, b, b_s, offsets).shape == (0, n)
        return
    a, a_s = H.mx_operand(total, k, seed=total + k)
    c = H.run_grouped(gpu, a, a_s, b, b_s, offsets)
    for i in range(e):
        r0, r1 = offsets[i], offsets[i + 1]
        if r1 > r0:
            H.assert_mx_close(c[r0:r1], a[r0:r1], a_s[r0:r1], b[i], b_s[i])


def _swiglu_cases():
    rng = np.random.default_rng(9)
    cases = []
    for _ in range(6):    # weight-streaming kernel
        m = int(rng.integers(1, 65))
        cases.append((m, int(rng.integers(1, 80)) * 8, int(rng.integers(1, 5)) * (1024 if m > 32 else 512)))
    for _ in range(4):    # shape-agnostic kernel
        cases.append((int(rng.integers(1, 150)), int(rng.integers(1, 150)), int(rng.choice([32, 96, 256, 544]))))
    for _ in range(8):    # LDS-staged kernel: M > 64, K % 512 == 0, any N
        cases.append((int(rng.integers(65, 700)), int(rng.integers(1, 500)), int(rng.integers(1, 4)) * 512))
    return cases


@pytest.mark.parametrize("m,n,k", _swiglu_cases())
def test_swiglu_random_shape(gpu, m, n, k):
    import torch
    from avelang_amd import gemm_mxfp4_swiglu_transposed_b

    a, a_s = H.mx_operand(m, k, seed=m + k)
    b, b_s = H.mx_operand(2 * n, k, seed=n + k, std=0.05)
    c = gemm_mxfp4_swiglu_transposed_b(H.to_dev(a, gpu), H.to_dev(a_s, gpu), H.to_dev(b, gpu), H.to_dev(b_s, gpu))
    torch.cuda.synchronize()
    ok, rep = orc.check_swiglu_bf16(H.bits(c), a, a_s, b, b_s)
    assert ok, rep


def _swiglu_quant_cases():
    rng = np.random.default_rng(13)
    cases = []
    for _ in range(8):    # plain and grouped, N % 32 == 0, K % 512 == 0; some with several m-tiles per expert
        e = int(rng.integers(1, 6))
        rows = rng.integers(0, 500, size=e)
        if e > 1:
            rows[rng.integers(0, e)] = 0
        offsets = np.concatenate([[0], np.cumsum(rows)]).astype(np.int32)
        cases.append((offsets.tolist(), int(rng.integers(1, 12)) * 32, int(rng.integers(1, 4)) * 512))
    return cases


@pytest.mark.parametrize("offsets,n,k", _swiglu_quant_cases())
def test_grouped_swiglu_and_fused_quantiser_random_shape(gpu, offsets, n, k):
    """Grouped SwiGLU against exact arithmetic per expert; the fused quantiser's codes and scales equal the
    CPU quantiser applied to the kernel's own bf16 output."""
    import torch
    from avelang_amd import grouped_gemm_mxfp4_swiglu_quant_transposed_b, grouped_gemm_mxfp4_swiglu_transposed_b

    total, e = offsets[-1], len(offsets) - 1
    ws = [H.mx_operand(2 * n, k, seed=200 + i + n, std=0.05) for i in range(e)]
    b, b_s = np.stack([w[0] for w in ws]), np.stack([w[1] for w in ws])
    ro = torch.tensor(offsets, dtype=torch.int32, device=gpu)
    if total == 0:   # every expert empty: both calls succeed and return empty results of the right shapes
        da, das = (H.to_dev(np.zeros((0, k // d), np.uint8), gpu) for d in (2, 32))
        db, dbs = H.to_dev(b, gpu), H.to_dev(b_s, gpu)
        assert tuple(grouped_gemm_mxfp4_swiglu_transposed_b(da, das, db, dbs, ro).shape) == (0, n)
        q, q_s = grouped_gemm_mxfp4_swiglu_quant_transposed_b(da, das, db, dbs, ro)
        assert tuple(q.shape) == (0, n // 2) and tuple(q_s.shape) == (0, n // 32)
        return
    a, a_s = H.mx_operand(total, k, seed=total + k)
    da, das, db, dbs = (H.to_dev(v, gpu) for v in (a, a_s, b, b_s))
    c = grouped_gemm_mxfp4_swiglu_transposed_b(da, das, db, dbs, ro)
    q, q_s = grouped_gemm_mxfp4_swiglu_quant_transposed_b(da, das, db, dbs, ro)
    torch.cuda.synchronize()
    for i in range(e):
        r0, r1 = offsets[i], offsets[i + 1]
        if r1 > r0:
            ok, rep = orc.check_swiglu_bf16(H.bits(c[r0:r1]), a[r0:r1], a_s[r0:r1], b[i], b_s[i])
            assert ok, (i, rep)
    cpu_q, cpu_s = orc.quantize_mxfp4(c.float().cpu().numpy())
    assert np.array_equal(q_s.cpu().numpy(), cpu_s) and np.array_equal(q.cpu().numpy(), cpu_q)
