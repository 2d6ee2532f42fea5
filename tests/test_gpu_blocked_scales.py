"""The MXFP4 GEMM on scale tensors in the 128 x 4 blocked layout, read by the kernels directly
(ave_fp4_gemm_mxfp4_blocked_scales), against the same GEMM on the row-major tensors: same kernel, same arithmetic, so
the results must agree BIT FOR BIT; and against the oracle's tolerance.  The blocked images are made by the oracle's
numpy restatement of the layout (pinned by its byte-offset formula in tests/test_oracle_formats.py), not by the
library's own conversion kernel.  Shapes: rows and columns that are no multiples of 128 (padded blocked tensors, a
row tile that lies behind the matrix), every K range (one pair of stages, many), both kernels, a persistent launch
with more tiles than compute units, and scale bytes drawn from the whole range in every block."""
import numpy as np
import pytest
import torch

from avelang_amd import gemm_mxfp4_blocked_scales_transposed_b
from oracle import fp4_oracle as orc
from tests import helpers as H

pytestmark = pytest.mark.gpu
TILE, DECODE = 2, 3


def _blocked(gpu, a, a_s, b, b_s):
    return H.bits(gemm_mxfp4_blocked_scales_transposed_b(H.to_dev(a, gpu), H.to_dev(orc.scales_to_blocked(a_s), gpu),
                                                         H.to_dev(b, gpu), H.to_dev(orc.scales_to_blocked(b_s), gpu)))


@pytest.mark.parametrize("m,n,k", [(256, 256, 512), (300, 520, 1024), (65, 1, 512), (129, 130, 2048), (1000, 1300, 512),
                                   (4096 + 77, 4096 + 300, 1024),      # more tiles than compute units: persistent walk
                                   (127, 385, 4096), (513, 255, 1536)])
def test_blocked_scales_tile_kernel_equals_row_major_and_oracle(gpu, m, n, k):
    a, a_s = H.mx_operand(m, k, seed=m + k, outliers=True)
    b, b_s = H.mx_operand(n, k, seed=n + k, std=0.02)
    c = _blocked(gpu, a, a_s, b, b_s)
    assert np.array_equal(c, H.run_mx(gpu, a, a_s, b, b_s, variant=TILE))
    if m * n * k <= 1 << 31:
        H.assert_mx_close(c, a, a_s, b, b_s)


@pytest.mark.parametrize("m,n,k", [(16, 28672, 4096), (1, 100, 512), (16, 4096, 14336), (32, 1000, 1024), (64, 520, 2048),
                                   (17, 129, 1536), (40, 2000, 3072), (64, 300, 1024), (7, 16 * 260 + 5, 2560)])
def test_blocked_scales_decode_kernel_equals_row_major_and_oracle(gpu, m, n, k):
    a, a_s = H.mx_operand(m, k, seed=m + k)
    b, b_s = H.mx_operand(n, k, seed=n + k, std=0.02)
    c = _blocked(gpu, a, a_s, b, b_s)
    units = k // 512
    if m > 32 and units % 2:   # 33..64 rows over an odd number of 512-units: the rings cannot take a blocked tensor there
        assert np.array_equal(c, H.run_mx(gpu, a, a_s, b, b_s, variant=TILE))
    else:
        assert np.array_equal(c, H.run_mx(gpu, a, a_s, b, b_s, variant=DECODE))
    H.assert_mx_close(c, a, a_s, b, b_s)


@pytest.mark.parametrize("m", [16, 300])
def test_blocked_scales_every_block_its_own_scale_byte(gpu, m):
    """Random codes under scale bytes drawn from a wide range, different in every block of every row: a scale byte taken
    from the wrong row, K step or tile shows up at once.  Exact in fp32 (integers x powers of two), so bit for bit."""
    rng = np.random.default_rng(m)
    n, k = 392, 1024
    a = rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    a_s = rng.integers(120, 135, size=(m, k // 32)).astype(np.uint8)
    b_s = rng.integers(120, 135, size=(n, k // 32)).astype(np.uint8)
    c = _blocked(gpu, a, a_s, b, b_s)
    assert np.array_equal(c, H.run_mx(gpu, a, a_s, b, b_s, variant=DECODE if m <= 64 else TILE))
    H.assert_mx_close(c, a, a_s, b, b_s)


def test_blocked_scales_validation(gpu):
    a, a_s = H.mx_operand(70, 544, seed=1)
    b, b_s = H.mx_operand(40, 544, seed=2)
    ops = (H.to_dev(a, gpu), H.to_dev(orc.scales_to_blocked(a_s), gpu), H.to_dev(b, gpu), H.to_dev(orc.scales_to_blocked(b_s), gpu))
    with pytest.raises(ValueError, match="whole 512-element units of K"):
        gemm_mxfp4_blocked_scales_transposed_b(*ops)
    a, a_s = H.mx_operand(70, 512, seed=1)
    b, b_s = H.mx_operand(40, 512, seed=2)
    with pytest.raises(ValueError, match="A_scale_blocked must have shape"):   # the row-major tensor is not a blocked one
        gemm_mxfp4_blocked_scales_transposed_b(H.to_dev(a, gpu), H.to_dev(a_s, gpu), H.to_dev(b, gpu),
                                               H.to_dev(orc.scales_to_blocked(b_s), gpu))
    empty = gemm_mxfp4_blocked_scales_transposed_b(H.to_dev(a[:0], gpu), torch.empty(0, dtype=torch.uint8, device=gpu),
                                                   H.to_dev(b, gpu), H.to_dev(orc.scales_to_blocked(b_s), gpu))
    assert tuple(empty.shape) == (0, 40)
