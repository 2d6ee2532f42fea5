"""Operands of 4 GiB and more: the fast kernels address operands with 32-bit byte offsets and must hand
such calls to the shape-agnostic kernel, whose offsets are 64-bit.  Rows either side of the 2^32-byte
boundary are checked against the oracle."""
import numpy as np
import pytest
import torch

from avelang_amd import gemm_mxfp4_transposed_b
from tests import helpers as H

pytestmark = pytest.mark.gpu
TILE, DECODE = 2, 3


def _random_operand(gpu, rows, k, seed):
    g = torch.Generator(device=gpu).manual_seed(seed)
    data = torch.randint(0, 256, (rows, k // 2), dtype=torch.uint8, device=gpu, generator=g)
    scales = torch.randint(121, 130, (rows, k // 32), dtype=torch.uint8, device=gpu, generator=g)
    return data, scales


def test_a_operand_past_4_gib(gpu):
    m, n, k = (1 << 20) + 300, 64, 8192           # A: 4.3 GB of packed codes; row 2^20 starts at byte 2^32
    a, a_s = _random_operand(gpu, m, k, 1)
    b, b_s = _random_operand(gpu, n, k, 2)
    with pytest.raises(ValueError, match="tile kernel does not support"):
        gemm_mxfp4_transposed_b(a, a_s, b, b_s, variant=TILE)
    c = gemm_mxfp4_transposed_b(a, a_s, b, b_s)
    torch.cuda.synchronize()
    rows = torch.tensor([0, 1, 255, 1 << 19, (1 << 20) - 1, 1 << 20, (1 << 20) + 1, m - 1], device=gpu)
    H.assert_mx_close(H.bits(c[rows]), a[rows].cpu().numpy(), a_s[rows].cpu().numpy(), b.cpu().numpy(),
                      b_s.cpu().numpy())


def test_b_operand_past_4_gib_with_decode_shape(gpu):
    m, n, k = 16, (1 << 20) + 48, 8192            # M <= 16, but B is past 4 GiB: no weight-streaming kernel
    a, a_s = _random_operand(gpu, m, k, 3)
    b, b_s = _random_operand(gpu, n, k, 4)
    with pytest.raises(ValueError, match="decode kernel does not support"):
        gemm_mxfp4_transposed_b(a, a_s, b, b_s, variant=DECODE)
    c = gemm_mxfp4_transposed_b(a, a_s, b, b_s)
    torch.cuda.synchronize()
    cols = torch.tensor([0, 17, (1 << 20) - 1, 1 << 20, (1 << 20) + 1, n - 1], device=gpu)
    H.assert_mx_close(H.bits(c[:, cols].contiguous()), a.cpu().numpy(), a_s.cpu().numpy(), b[cols].cpu().numpy(),
                      b_s[cols].cpu().numpy())
