"""Blocked <-> row-major scale layout conversion on the device against the oracle (bit-exact), and a GEMM
fed from a blocked scale tensor."""
import numpy as np
import pytest
import torch

from avelang_amd import blocked_numel, gemm_mxfp4_transposed_b, scales_from_blocked, scales_to_blocked
from oracle import fp4_oracle as orc
from tests import helpers as H

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rows,cols", [(1, 1), (128, 4), (130, 5), (300, 128), (256, 896), (8192, 128), (33, 7)])
def test_to_and_from_blocked_equal_oracle(gpu, rows, cols):
    rng = np.random.default_rng(rows + cols)
    s = rng.integers(1, 256, size=(rows, cols), dtype=np.uint8)
    want = orc.scales_to_blocked(s)
    out = torch.full((blocked_numel(rows, cols),), 0xAB, dtype=torch.uint8, device=gpu)
    got = scales_to_blocked(H.to_dev(s, gpu), out=out)
    assert got is out and np.array_equal(got.cpu().numpy(), want)      # padding overwritten with zeros
    back = scales_from_blocked(H.to_dev(want, gpu), rows, cols)
    assert np.array_equal(back.cpu().numpy(), s)


def test_unaligned_row_major_view_takes_the_byte_path(gpu):
    s = np.random.default_rng(3).integers(1, 256, size=(40, 8), dtype=np.uint8)
    buf = torch.zeros(40 * 8 + 1, dtype=torch.uint8, device=gpu)
    view = buf[1:].view(40, 8)
    view.copy_(H.to_dev(s, gpu))
    assert np.array_equal(scales_to_blocked(view).cpu().numpy(), orc.scales_to_blocked(s))
    out = torch.zeros(40 * 8 + 1, dtype=torch.uint8, device=gpu)
    scales_from_blocked(H.to_dev(orc.scales_to_blocked(s), gpu), 40, 8, out=out[1:].view(40, 8))
    assert np.array_equal(out[1:].view(40, 8).cpu().numpy(), s) and out[0].item() == 0


def test_gemm_from_blocked_scales_and_validation(gpu):
    a, a_s = H.mx_operand(200, 512, seed=1)
    b, b_s = H.mx_operand(136, 512, seed=2, std=0.02)
    da_s = scales_from_blocked(H.to_dev(orc.scales_to_blocked(a_s), gpu), 200, 16)
    db_s = scales_from_blocked(H.to_dev(orc.scales_to_blocked(b_s), gpu), 136, 16)
    c = gemm_mxfp4_transposed_b(H.to_dev(a, gpu), da_s, H.to_dev(b, gpu), db_s)
    H.assert_mx_close(H.bits(c), a, a_s, b, b_s)
    with pytest.raises(ValueError, match="blocked must hold"):
        scales_from_blocked(torch.zeros(100, dtype=torch.uint8, device=gpu), 200, 16)
    with pytest.raises(ValueError, match="scales must be 2-D"):
        scales_to_blocked(torch.zeros(100, dtype=torch.uint8, device=gpu))
    assert scales_to_blocked(torch.zeros((0, 4), dtype=torch.uint8, device=gpu)).numel() == 0
