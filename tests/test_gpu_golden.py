"""GPU results against the committed golden fixtures, through every kernel that accepts the shape."""
import os

import numpy as np
import pytest

from oracle import fp4_oracle as orc
from tests import helpers as H

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def within_one_ulp(got_bits, want_bits):
    got = orc.bf16_bits_to_f32(got_bits).astype(np.float64)
    want = orc.bf16_bits_to_f32(want_bits).astype(np.float64)
    return bool((np.abs(got - want) <= orc.bf16_ulp(want)).all())


@pytest.mark.parametrize("variant", [0, 1])
def test_golden_mxfp4(gpu, variant):
    z = np.load(os.path.join(GOLDEN, "mxfp4_32x48x64.npz"))
    c = H.run_mx(gpu, z["a"], z["a_scale"], z["b"], z["b_scale"], variant=variant)
    assert within_one_ulp(c, z["c_bf16_bits"])
    H.assert_mx_close(c, z["a"], z["a_scale"], z["b"], z["b_scale"])


@pytest.mark.parametrize("variant", [0, 1])
def test_golden_nvfp4(gpu, variant):
    z = np.load(os.path.join(GOLDEN, "nvfp4_32x48x64.npz"))
    c = H.run_nv(gpu, z["a"], z["a_scale"], float(z["a_global"]), z["b"], z["b_scale"], float(z["b_global"]),
                 variant=variant)
    assert within_one_ulp(c, z["c_bf16_bits"])


@pytest.mark.parametrize("variant", [0, 1])
def test_golden_grouped(gpu, variant):
    z = np.load(os.path.join(GOLDEN, "grouped_mxfp4_45x32x64.npz"))
    c = H.run_grouped(gpu, z["a"], z["a_scale"], z["b"], z["b_scale"], z["row_offsets"], variant=variant)
    assert within_one_ulp(c, z["c_bf16_bits"])


@pytest.mark.parametrize("variant", [0, 1, 2, 4])
def test_golden_mxfp4_k512(gpu, variant):
    """K = 512: shape-based dispatch (the narrow-tile kernel), the shape-agnostic, the 256 x 256 and the narrow-tile
    kernel by name; the first 16 rows alone through the weight-streaming kernel."""
    z = np.load(os.path.join(GOLDEN, "mxfp4_72x40x512.npz"))
    c = H.run_mx(gpu, z["a"], z["a_scale"], z["b"], z["b_scale"], variant=variant)
    assert within_one_ulp(c, z["c_bf16_bits"])
    H.assert_mx_close(c, z["a"], z["a_scale"], z["b"], z["b_scale"])
    if variant == 0:
        c16 = H.run_mx(gpu, z["a"][:16], z["a_scale"][:16], z["b"], z["b_scale"], variant=3)
        assert within_one_ulp(c16, z["c_bf16_bits"][:16])


@pytest.mark.parametrize("variant", [0, 1, 2, 3])
def test_golden_nvfp4_k512(gpu, variant):
    """K = 512 and 24 rows: the LDS rings (dispatch and by name), the shape-agnostic and the 256 x 256 kernel."""
    z = np.load(os.path.join(GOLDEN, "nvfp4_24x40x512.npz"))
    c = H.run_nv(gpu, z["a"], z["a_scale"], float(z["a_global"]), z["b"], z["b_scale"], float(z["b_global"]),
                 variant=variant)
    assert within_one_ulp(c, z["c_bf16_bits"])


@pytest.mark.parametrize("variant", [0, 1, 2])
def test_golden_mxfp4_k_tail(gpu, variant):
    """K = 736 = 512 + 7 blocks: shape-based dispatch and the 256 x 256 kernel by name take the K-tail form, the
    shape-agnostic kernel as a cross-check; the first 16 rows alone run on the register form of the weight-streaming
    kernel, whose last step of 128 elements holds three blocks."""
    z = np.load(os.path.join(GOLDEN, "mxfp4_72x40x736.npz"))
    c = H.run_mx(gpu, z["a"], z["a_scale"], z["b"], z["b_scale"], variant=variant)
    assert within_one_ulp(c, z["c_bf16_bits"])
    H.assert_mx_close(c, z["a"], z["a_scale"], z["b"], z["b_scale"])
    if variant == 0:
        c16 = H.run_mx(gpu, z["a"][:16], z["a_scale"][:16], z["b"], z["b_scale"], variant=3)
        assert within_one_ulp(c16, z["c_bf16_bits"][:16])


@pytest.mark.parametrize("variant", [0, 1, 5])
def test_golden_nvfp4_k320(gpu, variant):
    """K = 320, a multiple of 64 but not of 256: shape-based dispatch and variant 5 take the f16-staged tile kernel."""
    z = np.load(os.path.join(GOLDEN, "nvfp4_72x40x320.npz"))
    c = H.run_nv(gpu, z["a"], z["a_scale"], float(z["a_global"]), z["b"], z["b_scale"], float(z["b_global"]),
                 variant=variant)
    assert within_one_ulp(c, z["c_bf16_bits"])


def test_golden_nvfp4_quantiser(gpu):
    import torch
    from avelang_amd import quantize_nvfp4
    z = np.load(os.path.join(GOLDEN, "quantize_nvfp4_8x64.npz"))
    p, s = quantize_nvfp4(torch.from_numpy(z["x"]).to(gpu), torch.tensor([float(z["global_scale"])], dtype=torch.float32, device=gpu))
    assert np.array_equal(s.cpu().numpy(), z["scales"])
    got, want = orc.unpack_fp4(p.cpu().numpy()), orc.unpack_fp4(z["packed"])
    assert np.array_equal(np.where(got == 8, 0, got), np.where(want == 8, 0, want))     # -0 and +0 are the same value

