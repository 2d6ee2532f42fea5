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
