"""Device-side MXFP4 quantiser against the CPU oracle's quantiser (bit-exact), and through the GEMM."""
import numpy as np
import pytest
import torch

from avelang_amd import gemm_mxfp4_transposed_b, quantize_mxfp4
from oracle import fp4_oracle as orc

pytestmark = pytest.mark.gpu


def _canon(packed):
    """-0 and +0 are the same value: map code 8 to 0 before comparing."""
    codes = orc.unpack_fp4(packed)
    return np.where(codes == 8, 0, codes)


def _inputs():
    x = orc.activations_with_outliers(96, 512, seed=21)
    x[3, 32:64] = 0.0                       # an all-zero block
    x[4] *= 1e-30                           # tiny magnitudes
    x[5] *= 1e30                            # huge magnitudes
    x[6] *= 1e-38                           # subnormal amax in some blocks -> scale byte 0
    ties = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 7.0, -0.25, -5.0, 0.0, -0.0, 6.0, 4.0, 3.0, 2.0],
                    dtype=np.float32)
    x[7, :32] = np.tile(ties, 2)            # amax 7 -> scale 1: every tie of the grid
    x[8, :32] = np.tile(ties, 2) * 2.0 ** -40
    return x


def test_quantise_f32_equals_oracle(gpu):
    x = _inputs()
    want_p, want_s = orc.quantize_mxfp4(x)
    p, s = quantize_mxfp4(torch.from_numpy(x).to(gpu))
    assert np.array_equal(s.cpu().numpy(), want_s)
    assert np.array_equal(_canon(p.cpu().numpy()), _canon(want_p))


def test_quantise_bf16_equals_oracle(gpu):
    xb = torch.from_numpy(_inputs()).to(torch.bfloat16)
    want_p, want_s = orc.quantize_mxfp4(xb.float().numpy())
    p, s = quantize_mxfp4(xb.to(gpu))
    assert np.array_equal(s.cpu().numpy(), want_s)
    assert np.array_equal(_canon(p.cpu().numpy()), _canon(want_p))


def test_quantise_large_and_out_arguments(gpu):
    g = torch.Generator(device=gpu).manual_seed(5)
    x = torch.randn((4096, 4096), generator=g, device=gpu)
    p, s = quantize_mxfp4(x)
    # sampled rows against the oracle, whole tensor against the torch implementation of the same recipe
    rows = [0, 1, 2047, 4095]
    want_p, want_s = orc.quantize_mxfp4(x[rows].cpu().numpy())
    assert np.array_equal(s[rows].cpu().numpy(), want_s)
    assert np.array_equal(_canon(p[rows].cpu().numpy()), _canon(want_p))
    from avelang_amd import testing as synth
    tp, ts = synth.quantize_mxfp4(x)
    assert torch.equal(ts, s)
    assert torch.equal(torch.where((tp & 0xF) == 8, tp & 0xF0, tp), torch.where((p & 0xF) == 8, p & 0xF0, p)) or \
        np.array_equal(_canon(tp.cpu().numpy()), _canon(p.cpu().numpy()))
    # in-place outputs
    p2, s2 = torch.empty_like(p), torch.empty_like(s)
    rp, rs = quantize_mxfp4(x, packed=p2, scales=s2)
    assert rp is p2 and rs is s2 and torch.equal(p2, p) and torch.equal(s2, s)
    with pytest.raises(ValueError, match="multiple of 32"):
        quantize_mxfp4(x[:, :48].contiguous())
    with pytest.raises(ValueError, match="dtype"):
        quantize_mxfp4(x.half())


def test_quantise_then_gemm(gpu):
    g = torch.Generator(device=gpu).manual_seed(6)
    x = torch.randn((128, 512), generator=g, device=gpu)
    w = torch.randn((256, 512), generator=g, device=gpu) * 0.02
    a, a_s = quantize_mxfp4(x)
    b, b_s = quantize_mxfp4(w.to(torch.bfloat16))
    c = gemm_mxfp4_transposed_b(a, a_s, b, b_s)
    ref = orc.gemm_mxfp4_fp64(a.cpu().numpy(), a_s.cpu().numpy(), b.cpu().numpy(), b_s.cpu().numpy())
    ok, rep = orc.check_bf16_against_fp64(c.view(torch.uint16).cpu().numpy(), ref, None, 512)
    assert ok, rep
    # and the quantised product is close to the unquantised one (FP4 noise only)
    exact = (x.double() @ w.double().T).cpu().numpy()
    rel = np.linalg.norm(ref - exact) / np.linalg.norm(exact)
    assert rel < 0.25
