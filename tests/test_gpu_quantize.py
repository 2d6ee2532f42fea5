"""Device-side MXFP4 and NVFP4 quantisers against the CPU oracle's quantisers (bit-exact), and through the GEMMs."""
import numpy as np
import pytest
import torch

from avelang_amd import gemm_mxfp4_transposed_b, gemm_nvfp4_transposed_b, quantize_mxfp4, quantize_nvfp4
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


def _nv_inputs():
    x = orc.activations_with_outliers(96, 512, seed=41)
    x[3, 32:48] = 0.0                       # an all-zero block
    x[4] *= 1e-6                            # block scales in E4M3's subnormal range, some rounding to zero
    x[5] *= 1e-30                           # every scale byte zero: zero codes
    x[6] *= 3.0                             # beyond the calibrated range once g is halved: scales saturate at 448
    ties = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 7.0, -0.25, -5.0, 0.0, -0.0, 6.0, 4.0, 3.0, 2.0],
                    dtype=np.float32)
    x[7, :16] = ties
    return x


@pytest.mark.parametrize("g_factor", [1.0, 0.5])
def test_nv_quantise_f32_equals_oracle(gpu, g_factor):
    x = _nv_inputs()
    g = np.float32(np.abs(x[:5]).max() / np.float32(448 * 6)) * np.float32(g_factor)
    want_p, want_s = orc.quantize_nvfp4_fp32(x, g)
    p, s = quantize_nvfp4(torch.from_numpy(x).to(gpu), torch.tensor([g], dtype=torch.float32, device=gpu))
    assert np.array_equal(s.cpu().numpy(), want_s)
    assert np.array_equal(_canon(p.cpu().numpy()), _canon(want_p))
    assert (want_s == 0x7E).any() and (want_s == 0).any()       # saturated and vanished scales were both present


def test_nv_quantise_every_tie_of_the_grid(gpu):
    """g = 1/8 and a block amax of 6 give the scale byte of 8.0 and a divisor of exactly 1: the elements are
    rounded onto the grid as they stand, every tie to the even code."""
    x = np.zeros((2, 32), dtype=np.float32)
    x[0, :16] = [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0, -0.25, -5.0, 0.0, -0.0, -6.0, 4.0, 3.0, 2.0]
    x[1, 16:] = x[0, :16] * 2.0 ** -3          # the same through a scale byte of 1.0
    g = np.float32(0.125)
    p, s = quantize_nvfp4(torch.from_numpy(x).to(gpu), torch.tensor([g], dtype=torch.float32, device=gpu))
    want_p, want_s = orc.quantize_nvfp4_fp32(x, g)
    assert np.array_equal(s.cpu().numpy(), want_s) and want_s[0, 0] == 0x50 and want_s[1, 1] == 0x38
    assert np.array_equal(_canon(p.cpu().numpy()), _canon(want_p))
    codes = _canon(p.cpu().numpy())
    # 0.25 -> 0, 0.75 -> 1.0, 1.25 -> 1.0, 1.75 -> 2.0, 2.5 -> 2.0, 3.5 -> 4.0, 5.0 -> 4.0, 6.0 -> 6.0, ...
    assert list(codes[0, :16]) == [0, 2, 2, 4, 4, 6, 6, 7, 0, 14, 0, 0, 15, 6, 5, 4]
    assert list(codes[1, 16:]) == list(codes[0, :16])


def test_nv_quantise_bf16_equals_oracle(gpu):
    xb = torch.from_numpy(_nv_inputs()).to(torch.bfloat16)
    g = np.float32(float(xb.float().abs().max()) / (448 * 6))
    want_p, want_s = orc.quantize_nvfp4_fp32(xb.float().numpy(), g)
    p, s = quantize_nvfp4(xb.to(gpu), torch.tensor([g], dtype=torch.float32, device=gpu))
    assert np.array_equal(s.cpu().numpy(), want_s)
    assert np.array_equal(_canon(p.cpu().numpy()), _canon(want_p))


def test_nv_quantise_large_out_arguments_and_gemm(gpu):
    gen = torch.Generator(device=gpu).manual_seed(7)
    x = torch.randn((2048, 4096), generator=gen, device=gpu)
    w = torch.randn((256, 4096), generator=gen, device=gpu) * 0.02
    gx = (x.abs().amax() / (448 * 6)).reshape(1)
    gw = (w.abs().amax() / (448 * 6)).reshape(1)
    p, s = quantize_nvfp4(x, gx)
    rows = [0, 1, 1023, 2047]
    want_p, want_s = orc.quantize_nvfp4_fp32(x[rows].cpu().numpy(), gx.cpu().numpy()[0])
    assert np.array_equal(s[rows].cpu().numpy(), want_s)
    assert np.array_equal(_canon(p[rows].cpu().numpy()), _canon(want_p))
    p2, s2 = torch.empty_like(p), torch.empty_like(s)
    rp, rs = quantize_nvfp4(x, gx, packed=p2, scales=s2)
    assert rp is p2 and rs is s2 and torch.equal(p2, p) and torch.equal(s2, s)
    # quantised on the device, multiplied on the device, checked against the exact product of what was quantised
    b, b_s = quantize_nvfp4(w.to(torch.bfloat16), gw)
    a, a_s = p[:128].contiguous(), s[:128].contiguous()
    c = gemm_nvfp4_transposed_b(a, a_s, gx, b, b_s, gw)
    ref = orc.gemm_nvfp4_fp64(a.cpu().numpy(), a_s.cpu().numpy(), float(gx), b.cpu().numpy(), b_s.cpu().numpy(), float(gw))
    ok, rep = orc.check_bf16_against_fp64(c.view(torch.uint16).cpu().numpy(), ref, None, 4096)
    assert ok, rep
    # and the quantisation error is what 4-bit codes with a scale per 16 elements give
    dq = orc.dequantize_nvfp4(p[:64].cpu().numpy(), s[:64].cpu().numpy(), gx.cpu().numpy()[0])
    xs = x[:64].cpu().numpy()
    assert np.linalg.norm(dq - xs) / np.linalg.norm(xs) < 0.12
    with pytest.raises(ValueError, match="multiple of 16"):
        quantize_nvfp4(x[:, :40].contiguous(), gx)
    with pytest.raises(ValueError, match="global_scale"):
        quantize_nvfp4(x, gx.double())
    with pytest.raises(ValueError, match="dtype"):
        quantize_nvfp4(x.half(), gx)


def _non_finite_inputs():
    x = orc.randn((40, 256), seed=77)
    x[0, 5] = np.inf
    x[1, 40] = -np.inf
    x[2, 64] = np.nan
    x[3, 96:128] = np.nan
    x[4, 31], x[4, 32] = np.inf, np.nan          # neighbouring blocks
    x[5, 15], x[5, 16] = np.nan, 3.0             # the two halves of one 32-block
    x[6, 255] = np.inf
    x[7, :] = -np.inf
    x[8, 7] = 3.0e38                             # huge but finite: an ordinary block
    return x


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_quantisers_mark_blocks_with_non_finite_values(gpu, dtype):
    """A block that holds an infinity or a NaN gets the format's NaN scale byte and zero codes, bit for bit as the
    oracle defines it; every other block is untouched."""
    xt = torch.from_numpy(_non_finite_inputs()).to(dtype)
    x = xt.float().numpy()
    want_p, want_s = orc.quantize_mxfp4(x)
    p, s = quantize_mxfp4(xt.to(gpu))
    assert (want_s == 0xFF).sum() == 8 + 8
    assert np.array_equal(s.cpu().numpy(), want_s)
    assert np.array_equal(_canon(p.cpu().numpy()), _canon(want_p))
    g = np.float32(3.0 / (448 * 6))
    want_p, want_s = orc.quantize_nvfp4_fp32(x, g)
    p, s = quantize_nvfp4(xt.to(gpu), torch.tensor([g], dtype=torch.float32, device=gpu))
    assert (want_s == 0x7F).sum() == 9 + 16
    assert np.array_equal(s.cpu().numpy(), want_s)
    assert np.array_equal(_canon(p.cpu().numpy()), _canon(want_p))
