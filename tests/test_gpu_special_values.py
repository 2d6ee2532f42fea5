"""NaN scale bytes (E8M0 0xFF, E4M3 0x7F / 0xFF) poison exactly the rows and columns they belong to, in every
kernel, as they do in the oracle; everything else keeps its value."""
import numpy as np
import pytest

from oracle import fp4_oracle as orc
from tests import helpers as H

pytestmark = pytest.mark.gpu
GENERIC, TILE, DECODE, NARROW, TILE_STREAMED = 1, 2, 3, 4, 6


@pytest.mark.parametrize("m,n,k,variant", [(40, 48, 96, GENERIC), (300, 260, 512, TILE), (16, 64, 1024, DECODE),
                                           (48, 64, 2048, DECODE), (16, 64, 384, DECODE),
                                           (300, 260, 2048, TILE),            # scale rows in 64-byte chunks
                                           (300, 260, 768, TILE),             # scales per stage
                                           (100, 300, 1024, NARROW), (200, 130, 1056, NARROW),
                                           (2100, 9000, 512, TILE_STREAMED)])  # more tiles than compute units: touches
def test_mxfp4_nan_scale_bytes(gpu, m, n, k, variant):
    a, a_s = H.mx_operand(m, k, seed=1)
    b, b_s = H.mx_operand(n, k, seed=2, std=0.05)
    clean = H.run_mx(gpu, a, a_s, b, b_s, variant=variant)
    a_s, b_s = a_s.copy(), b_s.copy()
    a_s[3, 1] = 255
    b_s[5, 0] = 255
    got = H.run_mx(gpu, a, a_s, b, b_s, variant=variant)
    nan = np.isnan(orc.bf16_bits_to_f32(got))
    want_nan = np.isnan(orc.gemm_mxfp4_fp64(a, a_s, b, b_s))
    assert want_nan[3].all() and want_nan[:, 5].all() and want_nan.sum() == m + n - 1
    assert np.array_equal(nan, want_nan)
    assert np.array_equal(got[~nan], clean[~nan])


def test_mxfp4_nan_scale_bytes_in_blocked_scale_tensors(gpu):
    import torch
    from avelang_amd import gemm_mxfp4_blocked_scales_transposed_b, scales_to_blocked

    for m, n, k in ((300, 260, 1024), (16, 200, 2048)):   # 256 x 256 kernel, weight-streaming kernel
        a, a_s = H.mx_operand(m, k, seed=31)
        b, b_s = H.mx_operand(n, k, seed=32, std=0.05)
        a_n, b_n = a_s.copy(), b_s.copy()
        a_n[3, 1] = 255
        b_n[5, -1] = 255
        res = []
        for sa, sb in ((a_s, b_s), (a_n, b_n)):
            c = gemm_mxfp4_blocked_scales_transposed_b(H.to_dev(a, gpu), scales_to_blocked(H.to_dev(sa, gpu)),
                                                       H.to_dev(b, gpu), scales_to_blocked(H.to_dev(sb, gpu)))
            torch.cuda.synchronize()
            res.append(H.bits(c))
        clean, got = res
        nan = np.isnan(orc.bf16_bits_to_f32(got))
        want_nan = np.isnan(orc.gemm_mxfp4_fp64(a, a_n, b, b_n))
        assert want_nan.sum() == m + n - 1 and np.array_equal(nan, want_nan)
        assert np.array_equal(got[~nan], clean[~nan])


@pytest.mark.parametrize("m,n,k,variant", [(300, 260, 736, TILE), (70, 40, 544, TILE), (260, 300, 992, TILE),
                                           (16, 64, 672, DECODE), (9, 100, 160, DECODE)])
def test_mxfp4_nan_scale_bytes_in_the_k_tail(gpu, m, n, k, variant):
    """K with a tail behind the last multiple of 512 (tile kernel) or of 128 (register decode kernel): a NaN byte in
    the tail's last block poisons its row, and NaN bytes at the START of a row -- the bytes that lie right behind the
    previous row's tail in memory -- poison that row alone, not the row in front of it."""
    a, a_s = H.mx_operand(m, k, seed=11)
    b, b_s = H.mx_operand(n, k, seed=12, std=0.05)
    clean = H.run_mx(gpu, a, a_s, b, b_s, variant=variant)
    a_s, b_s = a_s.copy(), b_s.copy()
    a_s[3, -1] = 255
    b_s[5, -1] = 255
    b_s[8, :3] = 255
    a_s[6, 0] = 255
    got = H.run_mx(gpu, a, a_s, b, b_s, variant=variant)
    nan = np.isnan(orc.bf16_bits_to_f32(got))
    want_nan = np.isnan(orc.gemm_mxfp4_fp64(a, a_s, b, b_s))
    assert want_nan.sum() == 2 * n + 2 * m - 4
    assert np.array_equal(nan, want_nan)
    assert np.array_equal(got[~nan], clean[~nan])


@pytest.mark.parametrize("variant", [GENERIC, TILE])
def test_nvfp4_nan_scale_bytes(gpu, variant):
    m, n, k = 64, 72, 256
    a, a_s, a_g = H.nv_operand(m, k, seed=3)
    b, b_s, b_g = H.nv_operand(n, k, seed=4, std=0.05)
    clean = H.run_nv(gpu, a, a_s, a_g, b, b_s, b_g, variant=variant)
    a_s, b_s = a_s.copy(), b_s.copy()
    a_s[3, 1] = 0x7F
    b_s[5, 0] = 0xFF
    got = H.run_nv(gpu, a, a_s, a_g, b, b_s, b_g, variant=variant)
    nan = np.isnan(orc.bf16_bits_to_f32(got))
    want_nan = np.isnan(orc.gemm_nvfp4_fp64(a, a_s, a_g, b, b_s, b_g))
    assert want_nan.sum() == m + n - 1 and np.array_equal(nan, want_nan)
    assert np.array_equal(got[~nan], clean[~nan])
