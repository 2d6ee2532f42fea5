#!/usr/bin/env python3
"""Writes the golden fixtures of this directory.

The reference holds no vectors for FP4 GEMMs, so these come from this repository's CPU oracle
(``oracle/fp4_oracle.py``); ``tests/test_oracle_formats.py`` re-derives every expected value with an
independent pure-Python ``fractions`` implementation before trusting them.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import fp4_oracle as orc  # noqa: E402


def main():
    # MXFP4 32x48x64, wide-ranging scales
    a, a_s = orc.quantize_mxfp4(orc.activations_with_outliers(32, 64, seed=11, frac=0.05))
    b, b_s = orc.quantize_mxfp4(orc.randn((48, 64), seed=12, std=0.02))
    c = orc.f64_to_bf16_bits(orc.gemm_mxfp4_fp64(a, a_s, b, b_s))
    np.savez(os.path.join(HERE, "mxfp4_32x48x64.npz"), a=a, a_scale=a_s, b=b, b_scale=b_s, c_bf16_bits=c)
    # NVFP4 32x48x64
    a, a_s, a_g = orc.quantize_nvfp4(orc.randn((32, 64), seed=13))
    b, b_s, b_g = orc.quantize_nvfp4(orc.randn((48, 64), seed=14, std=0.02))
    c = orc.f64_to_bf16_bits(orc.gemm_nvfp4_fp64(a, a_s, a_g, b, b_s, b_g))
    np.savez(os.path.join(HERE, "nvfp4_32x48x64.npz"), a=a, a_scale=a_s, a_global=np.float32(a_g), b=b, b_scale=b_s,
             b_global=np.float32(b_g), c_bf16_bits=c)
    # grouped MXFP4: 3 experts (one empty), N=32, K=64
    ro = np.array([0, 20, 20, 45], dtype=np.int32)
    a, a_s = orc.quantize_mxfp4(orc.randn((45, 64), seed=15))
    ws = [orc.quantize_mxfp4(orc.randn((32, 64), seed=16 + i, std=0.02)) for i in range(3)]
    b, b_s = np.stack([w[0] for w in ws]), np.stack([w[1] for w in ws])
    c = orc.f64_to_bf16_bits(orc.grouped_gemm_mxfp4_fp64(a, a_s, b, b_s, ro))
    np.savez(os.path.join(HERE, "grouped_mxfp4_45x32x64.npz"), a=a, a_scale=a_s, b=b, b_scale=b_s, row_offsets=ro,
             c_bf16_bits=c)
    # K = 512, so that the LDS-staged kernels take them (K % 512 == 0): MXFP4 72x40 (the narrow-tile and 256 x 256
    # kernels; the first 16 rows alone go to the weight-streaming kernel), NVFP4 24x40 (the LDS rings)
    a, a_s = orc.quantize_mxfp4(orc.activations_with_outliers(72, 512, seed=21, frac=0.02))
    b, b_s = orc.quantize_mxfp4(orc.randn((40, 512), seed=22, std=0.02))
    c = orc.f64_to_bf16_bits(orc.gemm_mxfp4_fp64(a, a_s, b, b_s))
    np.savez_compressed(os.path.join(HERE, "mxfp4_72x40x512.npz"), a=a, a_scale=a_s, b=b, b_scale=b_s, c_bf16_bits=c)
    a, a_s, a_g = orc.quantize_nvfp4(orc.randn((24, 512), seed=23))
    b, b_s, b_g = orc.quantize_nvfp4(orc.randn((40, 512), seed=24, std=0.02))
    c = orc.f64_to_bf16_bits(orc.gemm_nvfp4_fp64(a, a_s, a_g, b, b_s, b_g))
    np.savez_compressed(os.path.join(HERE, "nvfp4_24x40x512.npz"), a=a, a_scale=a_s, a_global=np.float32(a_g), b=b,
                        b_scale=b_s, b_global=np.float32(b_g), c_bf16_bits=c)
    # K with a tail: 736 = 512 + 7 blocks of 32 (the LDS-staged kernel's K-tail form above 64 rows; the first 16 rows
    # alone go to the register form of the weight-streaming kernel, whose last step then holds three blocks), and
    # NVFP4 with K = 320 (a multiple of 64 but not of 256: the f16-staged tile kernel)
    a, a_s = orc.quantize_mxfp4(orc.activations_with_outliers(72, 736, seed=31, frac=0.02))
    b, b_s = orc.quantize_mxfp4(orc.randn((40, 736), seed=32, std=0.02))
    c = orc.f64_to_bf16_bits(orc.gemm_mxfp4_fp64(a, a_s, b, b_s))
    np.savez_compressed(os.path.join(HERE, "mxfp4_72x40x736.npz"), a=a, a_scale=a_s, b=b, b_scale=b_s, c_bf16_bits=c)
    a, a_s, a_g = orc.quantize_nvfp4(orc.randn((72, 320), seed=33))
    b, b_s, b_g = orc.quantize_nvfp4(orc.randn((40, 320), seed=34, std=0.02))
    c = orc.f64_to_bf16_bits(orc.gemm_nvfp4_fp64(a, a_s, a_g, b, b_s, b_g))
    np.savez_compressed(os.path.join(HERE, "nvfp4_72x40x320.npz"), a=a, a_scale=a_s, a_global=np.float32(a_g), b=b,
                        b_scale=b_s, b_global=np.float32(b_g), c_bf16_bits=c)
    # the device NVFP4 quantiser's recipe (fp32 steps, given per-tensor scale): input, scale, codes and scale bytes
    x = orc.activations_with_outliers(8, 64, seed=25, frac=0.05)
    x[1, 16:32] = 0.0
    g = np.float32(np.abs(x).max() / np.float32(448 * 6)) * np.float32(0.5)
    packed, sb = orc.quantize_nvfp4_fp32(x, g)
    np.savez(os.path.join(HERE, "quantize_nvfp4_8x64.npz"), x=x, global_scale=g, packed=packed, scales=sb)


if __name__ == "__main__":
    main()
