// Shared device-side helpers for the gfx950 FP4 GEMM kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ave {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef unsigned short v4us __attribute__((ext_vector_type(4)));
typedef unsigned short v8us __attribute__((ext_vector_type(8)));

constexpr int kMxBlock = 32;  // K elements per E8M0 scale
constexpr int kNvBlock = 16;  // K elements per E4M3 scale

// Operand/result lane maps of the CDNA4 scaled MFMAs with FP4 sources (cbsz = blgp = 4),
// established on hardware with random operands:
//   v_mfma_scale_f32_32x32x64_f8f6f4:  lane l supplies row (l % 32), K elements 32*(l/32) .. +31
//     (16 bytes, low nibble = even k, in the first 4 of the 8 source VGPRs) and ONE E8M0 byte
//     (byte `opsel` of its scale VGPR) for exactly those 32 elements.
//     D register t of lane l is D[8*(t/4) + 4*(l/32) + t%4][l % 32]  (row from srcA, col from srcB).
//   v_mfma_scale_f32_16x16x128_f8f6f4: lane l supplies row (l % 16), K elements 32*(l/16) .. +31;
//     D register t of lane l is D[4*(l/16) + t][l % 16].
constexpr int kFmtFp4 = 4;

template <int OPA, int OPB>
__device__ inline v16f mfma32(v4i a, v4i b, v16f c, int sa, int sb) {
  v8i a8 = {a[0], a[1], a[2], a[3], 0, 0, 0, 0};
  v8i b8 = {b[0], b[1], b[2], b[3], 0, 0, 0, 0};
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, c, kFmtFp4, kFmtFp4, OPA, sa, OPB, sb);
}

template <int OPA, int OPB>
__device__ inline v4f mfma16(v4i a, v4i b, v4f c, int sa, int sb) {
  v8i a8 = {a[0], a[1], a[2], a[3], 0, 0, 0, 0};
  v8i b8 = {b[0], b[1], b[2], b[3], 0, 0, 0, 0};
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a8, b8, c, kFmtFp4, kFmtFp4, OPA, sa, OPB, sb);
}

// fp32 -> bf16 bits, round to nearest even (v_cvt_pk_bf16_f32 on gfx950).
__device__ inline unsigned pack_bf16x2(float lo, float hi) {
  v2bf p = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(unsigned, p);
}
__device__ inline unsigned short to_bf16(float x) {
  __bf16 b = (__bf16)x;
  return __builtin_bit_cast(unsigned short, b);
}

// The SwiGLU gate function x / (1 + exp(-x)), evaluated in fp32 on fp32 accumulators by every kernel that fuses
// it: v_exp_f32 and v_rcp_f32 (1 ulp each) instead of the library exponential and an IEEE division -- five
// instructions instead of about twenty, with an error of a few fp32 ulps under a result that is rounded to bf16.
__device__ inline float silu(float x) {
  return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x));
}

// Largest magnitude of eight values as a bit pattern.  For non-negative IEEE numbers the unsigned order of the bit
// patterns is the numeric order, and every infinity and NaN sorts above every finite number: one chain of integer
// maxima finds the block maximum AND tells whether the block holds a non-finite value (result >= 0x7F800000), which
// a chain of fmaxf would swallow.
__device__ inline unsigned abs_max_bits(const float (&v)[8]) {
  unsigned m = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const unsigned b = __builtin_bit_cast(unsigned, v[j]) & 0x7FFFFFFFu;
    m = m > b ? m : b;
  }
  return m;
}
__device__ inline unsigned lane_xor_max_bits(unsigned v, int mask) {
  const unsigned o = (unsigned)__shfl_xor((int)v, mask, 64);
  return v > o ? v : o;
}
__device__ inline bool non_finite_bits(unsigned amax_bits) { return amax_bits >= 0x7F800000u; }

// MXFP4 block scale of the quantiser: E8M0 byte for a block whose largest magnitude has the bit pattern
// `amax_bits` -- the biased exponent minus 2, clamped; zero -> 127, subnormal -> 0; a block that holds an infinity or
// a NaN -> 0xFF, the E8M0 NaN (its codes are written as zeros, and every GEMM result that uses the block is NaN) --
// and the power of two a byte stands for.
__device__ inline int mx_scale_byte(unsigned amax_bits) {
  const int field = (int)(amax_bits >> 23);
  int byte = field - 2;
  byte = byte < 0 ? 0 : (byte > 254 ? 254 : byte);
  if (field == 0) byte = amax_bits == 0 ? 127 : 0;
  if (field == 0xFF) byte = 0xFF;
  return byte;
}
__device__ inline float mx_scale_value(int byte) {
  return __builtin_bit_cast(float, byte == 0 ? 0x00400000u : (unsigned)byte << 23);   // 2^(byte-127)
}

// two E4M3 bytes (bits 0-7 and 8-15 of x) -> packed f16 {s0, s1}, exact
__device__ inline v2h scale_pair(int x) { return __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(x, 1.0f, false); }

// eight E2M1 codes times one f16 scale; the splat of `s` folds into the op_sel bits of v_pk_mul_f16
__device__ inline v8h dequant8(unsigned codes, _Float16 s) {
  const v2h s2 = {s, s};
  v2h p0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 1.0f, 0) * s2;
  v2h p1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 1.0f, 1) * s2;
  v2h p2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 1.0f, 2) * s2;
  v2h p3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 1.0f, 3) * s2;
  return v8h{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
}

// 16-byte store that is written through to memory (system scope): the line is not left modified in the L2, so the
// write-back at the kernel's end has nothing to do for it
__device__ inline void store16_write_through(void* p, v4i v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" ::"v"(p), "v"(v) : "memory");
}

// rotate right by 8*n bits (n in 0..3): byte n of x becomes byte 0
__device__ inline int rotr_bytes(int x, int n) { return (int)__builtin_amdgcn_alignbit((unsigned)x, (unsigned)x, (unsigned)(8 * n)); }

// 32-bit buffer resource over [base, base+bytes): raw mode, out-of-range loads return 0,
// out-of-range stores are dropped.
__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* base, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

}  // namespace ave
