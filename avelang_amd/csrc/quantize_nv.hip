// Device-side NVFP4 quantiser: fp32 or bf16 rows -> packed E2M1 codes + one E4M3 scale per 16 consecutive k, for a
// per-tensor fp32 scale `g` that the caller supplies (calibrated ahead of time, e.g. amax / (448 * 6)): the
// operand format of the NVFP4 GEMM kernels.  HBM-bound: every element is read once, 0.5625 bytes per element
// are written.
//
// Recipe, every step one IEEE fp32 operation (the CPU oracle's quantize_nvfp4_fp32 does the same steps; the
// quotients are formed from one reciprocal per block plus a correction step that yields the same codes):
//   u = min((amax / 6) / g, 448);  scale byte = E4M3(u), round to nearest even;
//   d = decode(scale byte) * g;  codes = E2M1(x / d), round to nearest even, saturating;  d == 0: zero codes;
//   a block that holds an infinity or a NaN gets scale byte 0x7F (the E4M3 NaN) and zero codes.
//
// Two lanes share a block: each owns 8 consecutive elements (32 or 16 bytes in, one dword of codes out), the
// block amax takes one cross-lane exchange.
#include "fp4_common.hpp"
#include "kernels.hpp"

namespace ave {
namespace {

#pragma clang fp contract(off)   // every product and quotient below is rounded on its own

__device__ inline void quantize_nv_piece(const float (&v)[8], float g, size_t i, uint8_t* packed, uint8_t* scales) {
  const unsigned amax_bits = lane_xor_max_bits(abs_max_bits(v), 1);
  const float amax = __builtin_bit_cast(float, amax_bits);
  float u = (amax / 6.0f) / g;
  u = u < 448.0f ? u : 448.0f;
  // a block that holds an infinity or a NaN: scale byte 0x7F, the E4M3 NaN, and (d is NaN) zero codes
  const int byte = non_finite_bits(amax_bits) ? 0x7F : (__builtin_amdgcn_cvt_pk_fp8_f32(u, u, 0, false) & 0xFF);
  const float d = __builtin_amdgcn_cvt_f32_fp8(byte, 0) * g;
  unsigned codes = 0;
  if (d > 0.f) {
    float q[8];
    if (d >= 0x1p-100f && d <= 0x1p100f) {
      // One correctly rounded reciprocal per block, then per element a product and one correction step:
      // with y = RN(1 / d) and q0 = RN(x y), q0 + (x - q0 d) y rounded once IS RN(x / d) (Markstein) as long as
      // nothing underflows or overflows on the way -- which the range check on d guarantees wherever the
      // quotient is near a rounding boundary of the E2M1 grid (0.25 .. 5); further out both ways of
      // computing it give code 0, or saturate, alike.
      const float y = 1.0f / d;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float q0 = v[j] * y;
        const float rem = __builtin_fmaf(-q0, d, v[j]);
        const float q1 = __builtin_fmaf(rem, y, q0);
        q[j] = (q1 == q1) ? q1 : q0;   // q0 = +-inf gives rem = -+inf and q1 = NaN: keep the saturating infinity
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) q[j] = v[j] / d;
    }
    codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(codes, q[0], q[1], 1.0f, 0);
    codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(codes, q[2], q[3], 1.0f, 1);
    codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(codes, q[4], q[5], 1.0f, 2);
    codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(codes, q[6], q[7], 1.0f, 3);
  }
  reinterpret_cast<unsigned*>(packed)[i] = codes;
  if ((i & 1) == 0) scales[i >> 1] = (uint8_t)byte;
}

// T = float or __bf16; pieces 2b and 2b + 1 (8 elements each) form block b.  A lane handles U pieces per trip,
// `stride` lanes apart, with all its loads issued before the first use (U = 1 for fp32, 2 for bf16: 32 bytes in
// flight per lane either way).
template <typename T, int U>
__global__ __launch_bounds__(256) void quantize_nv_kernel(const T* __restrict__ x, const float* __restrict__ global_scale,
                                                          uint8_t* __restrict__ packed, uint8_t* __restrict__ scales,
                                                          size_t n_blocks) {
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;   // even: the two lanes of a block stay together
  const size_t pieces = n_blocks * 2;
  const float g = global_scale[0];
  for (size_t i0 = gid; i0 < pieces; i0 += stride * U) {
    float v[U][8];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t i = i0 + (size_t)u * stride;
      if (i < pieces) {
        if constexpr (sizeof(T) == 4) {
          const v4f* src = reinterpret_cast<const v4f*>(x) + i * 2;
          const v4f a = src[0], b = src[1];
          v[u][0] = a[0]; v[u][1] = a[1]; v[u][2] = a[2]; v[u][3] = a[3];
          v[u][4] = b[0]; v[u][5] = b[1]; v[u][6] = b[2]; v[u][7] = b[3];
        } else {
          const v4i raw = reinterpret_cast<const v4i*>(x)[i];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            v[u][2 * j] = __builtin_bit_cast(float, (unsigned)raw[j] << 16);
            v[u][2 * j + 1] = __builtin_bit_cast(float, (unsigned)raw[j] & 0xFFFF0000u);
          }
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t i = i0 + (size_t)u * stride;
      if (i < pieces) quantize_nv_piece(v[u], g, i, packed, scales);   // uniform over the two lanes of a block
    }
  }
}

template <typename T>
hipError_t launch(const void* x, const float* g, uint8_t* packed, uint8_t* scales, size_t n_blocks, hipStream_t s) {
  if (n_blocks == 0) return hipSuccess;
  const size_t lanes = n_blocks * 2;
  size_t grid = (lanes + 255) / 256;
  if (grid > 256 * 16) grid = 256 * 16;
  constexpr int kPieces = sizeof(T) == 4 ? 1 : 2;
  hipLaunchKernelGGL((quantize_nv_kernel<T, kPieces>), dim3((unsigned)grid), dim3(256), 0, s, static_cast<const T*>(x), g,
                     packed, scales, n_blocks);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_quantize_nv(const void* x, int is_bf16, const float* global_scale, uint8_t* packed, uint8_t* scales,
                              size_t n_blocks, hipStream_t s) {
  return is_bf16 ? launch<__bf16>(x, global_scale, packed, scales, n_blocks, s)
                 : launch<float>(x, global_scale, packed, scales, n_blocks, s);
}

}  // namespace ave
