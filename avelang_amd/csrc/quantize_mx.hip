// Device-side MXFP4 quantiser: fp32 or bf16 rows -> packed E2M1 codes + E8M0 scales, the operand
// format the GEMM kernels consume.  This is the step that precedes the GEMM in an MLP (the
// reference has no counterpart; the benchmark's synthetic operands were so far quantised with
// torch ops).  HBM-bound: every input element is read once, 0.53 bytes per element are written.
//
// Recipe (identical to the CPU oracle's quantize_mxfp4): per 32 consecutive k,
//   scale = 2^(floor(log2(amax)) - 2), exponent clamped to [-127, 127], stored as E8M0;
//   an all-zero block gets scale byte 127 and zero codes;
//   a block that holds an infinity or a NaN gets scale byte 0xFF (the E8M0 NaN) and zero codes;
//   elements are divided by the scale and rounded to nearest-even onto the E2M1 grid, saturating.
//
// Four lanes share a block: each lane owns 8 consecutive elements (32 or 16 bytes in, one dword of
// codes out), the block amax is formed with two cross-lane exchanges.  The division and rounding are
// done by v_cvt_scalef32_pk_fp4_f32, whose scale operand contributes only its exponent.
#include "fp4_common.hpp"
#include "kernels.hpp"

namespace ave {
namespace {

// One 8-element piece of a block: amax over the four lanes that share the block, scale byte, codes.
__device__ inline void quantize_piece(const float (&v)[8], size_t i, uint8_t* packed, uint8_t* scales) {
  const unsigned amax = lane_xor_max_bits(lane_xor_max_bits(abs_max_bits(v), 1), 2);
  const int byte = mx_scale_byte(amax);
  const float scale = mx_scale_value(byte);
  unsigned codes = 0;
  codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(codes, v[0], v[1], scale, 0);
  codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(codes, v[2], v[3], scale, 1);
  codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(codes, v[4], v[5], scale, 2);
  codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(codes, v[6], v[7], scale, 3);
  reinterpret_cast<unsigned*>(packed)[i] = byte == 0xFF ? 0u : codes;   // a block with an infinity or a NaN
  if ((i & 3) == 0) scales[i >> 2] = (uint8_t)byte;
}

// T = float or __bf16.  A lane handles U pieces per trip, `stride` lanes apart, with all its loads
// issued before the first use: 32 bytes in flight per lane either way (U = 1 for fp32, 2 for bf16).
// PAD: the output rows are laid out for row_pieces_out * 8 elements, more than the row_pieces_in * 8 that x has; the
// blocks behind a row's end are written as blocks of zeros (zero codes under the scale 2^0), which add nothing to a
// GEMM over the padded length.  n_blocks counts the OUTPUT blocks.
template <typename T, int U, bool PAD>
__global__ __launch_bounds__(256) void quantize_mx_kernel(const T* __restrict__ x, uint8_t* __restrict__ packed,
                                                          uint8_t* __restrict__ scales, size_t n_blocks,
                                                          unsigned row_pieces_in, unsigned row_pieces_out) {
  // lane group of 4 -> one block of 32 elements
  const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  const size_t pieces = n_blocks * 4;   // a multiple of 4, and so is stride: the four lanes of a block stay together
  for (size_t i0 = gid; i0 < pieces; i0 += stride * U) {
    float v[U][8];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t i = i0 + (size_t)u * stride;
      size_t in = i;                 // the piece of x that output piece i is made from
      bool real = true;
      if constexpr (PAD) {
        const size_t row = i / row_pieces_out;
        const unsigned col = (unsigned)(i - row * row_pieces_out);
        real = col < row_pieces_in;
        in = row * row_pieces_in + col;
      }
      if (PAD && !real) {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[u][j] = 0.0f;
      } else if (i < pieces) {
        if constexpr (sizeof(T) == 4) {
          const v4f* src = reinterpret_cast<const v4f*>(x) + in * 2;
          const v4f a = src[0], b = src[1];
          v[u][0] = a[0]; v[u][1] = a[1]; v[u][2] = a[2]; v[u][3] = a[3];
          v[u][4] = b[0]; v[u][5] = b[1]; v[u][6] = b[2]; v[u][7] = b[3];
        } else {
          const v4i raw = reinterpret_cast<const v4i*>(x)[in];
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
      if (i < pieces) quantize_piece(v[u], i, packed, scales);   // uniform over the four lanes of a block
    }
  }
}

template <typename T>
hipError_t launch(const void* x, uint8_t* packed, uint8_t* scales, size_t rows, int k, int k_padded, hipStream_t s) {
  const size_t n_blocks = rows * (size_t)(k_padded / 32);
  if (n_blocks == 0) return hipSuccess;
  const size_t lanes = n_blocks * 4;
  size_t grid = (lanes + 255) / 256;
  if (grid > 256 * 16) grid = 256 * 16;   // grid-stride beyond 16 workgroups per CU
  constexpr int kPieces = sizeof(T) == 4 ? 1 : 2;   // fp32 gains nothing from a second piece (28.0 vs 28.4 us)
  if (k_padded == k)
    hipLaunchKernelGGL((quantize_mx_kernel<T, kPieces, false>), dim3((unsigned)grid), dim3(256), 0, s,
                       static_cast<const T*>(x), packed, scales, n_blocks, 0u, 0u);
  else
    hipLaunchKernelGGL((quantize_mx_kernel<T, kPieces, true>), dim3((unsigned)grid), dim3(256), 0, s,
                       static_cast<const T*>(x), packed, scales, n_blocks, (unsigned)(k / 8), (unsigned)(k_padded / 8));
  return hipGetLastError();
}

}  // namespace

hipError_t launch_quantize_mx(const void* x, int is_bf16, uint8_t* packed, uint8_t* scales, size_t rows, int k,
                              int k_padded, hipStream_t s) {
  return is_bf16 ? launch<__bf16>(x, packed, scales, rows, k, k_padded, s)
                 : launch<float>(x, packed, scales, rows, k, k_padded, s);
}

}  // namespace ave
