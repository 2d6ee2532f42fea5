// Diagnostic: the rate at which this GPU sustains v_mfma_scale_f32_32x32x64_f8f6f4 on FP4 operands when
// nothing else runs -- eight wavefronts per workgroup (two per SIMD), eight independent accumulators per
// wave fed from four "B" and two "A" fragments as in the tile kernel, operands taken once from a caller's
// buffer and kept in registers.  The clock under this load depends on how many operand bits toggle between
// consecutive MFMAs: fragments of zeros run near the published peak, fragments of real quantised data far
// below it.  This measured rate, not the published one, is the ceiling a GEMM on that data can approach.
#include "fp4_common.hpp"
#include "kernels.hpp"

namespace ave {
namespace {

constexpr int kThreads = 512, kFragsPerLane = 6;

__global__ __launch_bounds__(kThreads) void mfma_rate_kernel(const v4i* codes, size_t n_frags, int iters, float* sink) {
  const size_t lane_id = (size_t)blockIdx.x * kThreads + threadIdx.x;
  v4i a[2], b[4];
#pragma unroll
  for (int i = 0; i < 2; ++i) a[i] = codes[(lane_id * kFragsPerLane + i) % n_frags];
#pragma unroll
  for (int i = 0; i < 4; ++i) b[i] = codes[(lane_id * kFragsPerLane + 2 + i) % n_frags];
  v16f acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = v16f{};
  const int one = 0x7f7f7f7f;   // four E8M0 bytes of 2^0
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = mfma32<0, 0>(b[i], a[j], acc[i][j], one, one);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) s += acc[i][j][e];
  if (s == 12345.678f) sink[0] = s;   // keeps the accumulators alive; practically never true
}

// The same loop for the f16 MFMA that the NVFP4 kernels multiply with (v_mfma_f32_32x32x16_f16): the operands are
// the caller's codes dequantised to f16 once (E2M1 x 1.0), eight elements per lane and MFMA.
__global__ __launch_bounds__(kThreads) void mfma_rate_f16_kernel(const v4i* codes, size_t n_frags, int iters, float* sink) {
  const size_t lane_id = (size_t)blockIdx.x * kThreads + threadIdx.x;
  v8h a[2], b[4];
#pragma unroll
  for (int i = 0; i < 2; ++i) a[i] = dequant8((unsigned)codes[(lane_id * kFragsPerLane + i) % n_frags][0], (_Float16)1.0f);
#pragma unroll
  for (int i = 0; i < 4; ++i) b[i] = dequant8((unsigned)codes[(lane_id * kFragsPerLane + 2 + i) % n_frags][0], (_Float16)1.0f);
  v16f acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = v16f{};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b[i], a[j], acc[i][j], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) s += acc[i][j][e];
  if (s == 12345.678f) sink[0] = s;
}

// Second probe: a plain streaming read.  Every lane loads 16 bytes per trip, consecutive lanes consecutive
// addresses, four loads in flight per lane; nothing is computed beyond an OR that keeps the loads alive and nothing
// is written.  Over a buffer larger than the last-level cache this is the rate at which this GPU delivers bytes from
// HBM to a kernel that does nothing else: the floor under any weight-streaming (decode) GEMM of the same bytes.
// With `dst` the kernel then writes n16_dst 16-byte pieces derived from what it read, consecutive lanes consecutive
// addresses: the same floor for a GEMM that also has a result of that size to store.
__global__ __launch_bounds__(256) void stream_read_kernel(const v4i* __restrict__ src, size_t n16, int* sink, v4i* dst,
                                                          size_t n16_dst) {
  const size_t stride = (size_t)gridDim.x * 256;
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  v4i acc = {0, 0, 0, 0};
  for (; i + 3 * stride < n16; i += 4 * stride) {
    const v4i x0 = __builtin_nontemporal_load(src + i), x1 = __builtin_nontemporal_load(src + i + stride);
    const v4i x2 = __builtin_nontemporal_load(src + i + 2 * stride), x3 = __builtin_nontemporal_load(src + i + 3 * stride);
    acc |= x0 | x1 | x2 | x3;
  }
  for (; i < n16; i += stride) acc |= __builtin_nontemporal_load(src + i);
  if ((acc[0] | acc[1] | acc[2] | acc[3]) == 0x5A5A5A5B) sink[0] = acc[0];   // practically never true
  if (dst)
    for (size_t j = (size_t)blockIdx.x * 256 + threadIdx.x; j < n16_dst; j += stride) dst[j] = acc;
}

}  // namespace

hipError_t launch_stream_read(const void* src, size_t bytes, int workgroups, int* sink, void* dst, size_t dst_bytes,
                              hipStream_t s) {
  hipLaunchKernelGGL(stream_read_kernel, dim3((unsigned)workgroups), dim3(256), 0, s, reinterpret_cast<const v4i*>(src),
                     bytes / 16, sink, reinterpret_cast<v4i*>(dst), dst_bytes / 16);
  return hipGetLastError();
}

double mfma_rate_flop(int workgroups, int iters) {
  return (double)workgroups * (kThreads / 64) * (double)iters * 8.0 * 2.0 * 32 * 32 * 64;
}
double mfma_rate_f16_flop(int workgroups, int iters) {
  return (double)workgroups * (kThreads / 64) * (double)iters * 8.0 * 2.0 * 32 * 32 * 16;
}

hipError_t launch_mfma_rate_f16(const uint8_t* codes, size_t bytes, int workgroups, int iters, float* sink, hipStream_t s) {
  hipLaunchKernelGGL(mfma_rate_f16_kernel, dim3((unsigned)workgroups), dim3(kThreads), 0, s,
                     reinterpret_cast<const v4i*>(codes), bytes / 16, iters, sink);
  return hipGetLastError();
}

hipError_t launch_mfma_rate(const uint8_t* codes, size_t bytes, int workgroups, int iters, float* sink,
                            hipStream_t s) {
  hipLaunchKernelGGL(mfma_rate_kernel, dim3((unsigned)workgroups), dim3(kThreads), 0, s,
                     reinterpret_cast<const v4i*>(codes), bytes / 16, iters, sink);
  return hipGetLastError();
}

}  // namespace ave
