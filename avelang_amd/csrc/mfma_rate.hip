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

}  // namespace

double mfma_rate_flop(int workgroups, int iters) {
  return (double)workgroups * (kThreads / 64) * (double)iters * 8.0 * 2.0 * 32 * 32 * 64;
}

hipError_t launch_mfma_rate(const uint8_t* codes, size_t bytes, int workgroups, int iters, float* sink,
                            hipStream_t s) {
  hipLaunchKernelGGL(mfma_rate_kernel, dim3((unsigned)workgroups), dim3(kThreads), 0, s,
                     reinterpret_cast<const v4i*>(codes), bytes / 16, iters, sink);
  return hipGetLastError();
}

}  // namespace ave
