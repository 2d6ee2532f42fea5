// Shape-agnostic FP4 GEMM kernels for gfx950: one wavefront per 32x32 tile of C, operands
// loaded straight from global memory in MFMA operand order, every access guarded.
// They exist so that any (M, N, K) the format allows has a device path; the LDS-staged
// kernels take over for the aligned shapes that matter for throughput.
#include "fp4_common.hpp"
#include "kernels.hpp"
#include "tile_map.hpp"

namespace ave {

// grid: ceil(N/128) * m_tiles workgroups in one dimension (workgroup id = by * n_blocks + bx: a second grid
// dimension would cap the m-tiles at 65535); block 256 = 4 waves, wave w owns columns [128*bx + 32*w, +32).
// SWIGLU: B holds 2N rows (gate rows, then up rows); a second accumulator takes the up projection of
// the same columns and C = silu(gate) * up.
template <bool SWIGLU>
__global__ __launch_bounds__(256) void mx_generic_kernel(MxArgs p, unsigned n_blocks) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 31, h = lane >> 5;
  const int bx = (int)(blockIdx.x % n_blocks), by = (int)(blockIdx.x / n_blocks);
  int m_begin = by * 32, m_end = p.M, expert = 0;
  if (p.row_offsets) {
    if (!locate_group_tile(p.row_offsets, p.E, p.M, 32, by, expert, m_begin, m_end)) return;
  }
  const int n0 = bx * 128 + wave * 32;
  if (n0 >= p.N || m_begin >= m_end) return;
  const size_t row_bytes = (size_t)p.K / 2, row_scales = (size_t)p.K / kMxBlock;
  const size_t expert_rows = (size_t)expert * (SWIGLU ? 2 : 1) * p.N;   // an expert holds N, or N gate + N up rows
  const uint8_t* B = p.B + expert_rows * row_bytes;
  const uint8_t* Bs = p.Bs + expert_rows * row_scales;
  const int m = m_begin + r, n = n0 + r;
  const bool mv = m < m_end, nv = n < p.N;
  const uint8_t* a_row = p.A + (size_t)m * row_bytes;
  const uint8_t* as_row = p.As + (size_t)m * row_scales;
  const uint8_t* b_row = B + (size_t)n * row_bytes;
  const uint8_t* bs_row = Bs + (size_t)n * row_scales;
  const uint8_t* u_row = b_row + (size_t)p.N * row_bytes;      // SWIGLU: the up projection's row
  const uint8_t* us_row = bs_row + (size_t)p.N * row_scales;
  const int kblocks = p.K / kMxBlock;
  v16f acc = {}, acc_up = {};
  for (int kb0 = 0; kb0 < kblocks; kb0 += 2) {
    const int kb = kb0 + h;
    const bool kv = kb < kblocks;
    v4i a = {0, 0, 0, 0}, b = {0, 0, 0, 0}, u = {0, 0, 0, 0};
    int sa = 127, sb = 127, su = 127;
    if (mv && kv) {
      a = *reinterpret_cast<const v4i*>(a_row + (size_t)kb * 16);
      sa = as_row[kb];
    }
    if (nv && kv) {
      b = *reinterpret_cast<const v4i*>(b_row + (size_t)kb * 16);
      sb = bs_row[kb];
      if (SWIGLU) {
        u = *reinterpret_cast<const v4i*>(u_row + (size_t)kb * 16);
        su = us_row[kb];
      }
    }
    // srcA carries B's rows (n), srcB carries A's rows (m): D[n_local][m_local]
    acc = mfma32<0, 0>(b, a, acc, sb, sa);
    if (SWIGLU) acc_up = mfma32<0, 0>(u, a, acc_up, su, sa);
  }
  if (mv) {
    uint16_t* c_row = p.C + (size_t)m * p.N;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      const int nn = n0 + 8 * (t / 4) + 4 * h + (t % 4);
      const float v = SWIGLU ? silu(acc[t]) * acc_up[t] : acc[t];
      if (nn < p.N) c_row[nn] = to_bf16(v);
    }
  }
}

// E4M3 byte -> fp32 (v_cvt_f32_fp8; gfx950 decodes the OCP "fn" encoding).
__device__ inline float e4m3_to_f32(int byte) { return __builtin_amdgcn_cvt_f32_fp8(byte, 0); }

// 8 packed E2M1 codes (one dword, low nibble first) times an f16 scale -> 8 f16.
// fp4 * e4m3 has at most 6 significant bits and lies in [2^-10, 2688]: exact in f16.
__device__ inline v8h dequant8_f16(unsigned codes, v2h s2) {
  v2h p0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 1.0f, 0) * s2;
  v2h p1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 1.0f, 1) * s2;
  v2h p2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 1.0f, 2) * s2;
  v2h p3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 1.0f, 3) * s2;
  return v8h{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
}

// NVFP4, one wave per 32x32 tile, v_mfma_f32_32x32x16_f16 on operands dequantised in
// registers.  Per trip the wave consumes 64 k: lane (r, h) owns k in [64*i + 32*h, +32)
// of row r = two 16-element scale blocks, fed to four MFMAs eight elements at a time
// (A and B use the same assignment, so the K order inside a trip is immaterial).
__global__ __launch_bounds__(256) void nv_generic_kernel(NvArgs p, unsigned n_blocks) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 31, h = lane >> 5;
  const int m0 = (int)(blockIdx.x / n_blocks) * 32;
  const int n0 = (int)(blockIdx.x % n_blocks) * 128 + wave * 32;
  if (n0 >= p.N) return;
  const size_t row_bytes = (size_t)p.K / 2, row_scales = (size_t)p.K / kNvBlock;
  const int m = m0 + r, n = n0 + r;
  const bool mv = m < p.M, nv = n < p.N;
  const uint8_t* a_row = p.A + (size_t)m * row_bytes;
  const uint8_t* as_row = p.As + (size_t)m * row_scales;
  const uint8_t* b_row = p.B + (size_t)n * row_bytes;
  const uint8_t* bs_row = p.Bs + (size_t)n * row_scales;
  const int blocks = p.K / kNvBlock;
  v16f acc = {};
  for (int b0 = 0; b0 < blocks; b0 += 4) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int blk = b0 + 2 * h + j;
      const bool kv = blk < blocks;
      v2i a = {0, 0}, b = {0, 0};
      float sa = 0.f, sb = 0.f;
      if (mv && kv) {
        a = *reinterpret_cast<const v2i*>(a_row + (size_t)blk * 8);
        sa = e4m3_to_f32(as_row[blk]);
      }
      if (nv && kv) {
        b = *reinterpret_cast<const v2i*>(b_row + (size_t)blk * 8);
        sb = e4m3_to_f32(bs_row[blk]);
      }
      const _Float16 sah = (_Float16)sa, sbh = (_Float16)sb;
      const v2h sa2 = {sah, sah}, sb2 = {sbh, sbh};
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        v8h af = dequant8_f16((unsigned)a[d], sa2);
        v8h bf = dequant8_f16((unsigned)b[d], sb2);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf, af, acc, 0, 0, 0);
      }
    }
  }
  const float g = p.Ag[0] * p.Bg[0];
  if (mv) {
    uint16_t* c_row = p.C + (size_t)m * p.N;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      const int nn = n0 + 8 * (t / 4) + 4 * h + (t % 4);
      if (nn < p.N) c_row[nn] = to_bf16(acc[t] * g);
    }
  }
}

// Workgroups of the shape-agnostic kernels for m_tiles 32-row tiles: ceil(N/128) * m_tiles in grid.x, 0 when that
// exceeds what one grid dimension holds (2^31 - 1).
unsigned generic_grid(int N, uint64_t m_tiles, unsigned* n_blocks) {
  *n_blocks = ((unsigned)N + 127u) / 128u;
  const uint64_t total = (uint64_t)*n_blocks * m_tiles;
  return total <= 0x7FFFFFFFull ? (unsigned)total : 0u;
}

hipError_t launch_mx_generic(const MxArgs& p, hipStream_t s) {
  if (p.M <= 0 || p.N <= 0) return hipSuccess;
  unsigned n_blocks;
  const unsigned grid = generic_grid(p.N, ((uint64_t)p.M + 31) / 32 + (p.row_offsets ? (uint64_t)p.E : 0u), &n_blocks);
  if (grid == 0) return hipErrorInvalidConfiguration;
  if (p.swiglu) hipLaunchKernelGGL(mx_generic_kernel<true>, dim3(grid), dim3(256), 0, s, p, n_blocks);
  else hipLaunchKernelGGL(mx_generic_kernel<false>, dim3(grid), dim3(256), 0, s, p, n_blocks);
  return hipGetLastError();
}

hipError_t launch_nv_generic(const NvArgs& p, hipStream_t s) {
  if (p.M <= 0 || p.N <= 0) return hipSuccess;
  unsigned n_blocks;
  const unsigned grid = generic_grid(p.N, ((uint64_t)p.M + 31) / 32, &n_blocks);
  if (grid == 0) return hipErrorInvalidConfiguration;
  hipLaunchKernelGGL(nv_generic_kernel, dim3(grid), dim3(256), 0, s, p, n_blocks);
  return hipGetLastError();
}

}  // namespace ave
