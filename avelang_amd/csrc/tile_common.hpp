// Pieces shared by the LDS-staged 256x256 kernels: direct-to-LDS loads, LDS reads, the
// B-row permutation of the epilogue, and the bf16 store of one wave's 128x128 block.
#pragma once
#include "fp4_common.hpp"

namespace ave {

// global_load_lds: lane l of the wave writes its 16 (4) bytes at LDS address lds_addr + 16*l
// (4*l); lds_addr and gbase are wave-uniform, voff is the lane's byte offset from gbase.
// The instruction counts on vmcnt.  Issued through inline asm so that the compiler's own
// wait-count bookkeeping does not serialise later LDS reads behind loads that target the
// *other* stage buffer; the kernels wait explicitly (wait_all_loads + barrier).
__device__ inline void dma16(const void* gbase, unsigned voff, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voff), "s"(gbase) : "m0");
}
__device__ inline void dma4(const void* gbase, unsigned voff, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voff), "s"(gbase) : "m0");
}
__device__ inline void wait_all_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

__device__ inline v4i lds_read16(unsigned addr) {
  return *reinterpret_cast<const __attribute__((address_space(3))) v4i*>((uintptr_t)addr);
}
__device__ inline v2i lds_read8(unsigned addr) {
  return *reinterpret_cast<const __attribute__((address_space(3))) v2i*>((uintptr_t)addr);
}

__device__ inline int pi_row(int rho) {
  const int u = rho >> 3, q = (rho >> 2) & 1, v = rho & 3;
  return 16 * (u >> 1) + 8 * q + 4 * (u & 1) + v;
}


// Stores one wave's grid of 4 (n) x MI (m) 32x32 accumulator blocks.  acc[nj][mi] holds, for lane
// (c = lane%32, q = lane/32), row m = m0 + 32*mi + c and columns n0 + 32*nj + 16*piece + 8*q + 0..7
// in registers 8*piece .. 8*piece+7.
template <int MI>
__device__ inline void store_wave_block(const v16f (&acc)[4][MI], uint16_t* C, int N, int m0, int m_end, int n0,
                                        int lane, float scale) {
  const int c = lane & 31, q = lane >> 5;
  const bool vec_ok = (N % 8 == 0) && ((reinterpret_cast<uintptr_t>(C) & 15) == 0);
#pragma unroll
  for (int mi = 0; mi < MI; ++mi) {
    const int m = m0 + 32 * mi + c;
    if (m >= m_end) continue;
    uint16_t* crow = C + (size_t)m * N;
#pragma unroll
    for (int nj = 0; nj < 4; ++nj) {
      const v16f& d = acc[nj][mi];
#pragma unroll
      for (int piece = 0; piece < 2; ++piece) {
        const int n = n0 + 32 * nj + 16 * piece + 8 * q;
        v4i o;
        o[0] = (int)pack_bf16x2(d[8 * piece + 0] * scale, d[8 * piece + 1] * scale);
        o[1] = (int)pack_bf16x2(d[8 * piece + 2] * scale, d[8 * piece + 3] * scale);
        o[2] = (int)pack_bf16x2(d[8 * piece + 4] * scale, d[8 * piece + 5] * scale);
        o[3] = (int)pack_bf16x2(d[8 * piece + 6] * scale, d[8 * piece + 7] * scale);
        if (vec_ok && n + 8 <= N) {
          *reinterpret_cast<v4i*>(crow + n) = o;
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (n + e < N) crow[n + e] = (uint16_t)(((unsigned)o[e >> 1] >> (16 * (e & 1))) & 0xFFFF);
        }
      }
    }
  }
}

}  // namespace ave
