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
// The loads of one issuing wave for one stage of a 256x256 tile -- eight 1 KB pieces of A to LDS addresses
// md + 1024 i and eight of B to md + 32768 + 1024 i -- as ONE asm statement that is skipped as a whole when
// the wave's group (waves 0-3: 0, waves 4-7: 1; a scalar) is not `group`.  A wave-dependent choice of the issuing
// waves then costs no control flow that the compiler can see (a branch around sixteen asm statements made it
// spill).
__device__ inline void dma16_stage(int wave_group, int group, unsigned md, const void* ga, const void* gb, const unsigned (&a)[8],
                                   const unsigned (&b)[8]) {
  asm volatile(
      "s_cmp_eq_u32 %[wg], %[g]\n\t"
      "s_cbranch_scc0 1f\n\t"
      "s_mov_b32 m0, %[md]\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a0], %[ga]\n\t"
      "s_add_u32 m0, %[md], 0x8000\n\t s_nop 0\n\t global_load_lds_dwordx4 %[b0], %[gb]\n\t"
      "s_add_u32 m0, %[md], 0x0400\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a1], %[ga]\n\t"
      "s_add_u32 m0, %[md], 0x8400\n\t s_nop 0\n\t global_load_lds_dwordx4 %[b1], %[gb]\n\t"
      "s_add_u32 m0, %[md], 0x0800\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a2], %[ga]\n\t"
      "s_add_u32 m0, %[md], 0x8800\n\t s_nop 0\n\t global_load_lds_dwordx4 %[b2], %[gb]\n\t"
      "s_add_u32 m0, %[md], 0x0c00\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a3], %[ga]\n\t"
      "s_add_u32 m0, %[md], 0x8c00\n\t s_nop 0\n\t global_load_lds_dwordx4 %[b3], %[gb]\n\t"
      "s_add_u32 m0, %[md], 0x1000\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a4], %[ga]\n\t"
      "s_add_u32 m0, %[md], 0x9000\n\t s_nop 0\n\t global_load_lds_dwordx4 %[b4], %[gb]\n\t"
      "s_add_u32 m0, %[md], 0x1400\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a5], %[ga]\n\t"
      "s_add_u32 m0, %[md], 0x9400\n\t s_nop 0\n\t global_load_lds_dwordx4 %[b5], %[gb]\n\t"
      "s_add_u32 m0, %[md], 0x1800\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a6], %[ga]\n\t"
      "s_add_u32 m0, %[md], 0x9800\n\t s_nop 0\n\t global_load_lds_dwordx4 %[b6], %[gb]\n\t"
      "s_add_u32 m0, %[md], 0x1c00\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a7], %[ga]\n\t"
      "s_add_u32 m0, %[md], 0x9c00\n\t s_nop 0\n\t global_load_lds_dwordx4 %[b7], %[gb]\n\t"
      "1:\n\t"
      :
      : [wg] "s"(__builtin_amdgcn_readfirstlane(wave_group)), [g] "s"(__builtin_amdgcn_readfirstlane(group)),
        [md] "s"(__builtin_amdgcn_readfirstlane(md)), [ga] "s"(ga), [gb] "s"(gb), [a0] "v"(a[0]), [a1] "v"(a[1]), [a2] "v"(a[2]), [a3] "v"(a[3]), [a4] "v"(a[4]), [a5] "v"(a[5]),
        [a6] "v"(a[6]), [a7] "v"(a[7]), [b0] "v"(b[0]), [b1] "v"(b[1]), [b2] "v"(b[2]), [b3] "v"(b[3]), [b4] "v"(b[4]),
        [b5] "v"(b[5]), [b6] "v"(b[6]), [b7] "v"(b[7])
      : "m0", "scc", "memory");
}
// Same for the two 1 KB pieces of 16-byte scale rows: 64 rows of A to LDS address ms, 64 rows of B to ms + 4096.
__device__ inline void dma16_scale_rows(int wave_group, int group, unsigned ms, const void* gas, const void* gbs, unsigned as,
                                        unsigned bs) {
  asm volatile(
      "s_cmp_eq_u32 %[wg], %[g]\n\t"
      "s_cbranch_scc0 1f\n\t"
      "s_mov_b32 m0, %[ms]\n\t s_nop 0\n\t global_load_lds_dwordx4 %[as], %[gas]\n\t"
      "s_add_u32 m0, %[ms], 0x1000\n\t s_nop 0\n\t global_load_lds_dwordx4 %[bs], %[gbs]\n\t"
      "1:\n\t"
      :
      : [wg] "s"(__builtin_amdgcn_readfirstlane(wave_group)), [g] "s"(__builtin_amdgcn_readfirstlane(group)),
        [ms] "s"(__builtin_amdgcn_readfirstlane(ms)), [gas] "s"(gas), [gbs] "s"(gbs), [as] "v"(as), [bs] "v"(bs)
      : "m0", "scc", "memory");
}
// The eight 1 KB pieces of a chunk of 64-byte scale rows that one issuing wave moves: 16 rows of A per instruction to
// LDS addresses ms + 1024 i, 16 rows of B to ms + 16384 + 1024 i; skipped as a whole when `enable` (a scalar) is 0.
__device__ inline void dma16_scale_chunk(unsigned enable, unsigned ms, const void* gas, const void* gbs, const unsigned (&a)[4],
                                         const unsigned (&b)[4]) {
  asm volatile(
      "s_cmp_eq_u32 %[en], 0\n\t"
      "s_cbranch_scc1 1f\n\t"
      "s_mov_b32 m0, %[ms]\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a0], %[gas]\n\t"
      "s_add_u32 m0, %[ms], 0x4000\n\t s_nop 0\n\t global_load_lds_dwordx4 %[b0], %[gbs]\n\t"
      "s_add_u32 m0, %[ms], 0x0400\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a1], %[gas]\n\t"
      "s_add_u32 m0, %[ms], 0x4400\n\t s_nop 0\n\t global_load_lds_dwordx4 %[b1], %[gbs]\n\t"
      "s_add_u32 m0, %[ms], 0x0800\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a2], %[gas]\n\t"
      "s_add_u32 m0, %[ms], 0x4800\n\t s_nop 0\n\t global_load_lds_dwordx4 %[b2], %[gbs]\n\t"
      "s_add_u32 m0, %[ms], 0x0c00\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a3], %[gas]\n\t"
      "s_add_u32 m0, %[ms], 0x4c00\n\t s_nop 0\n\t global_load_lds_dwordx4 %[b3], %[gbs]\n\t"
      "1:\n\t"
      :
      : [en] "s"(__builtin_amdgcn_readfirstlane(enable)), [ms] "s"(__builtin_amdgcn_readfirstlane(ms)), [gas] "s"(gas), [gbs] "s"(gbs),
        [a0] "v"(a[0]), [a1] "v"(a[1]), [a2] "v"(a[2]), [a3] "v"(a[3]), [b0] "v"(b[0]), [b1] "v"(b[1]), [b2] "v"(b[2]), [b3] "v"(b[3])
      : "m0", "scc", "memory");
}
// Before a stage barrier: waves 0-3 (which issue the stage loads) wait for their loads and LDS reads, waves 4-7 for
// their LDS reads only, so that look-ahead touches they have in flight do not hold them.
__device__ inline void wait_loads_if_issuer(int wave) {
  asm volatile(
      "s_cmp_lt_u32 %0, 4\n\t"
      "s_cbranch_scc0 1f\n\t"
      "s_waitcnt vmcnt(0)\n\t"
      "1:\n\t"
      "s_waitcnt lgkmcnt(0)" ::"s"(__builtin_amdgcn_readfirstlane(wave))
      : "scc", "memory");
}

__device__ inline void wait_all_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

__device__ inline v4i lds_read16(unsigned addr) {
  return *reinterpret_cast<const __attribute__((address_space(3))) v4i*>((uintptr_t)addr);
}
__device__ inline int lds_read4(unsigned addr) {
  return *reinterpret_cast<const __attribute__((address_space(3))) int*>((uintptr_t)addr);
}
__device__ inline v2i lds_read8(unsigned addr) {
  return *reinterpret_cast<const __attribute__((address_space(3))) v2i*>((uintptr_t)addr);
}

__device__ inline int pi_row(int rho) {
  const int u = rho >> 3, q = (rho >> 2) & 1, v = rho & 3;
  return 16 * (u >> 1) + 8 * q + 4 * (u & 1) + v;
}


// Stores one wave's grid of NJ (n) x MI (m) 32x32 accumulator blocks.  acc[nj][mi] holds, for lane
// (c = lane%32, q = lane/32), row m = m0 + 32*mi + c and columns n0 + 32*nj + 16*piece + 8*q + 0..7
// in registers 8*piece .. 8*piece+7.
template <int MI, int NJ = 4>
__device__ inline void store_wave_block(const v16f (&acc)[NJ][MI], uint16_t* C, int N, int m0, int m_end, int n0,
                                        int lane, float scale) {
  const int c = lane & 31, q = lane >> 5;
  const bool vec_ok = (N % 8 == 0) && ((reinterpret_cast<uintptr_t>(C) & 15) == 0);
#pragma unroll
  for (int mi = 0; mi < MI; ++mi) {
    const int m = m0 + 32 * mi + c;
    if (m >= m_end) continue;
    uint16_t* crow = C + (size_t)m * N;
#pragma unroll
    for (int nj = 0; nj < NJ; ++nj) {
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

// The same grid of blocks as fp32, unrounded: a K slice's partial sums, [M][N] row-major.
template <int MI, int NJ = 4>
__device__ inline void store_wave_block_f32(const v16f (&acc)[NJ][MI], float* P, int N, int m0, int m_end, int n0,
                                            int lane, float scale = 1.0f) {
  const int c = lane & 31, q = lane >> 5;
  const bool vec_ok = (N % 4 == 0) && ((reinterpret_cast<uintptr_t>(P) & 15) == 0);
#pragma unroll
  for (int mi = 0; mi < MI; ++mi) {
    const int m = m0 + 32 * mi + c;
    if (m >= m_end) continue;
    float* prow = P + (size_t)m * N;
#pragma unroll
    for (int nj = 0; nj < NJ; ++nj) {
      const v16f& d = acc[nj][mi];
#pragma unroll
      for (int piece = 0; piece < 2; ++piece) {
        const int n = n0 + 32 * nj + 16 * piece + 8 * q;
        if (vec_ok && n + 8 <= N) {
          *reinterpret_cast<v4f*>(prow + n) =
              v4f{d[8 * piece + 0] * scale, d[8 * piece + 1] * scale, d[8 * piece + 2] * scale, d[8 * piece + 3] * scale};
          *reinterpret_cast<v4f*>(prow + n + 4) =
              v4f{d[8 * piece + 4] * scale, d[8 * piece + 5] * scale, d[8 * piece + 6] * scale, d[8 * piece + 7] * scale};
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (n + e < N) prow[n + e] = d[8 * piece + e] * scale;
        }
      }
    }
  }
}

}  // namespace ave
