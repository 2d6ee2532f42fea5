// NVFP4 GEMM for gfx950, LDS-staged: 256x256 tile per workgroup, eight wavefronts (two per SIMD)
// of 64(m) x 128(n): one wave's register dequantisation (VALU) runs under the other's MFMAs.
// E4M3 scales per 16 elements do not fit the scaled MFMA (it takes one E8M0 per 32), so the
// operands are dequantised in registers to f16 -- E2M1 x E4M3 has at most 6 significant bits
// and lies in [2^-10, 2688], exact in f16 -- and multiplied with v_mfma_f32_32x32x16_f16.
// The two fp32 per-tensor scales are applied once, in the epilogue.
//
// Staging is the MXFP4 tile kernel's: packed codes move global -> LDS with
// global_load_lds_dwordx4 into a row-major [256][128 B] image whose 16-byte chunks are
// XOR-swizzled on the source side (chunk ^ ((row >> 1) & 7), conflict-free for 16-lane LDS reads); the scale image is [256 rows][16 B] per operand and stage.
//
// K order inside a 64-element group: lane (rho, h) reads the 16 bytes holding k = 32h .. 32h+31
// of its row and feeds dword d (8 elements) to MFMA d of the group; A and B fragments use the
// same assignment, so the sum runs over every k exactly once.
#include "fp4_common.hpp"
#include "kernels.hpp"
#include "tile_common.hpp"
#include "tile_map.hpp"

namespace ave {
namespace {

constexpr int BM = 256, BN = 256, BK = 256;
constexpr int kWaves = 8;
constexpr int kRowBytes = BK / 2;                     // 128
constexpr int kScaleRow = BK / 16;                    // 16 bytes
constexpr int kOffA = 0;
constexpr int kOffB = BM * kRowBytes;                 // 32768
constexpr int kOffAs = kOffB + BN * kRowBytes;        // 65536
constexpr int kOffBs = kOffAs + BM * kScaleRow;       // +4096
constexpr int kStageBytes = kOffBs + BN * kScaleRow;  // 73728
constexpr int kLdsBytes = 2 * kStageBytes;            // 147456


// SPLITK: workgroup pid is tile pid % tiles of K slice pid / tiles; a slice is p.slice_stages stages (the last one
// what is left), its fp32 sums (times the two per-tensor scales) go to p.P[slice][M][N] and launch_splitk_reduce adds
// the slices up.
template <bool SPLITK>
__global__ __launch_bounds__(kWaves * 64) void nv_tile_kernel(NvArgs p, int m_tiles, int n_tiles) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int wm = w >> 1, wn = w & 1;

  int tm, tn, slice = 0;
  {
    int pid = blockIdx.x;
    if (SPLITK) {
      slice = pid / (m_tiles * n_tiles);
      pid -= slice * (m_tiles * n_tiles);
    }
    map_tile(pid, m_tiles, n_tiles, tm, tn);
  }
  const int m_begin = tm * BM, n_begin = tn * BN;
  const unsigned row_bytes = (unsigned)p.K / 2, row_scales = (unsigned)p.K / 16;
  // A wave whose 64 rows lie past the end of A multiplies nothing: it only keeps the barrier count and, if it is
  // one of the issuing waves, its loads.  The kernel is bound by the conversions, two waves to a SIMD: with at most
  // 128 rows the four waves of the upper half (one per SIMD) drop out and the stage takes half the time.
  const bool active = m_begin + wm * 64 < p.M;

  // Waves 0-3 issue all loads of the workgroup: wave w moves tile rows 64w .. 64w+63 of both operands (eight
  // 1 KB pieces each per stage) and their 16-byte scale rows.  With every wave issuing its share, both waves of
  // a SIMD sit in load issue at the same time.
  unsigned a_off[8], b_off[8], as_off, bs_off;
  {
    const int lr = lane >> 3, cprime = lane & 7, wi = w & 3;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = (wi * 8 + i) * 8 + lr;
      const int chunk = cprime ^ ((row >> 1) & 7);
      int am = m_begin + row;
      am = am < p.M ? am : p.M - 1;
      int bn = n_begin + row;
      bn = bn < p.N ? bn : p.N - 1;
      a_off[i] = (unsigned)am * row_bytes + chunk * 16;
      b_off[i] = (unsigned)bn * row_bytes + chunk * 16;
    }
    const int row = wi * 64 + lane;
    int am = m_begin + row;
    am = am < p.M ? am : p.M - 1;
    int bn = n_begin + row;
    bn = bn < p.N ? bn : p.N - 1;
    as_off = (unsigned)am * row_scales;
    bs_off = (unsigned)bn * row_scales;
  }
  const unsigned lds_base = (unsigned)(uintptr_t)lds;
  static_assert(kOffB == 0x8000 && kOffBs - kOffAs == 0x1000, "the LDS offsets built into dma16_stage / dma16_scale_rows");

  auto issue_stage = [&](int s, int buf) {
    const unsigned sb = lds_base + buf * kStageBytes;
    dma16_stage(w >> 2, 0, sb + kOffA + (w & 3) * 8192, p.A + (size_t)s * kRowBytes, p.B + (size_t)s * kRowBytes, a_off, b_off);
    dma16_scale_rows(w >> 2, 0, sb + kOffAs + (w & 3) * 1024, p.As + (size_t)s * kScaleRow, p.Bs + (size_t)s * kScaleRow,
                     as_off, bs_off);
  };

  const int rho = lane & 31, h = lane >> 5;
  const int a_row = wm * 64 + rho;
  const int b_row = wn * 128 + pi_row(rho);
  const unsigned a_frag = kOffA + a_row * kRowBytes + ((h ^ ((a_row >> 1) & 7)) * 16);
  const unsigned b_frag = kOffB + b_row * kRowBytes + ((h ^ ((b_row >> 1) & 7)) * 16);
  const unsigned a_sc = kOffAs + a_row * kScaleRow;  // + mi*32*16
  const unsigned b_sc = kOffBs + b_row * kScaleRow;

  v16f acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = v16f{};

  const int all_stages = p.K / BK;
  const int s_begin = SPLITK ? slice * p.slice_stages : 0;
  const int s_end = SPLITK && s_begin + p.slice_stages < all_stages ? s_begin + p.slice_stages : all_stages;
  issue_stage(s_begin, 0);
  for (int s = s_begin; s < s_end; ++s) {
    const int buf = (s - s_begin) & 1;
    wait_all_loads();
    __syncthreads();
    if (s + 1 < s_end) issue_stage(s + 1, buf ^ 1);
    if (!active) continue;
    const unsigned sb = lds_base + buf * kStageBytes;

    // the 16 scale bytes of each fragment row, once per stage: consecutive rows are consecutive 16-byte
    // slots, which a 16-lane LDS read serves without bank conflicts (dword reads at this stride are 2-way)
    v4i asw4[2], bsw4[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      bsw4[i] = lds_read16(sb + b_sc + i * 32 * kScaleRow);
      if (i < 2) asw4[i] = lds_read16(sb + a_sc + i * 32 * kScaleRow);
    }
    // 16 steps of 16 k each (4 groups of 64 elements x 4 dwords per lane), software-pipelined by one step: the
    // fragments of step t+1 are converted under the 8 MFMAs of step t, and the order is pinned to one MFMA followed
    // by six conversion instructions (a step has 48).  Measured on one device: 1 + 6 0.350 ms, 1 + 5 0.353, 1 + 7
    // 0.357, 2 + 12 0.362, 4 + 24 0.368, all conversions before all MFMAs 0.395, the compiler's own order of the
    // unpipelined loop 0.365.
    v4i araw[2], braw[4];
    v2h asc[2], bsc[4];
    v8h af[2][2], bf[2][4];
    auto fetch_group = [&](int u) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        braw[i] = lds_read16(sb + (b_frag ^ (u * 32)) + i * 4096);
        bsc[i] = scale_pair(bsw4[i][u] >> (16 * h));   // this lane's k range: scale blocks 4u + 2h, 4u + 2h + 1
        if (i < 2) {
          araw[i] = lds_read16(sb + (a_frag ^ (u * 32)) + i * 4096);
          asc[i] = scale_pair(asw4[i][u] >> (16 * h));
        }
      }
    };
    auto convert = [&](int d, int slot) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        bf[slot][i] = dequant8((unsigned)braw[i][d], bsc[i][d >> 1]);
        if (i < 2) af[slot][i] = dequant8((unsigned)araw[i][d], asc[i][d >> 1]);
      }
    };
    fetch_group(0);
    convert(0, 0);
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      if (t + 1 < 16) {
        if (((t + 1) & 3) == 0) fetch_group((t + 1) >> 2);
        convert((t + 1) & 3, (t + 1) & 1);
      }
#pragma unroll
      for (int nj = 0; nj < 4; ++nj)
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
          acc[nj][mi] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[t & 1][nj], af[t & 1][mi], acc[nj][mi], 0, 0, 0);
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one MFMA
        __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);   // six VALU
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  const float g = p.Ag[0] * p.Bg[0];
  if constexpr (SPLITK) {
    store_wave_block_f32<2>(acc, p.P + (size_t)slice * (size_t)p.M * (size_t)p.N, p.N, m_begin + wm * 64, p.M,
                            n_begin + wn * 128, lane, g);
  } else {
    store_wave_block<2>(acc, p.C, p.N, m_begin + wm * 64, p.M, n_begin + wn * 128, lane, g);
  }
}


// v_mfma_f32_32x32x16_f16 with its accumulator in the AGPR half of the register file, which the compiler does not
// manage for a kernel that needs all 256 of them (it moved accumulators to and from VGPRs inside the loop).  The
// operands were written by VALU instructions at least one MFMA earlier.
__device__ inline void mfma_agpr(v16f& acc, const v8h& b, const v8h& a) {
  asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(b), "v"(a));
}

// The same GEMM with FOUR wavefronts of 128 x 128 (one per SIMD, 512 registers each: 256 accumulators in AGPRs).
// A wave converts (128 + 128) x 16 operand elements for its 16 MFMAs of a step where two waves of 64 x 128 convert
// 2 x (64 + 128) x 16 for the same 16: a third fewer conversion instructions per MFMA.  One wave per SIMD has nobody
// to hide behind, so the order is written out: each MFMA is followed by the conversion of half a fragment (2 cvt +
// 2 multiplies) of the next step, and the raw fragments of the next group of 64 k are read from LDS a whole step
// before their first conversion.  Measured on 4096 x 4096 x 14336: 75 % MFMA-busy (42 cycles per MFMA and its four
// conversion instructions, where the matrix core needs 32) against 71 % with eight waves -- a wave on its own issues
// one VALU instruction in about 6 cycles (loops of independent v_add_u32, v_pk_mul_f16 or
// v_cvt_scalef32_pk_f16_fp4 all take 2.5 ns per instruction), and what one wave can issue is the limit of this form.
template <bool SPLITK>
__global__ __launch_bounds__(4 * 64) void nv_tile4_kernel(NvArgs p, int m_tiles, int n_tiles) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int wm = w >> 1, wn = w & 1;
  int tm, tn, slice = 0;   // SPLITK: as in nv_tile_kernel
  {
    int pid = blockIdx.x;
    if (SPLITK) {
      slice = pid / (m_tiles * n_tiles);
      pid -= slice * (m_tiles * n_tiles);
    }
    map_tile(pid, m_tiles, n_tiles, tm, tn);
  }
  const int m_begin = tm * BM, n_begin = tn * BN;
  const unsigned row_bytes = (unsigned)p.K / 2, row_scales = (unsigned)p.K / 16;

  // wave w moves tile rows 64w .. 64w+63 of both operands (eight 1 KB pieces each per stage) and their scale rows
  unsigned a_off[8], b_off[8], as_off, bs_off;
  {
    const int lr = lane >> 3, cprime = lane & 7;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = (w * 8 + i) * 8 + lr;
      const int chunk = cprime ^ ((row >> 1) & 7);
      int am = m_begin + row;
      am = am < p.M ? am : p.M - 1;
      int bn = n_begin + row;
      bn = bn < p.N ? bn : p.N - 1;
      a_off[i] = (unsigned)am * row_bytes + chunk * 16;
      b_off[i] = (unsigned)bn * row_bytes + chunk * 16;
    }
    const int row = w * 64 + lane;
    int am = m_begin + row;
    am = am < p.M ? am : p.M - 1;
    int bn = n_begin + row;
    bn = bn < p.N ? bn : p.N - 1;
    as_off = (unsigned)am * row_scales;
    bs_off = (unsigned)bn * row_scales;
  }
  const unsigned lds_base = (unsigned)(uintptr_t)lds;
  auto issue_stage = [&](int s, int buf, bool on) {   // off: the asm statements skip their loads
    const unsigned sb = lds_base + buf * kStageBytes;
    dma16_stage((w >> 2) + (on ? 0 : 1), 0, sb + kOffA + w * 8192, p.A + (size_t)s * kRowBytes, p.B + (size_t)s * kRowBytes, a_off, b_off);
    dma16_scale_rows((w >> 2) + (on ? 0 : 1), 0, sb + kOffAs + w * 1024, p.As + (size_t)s * kScaleRow, p.Bs + (size_t)s * kScaleRow, as_off, bs_off);
  };

  const int rho = lane & 31, h = lane >> 5;
  const int a_row = wm * 128 + rho;
  const int b_row = wn * 128 + pi_row(rho);
  const unsigned a_frag = kOffA + a_row * kRowBytes + ((h ^ ((a_row >> 1) & 7)) * 16);
  const unsigned b_frag = kOffB + b_row * kRowBytes + ((h ^ ((b_row >> 1) & 7)) * 16);
  const unsigned a_sc = kOffAs + a_row * kScaleRow;
  const unsigned b_sc = kOffBs + b_row * kScaleRow;

  v16f acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = v16f{};

  // fragments 0-3: B rows 32 f .., fragments 4-7: A rows 32 (f - 4) ..
  v4i sw4[8];        // the 16 scale bytes of each fragment row, one stage
  v4i raw[2][8];     // the packed codes of a group of 64 k, two groups in flight
  v2h sc[8];         // the two scales of this lane's 32 k of the group being converted
  v8h fr[2][8];      // converted fragments of two steps
  auto read_scales = [&](unsigned sb) {
#pragma unroll
    for (int f = 0; f < 8; ++f) sw4[f] = lds_read16(sb + (f < 4 ? b_sc + f * 32 * kScaleRow : a_sc + (f - 4) * 32 * kScaleRow));
  };
  auto fetch_group = [&](unsigned sb, int u) {
#pragma unroll
    for (int f = 0; f < 8; ++f)
      raw[u & 1][f] = lds_read16(sb + ((f < 4 ? b_frag : a_frag) ^ (u * 32)) + (f & 3) * 4096);
  };
  auto group_scales = [&](int u) {   // scale blocks 4u + 2h, 4u + 2h + 1 of the row's 16
#pragma unroll
    for (int f = 0; f < 8; ++f) sc[f] = scale_pair(sw4[f][u] >> (16 * h));
  };
  // half hh (2 cvt + 2 multiplies) of fragment f of step t
  auto convert_half = [&](int t, int f, int hh) {
    const unsigned codes = (unsigned)raw[(t >> 2) & 1][f][t & 3];
    const _Float16 sv = sc[f][(t & 3) >> 1];
    const v2h s2 = {sv, sv};
    v2h p0, p1;
    if (hh) {
      p0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 1.0f, 2) * s2;
      p1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 1.0f, 3) * s2;
    } else {
      p0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 1.0f, 0) * s2;
      p1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 1.0f, 1) * s2;
    }
    v8h& d = fr[t & 1][f];
    d[4 * hh + 0] = p0[0];
    d[4 * hh + 1] = p0[1];
    d[4 * hh + 2] = p1[0];
    d[4 * hh + 3] = p1[1];
  };
  // The pipeline runs across stages and the loop body has no branches (a path around the MFMAs made the compiler
  // spill accumulators): the stage's barrier sits in step 12, when every wave has read the last of the stage's
  // codes (group 3, in step 10) and scale rows, so the buffer can take the stage after the next; behind it the
  // wave reads the next stage's scale rows (step 12) and first group (step 14) and converts the next stage's step 0
  // under the MFMAs of step 15.  In the last stage these reads and conversions run on stale LDS contents and are
  // not used, and the loads are switched off inside their asm statement.
  const int all_stages = p.K / BK;
  const int s_begin = SPLITK ? slice * p.slice_stages : 0;
  const int stages = (SPLITK && s_begin + p.slice_stages < all_stages ? s_begin + p.slice_stages : all_stages) - s_begin;
  issue_stage(s_begin, 0, true);
  wait_all_loads();
  __syncthreads();
  issue_stage(s_begin + 1, 1, 1 < stages);
  read_scales(lds_base);
  fetch_group(lds_base, 0);
  group_scales(0);
#pragma unroll
  for (int q = 0; q < 16; ++q) convert_half(0, q >> 1, q & 1);
  for (int s = 0; s < stages; ++s) {
    const int buf = s & 1;
    const unsigned sb = lds_base + buf * kStageBytes, sbn = lds_base + (buf ^ 1) * kStageBytes;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      if ((t & 3) == 2 && t + 2 < 16) fetch_group(sb, (t >> 2) + 1);
      if ((t & 3) == 3 && t + 1 < 16) group_scales((t + 1) >> 2);
      if (t == 12) {
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __syncthreads();
        issue_stage(s_begin + s + 2, buf, s + 2 < stages);
        read_scales(sbn);
      }
      if (t == 14) fetch_group(sbn, 0);
      if (t == 15) group_scales(0);
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        mfma_agpr(acc[q >> 2][q & 3], fr[t & 1][q >> 2], fr[t & 1][4 + (q & 3)]);
        convert_half((t + 1) & 15, q >> 1, q & 1);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  // the last MFMAs' results are read below by instructions the compiler does not know to be behind MFMAs
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
  const float g = p.Ag[0] * p.Bg[0];
  if constexpr (SPLITK) {
    store_wave_block_f32<4>(acc, p.P + (size_t)slice * (size_t)p.M * (size_t)p.N, p.N, m_begin + wm * 128, p.M,
                            n_begin + wn * 128, lane, g);
  } else {
    store_wave_block<4>(acc, p.C, p.N, m_begin + wm * 128, p.M, n_begin + wn * 128, lane, g);
  }
}

}  // namespace

bool nv_tile_supports(const NvArgs& p) {
  if (p.K % BK != 0 || p.M <= 0 || p.N <= 0) return false;
  if ((uint64_t)p.M * (uint64_t)(p.K / 2) >= (1ull << 32)) return false;
  if ((uint64_t)p.N * (uint64_t)(p.K / 2) >= (1ull << 32)) return false;
  // packed rows and scale rows are fetched as aligned 16-byte chunks
  if ((reinterpret_cast<uintptr_t>(p.A) & 15) || (reinterpret_cast<uintptr_t>(p.B) & 15)) return false;
  if ((reinterpret_cast<uintptr_t>(p.As) & 15) || (reinterpret_cast<uintptr_t>(p.Bs) & 15)) return false;
  return true;
}

hipError_t launch_nv_tile(const NvArgs& p, hipStream_t s) {
  const int m_tiles = (p.M + BM - 1) / BM, n_tiles = (p.N + BN - 1) / BN;
  if (p.M > 128) {
    // four waves of 128 x 128: 4096 x 4096 x 14336 0.334 ms against 0.355 ms with eight of 64 x 128, same bits.  With
    // at most 128 rows the eight-wave kernel's upper four waves drop out and it is the faster one.
    if (hipError_t e = allow_dynamic_lds<nv_tile4_kernel<false>>(kLdsBytes); e != hipSuccess) return e;
    hipLaunchKernelGGL(nv_tile4_kernel<false>, dim3((unsigned)(m_tiles * n_tiles)), dim3(4 * 64), kLdsBytes, s, p, m_tiles, n_tiles);
    return hipGetLastError();
  }
  if (hipError_t e = allow_dynamic_lds<nv_tile_kernel<false>>(kLdsBytes); e != hipSuccess) return e;
  hipLaunchKernelGGL(nv_tile_kernel<false>, dim3((unsigned)(m_tiles * n_tiles)), dim3(kWaves * 64), kLdsBytes, s, p, m_tiles,
                     n_tiles);
  return hipGetLastError();
}

// The kernel is bound by its conversions (about 2.5 us per stage and active half of the tile), far above what the
// partial sums of a split cost: with at most half as many tiles as compute units, K is cut into as many slices as
// there are compute units per tile, of at least two stages each.
SplitPlan nv_tile_split_plan_for(int M, int N, int K, int cus) {
  SplitPlan plan;
  if (M <= 64 || N <= 0 || K <= 0 || K % BK != 0 || cus <= 0) return plan;   // the weight-streaming kernel owns M <= 64
  if ((uint64_t)M * (uint64_t)(K / 2) >= (1ull << 32) || (uint64_t)N * (uint64_t)(K / 2) >= (1ull << 32)) return plan;
  const long tiles = (long)((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  const int stages = K / BK;
  if (tiles * 2 > cus || stages < 4) return plan;
  int slices = (int)(cus / tiles);
  if (slices > stages / 2) slices = stages / 2;
  const int per = (stages + slices - 1) / slices;
  slices = (stages + per - 1) / per;
  if (slices < 2) return plan;
  plan.slices = slices;
  plan.slice_pairs = per;   // stages per slice for this kernel
  plan.workspace_bytes = (size_t)slices * (size_t)M * (size_t)N * sizeof(float);
  return plan;
}

SplitPlan nv_tile_split_plan(int M, int N, int K) { return nv_tile_split_plan_for(M, N, K, compute_units()); }

hipError_t launch_nv_tile_splitk(const NvArgs& p, hipStream_t s) {
  const int m_tiles = (p.M + BM - 1) / BM, n_tiles = (p.N + BN - 1) / BN;
  if (p.M > 128) {   // four waves of 128 x 128, as in launch_nv_tile
    if (hipError_t e = allow_dynamic_lds<nv_tile4_kernel<true>>(kLdsBytes); e != hipSuccess) return e;
    hipLaunchKernelGGL(nv_tile4_kernel<true>, dim3((unsigned)(m_tiles * n_tiles * p.slices)), dim3(4 * 64), kLdsBytes, s, p,
                       m_tiles, n_tiles);
  } else {
    if (hipError_t e = allow_dynamic_lds<nv_tile_kernel<true>>(kLdsBytes); e != hipSuccess) return e;
    hipLaunchKernelGGL(nv_tile_kernel<true>, dim3((unsigned)(m_tiles * n_tiles * p.slices)), dim3(kWaves * 64), kLdsBytes, s, p,
                       m_tiles, n_tiles);
  }
  if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
  return launch_splitk_reduce(p.P, p.C, (size_t)p.M * (size_t)p.N, p.slices, s);
}

}  // namespace ave
