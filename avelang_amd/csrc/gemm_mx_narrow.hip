// MXFP4 GEMM for gfx950 for shapes with few output tiles -- a few hundred rows of activations against many weight
// rows (batched decode of a wide projection), or any shape with no more 256 x 128 tiles than compute units:
// 256 x 128 output tile per workgroup and a RING OF THREE stage buffers.
//
// With 65..256 rows of A the 256 x 256 tiling of gemm_mx_tile.hip yields one row of N/256 tiles -- 112 for
// N = 28672, fewer than half of the compute units -- and every workgroup streams a weight panel of its own from
// HBM with a single stage of 64 KB in flight: it runs at the latency of that stream (1.5-1.7 us per stage).
// Halving the tile along N doubles the workgroups, and a stage of 48 KB (256 rows of A, 128 rows of B, 256
// elements of K) leaves room for three stage buffers, so that two stages are in flight while one is multiplied.
//
// Everything else follows gemm_mx_tile.hip: global -> LDS with global_load_lds_dwordx4 issued by waves 0-3,
// source-side XOR swizzle, scales as 16-byte rows per pair of stages, eight waves (two per SIMD), here of
// 64 (m) x 64 (n) each = 2 x 2 accumulator blocks of v_mfma_scale_f32_32x32x64_f8f6f4, the barrier of a stage in
// front of its last K quarter.  K % 512 == 0, 16-byte aligned scale tensors.
//
// SWIGLU: B holds the N gate rows followed by the N up rows and a tile is 256 rows of C by 64 outputs.  The 64
// B-image rows of wave (wm, wn) are the gate rows (first 32) and the up rows (last 32) of outputs 32 wn .. 32 wn + 31,
// so the wave's two accumulator blocks of a row block hold the gate and the up value of the same outputs and
// silu(gate) * up is evaluated in registers, in fp32, exactly as in the 256 x 256 kernel's fused form.
// GROUPED: the rows of A belong to p.E experts (p.row_offsets, on the device) with weights of their own; the m-tile
// list is the concatenation of the experts' tile lists, as in the 256 x 256 kernel.  For expert layers at decode
// batch sizes, where an expert has a few dozen rows: 128-row tiles, and PERSISTENT -- such a launch is several rounds
// of tiles (8 experts x 224 tiles of gate+up rows), so one workgroup per compute unit walks them and the loads of
// the next tile go out before the current tile has ended (inside the kernel: PERSIST, cross).
// QUANT (with SWIGLU): the bf16 result is not stored but quantised to MXFP4 (p.Q, p.Qs) with the stand-alone
// quantiser's steps: the 32 outputs of a block are the 2 x 8 values of lane l and the 2 x 8 of lane l ^ 32.
#include "fp4_common.hpp"
#include "kernels.hpp"
#include "tile_common.hpp"
#include "tile_map.hpp"

namespace ave {
namespace {

constexpr int NM = 256, NN = 128, BK = 256;
constexpr int kRowBytes = BK / 2;                       // 128
// Geometry of the two forms.  Full: 256 rows of A per tile, stages of 48 KB, a ring of three.  HALF: 128 rows of A
// per tile -- waves 0-3 multiply, waves 4-7 load, always -- stages of 32 KB, a ring of four: a third more weight
// bytes in flight per compute unit, for shapes and expert layers with at most 128 rows (per expert), where the
// upper half of a 256-row tile would be loaded for nothing.
template <bool HALF>
struct Geo {
  static constexpr int kRows = HALF ? 128 : 256;            // rows of A and C per tile
  static constexpr int kOffB = kRows * kRowBytes;           // 16384 / 32768
  static constexpr int kStage = kOffB + NN * kRowBytes;     // 32768 / 49152
  static constexpr int kRing = HALF ? 4 : 3;
  static constexpr int kScaleBase = kRing * kStage;         // 131072 / 147456
  static constexpr int kALoads = HALF ? 4 : 8;              // 1 KB pieces of A per issuing wave and stage
  static constexpr int kDataLoads = kALoads + 4;
};
// a pair of stages: 256 A rows x 16 B, then B rows x 16 B in a 4 KB area of which the first 2 KB (128 rows) are
// read; the second 2 KB receive what issuing waves 2 and 3 load (repeats of row 127), so that all four issuing
// waves run the same two scale loads
constexpr int kScalePair = 8192;
template <bool HALF>
constexpr int kLds = Geo<HALF>::kScaleBase + 2 * kScalePair;   // 147456 / 163840
static_assert(kLds<false> <= 160 * 1024 && kLds<true> <= 160 * 1024, "LDS of one compute unit");
constexpr int kScaleLoads = 2;   // loads of an issuing wave for one pair of scale rows

// The loads of one issuing wave for one stage: eight 1 KB pieces of A to LDS addresses mda + 1024 i and four of B
// to mdb + 1024 i, as one asm statement that the waves outside the issuing group (waves 0-3: 0, waves 4-7: 1) jump over.
__device__ inline void dma16_stage_narrow(int wave_group, int group, unsigned mda, unsigned mdb, const void* ga, const void* gb,
                                          const unsigned (&a)[8], const unsigned (&b)[4]) {
  asm volatile(
      "s_cmp_eq_u32 %[wg], %[g]\n\t"
      "s_cbranch_scc0 1f\n\t"
      "s_mov_b32 m0, %[mda]\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a0], %[ga]\n\t"
      "s_mov_b32 m0, %[mdb]\n\t s_nop 0\n\t global_load_lds_dwordx4 %[b0], %[gb]\n\t"
      "s_add_u32 m0, %[mda], 0x0400\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a1], %[ga]\n\t"
      "s_add_u32 m0, %[mda], 0x0800\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a2], %[ga]\n\t"
      "s_add_u32 m0, %[mdb], 0x0400\n\t s_nop 0\n\t global_load_lds_dwordx4 %[b1], %[gb]\n\t"
      "s_add_u32 m0, %[mda], 0x0c00\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a3], %[ga]\n\t"
      "s_add_u32 m0, %[mda], 0x1000\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a4], %[ga]\n\t"
      "s_add_u32 m0, %[mdb], 0x0800\n\t s_nop 0\n\t global_load_lds_dwordx4 %[b2], %[gb]\n\t"
      "s_add_u32 m0, %[mda], 0x1400\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a5], %[ga]\n\t"
      "s_add_u32 m0, %[mda], 0x1800\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a6], %[ga]\n\t"
      "s_add_u32 m0, %[mdb], 0x0c00\n\t s_nop 0\n\t global_load_lds_dwordx4 %[b3], %[gb]\n\t"
      "s_add_u32 m0, %[mda], 0x1c00\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a7], %[ga]\n\t"
      "1:\n\t"
      :
      : [wg] "s"(__builtin_amdgcn_readfirstlane(wave_group)), [g] "s"(__builtin_amdgcn_readfirstlane(group)), [mda] "s"(__builtin_amdgcn_readfirstlane(mda)),
        [mdb] "s"(__builtin_amdgcn_readfirstlane(mdb)), [ga] "s"(ga), [gb] "s"(gb), [a0] "v"(a[0]), [a1] "v"(a[1]),
        [a2] "v"(a[2]), [a3] "v"(a[3]), [a4] "v"(a[4]), [a5] "v"(a[5]), [a6] "v"(a[6]), [a7] "v"(a[7]), [b0] "v"(b[0]),
        [b1] "v"(b[1]), [b2] "v"(b[2]), [b3] "v"(b[3])
      : "m0", "scc", "memory");
}

// The same for a 128-row A image: four pieces of A and four of B.
__device__ inline void dma16_stage_half(int wave_group, int group, unsigned mda, unsigned mdb, const void* ga, const void* gb,
                                        const unsigned (&a)[8], const unsigned (&b)[4]) {
  asm volatile(
      "s_cmp_eq_u32 %[wg], %[g]\n\t"
      "s_cbranch_scc0 1f\n\t"
      "s_mov_b32 m0, %[mda]\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a0], %[ga]\n\t"
      "s_mov_b32 m0, %[mdb]\n\t s_nop 0\n\t global_load_lds_dwordx4 %[b0], %[gb]\n\t"
      "s_add_u32 m0, %[mda], 0x0400\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a1], %[ga]\n\t"
      "s_add_u32 m0, %[mdb], 0x0400\n\t s_nop 0\n\t global_load_lds_dwordx4 %[b1], %[gb]\n\t"
      "s_add_u32 m0, %[mda], 0x0800\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a2], %[ga]\n\t"
      "s_add_u32 m0, %[mdb], 0x0800\n\t s_nop 0\n\t global_load_lds_dwordx4 %[b2], %[gb]\n\t"
      "s_add_u32 m0, %[mda], 0x0c00\n\t s_nop 0\n\t global_load_lds_dwordx4 %[a3], %[ga]\n\t"
      "s_add_u32 m0, %[mdb], 0x0c00\n\t s_nop 0\n\t global_load_lds_dwordx4 %[b3], %[gb]\n\t"
      "1:\n\t"
      :
      : [wg] "s"(__builtin_amdgcn_readfirstlane(wave_group)), [g] "s"(__builtin_amdgcn_readfirstlane(group)),
        [mda] "s"(__builtin_amdgcn_readfirstlane(mda)), [mdb] "s"(__builtin_amdgcn_readfirstlane(mdb)), [ga] "s"(ga),
        [gb] "s"(gb), [a0] "v"(a[0]), [a1] "v"(a[1]), [a2] "v"(a[2]), [a3] "v"(a[3]), [b0] "v"(b[0]), [b1] "v"(b[1]),
        [b2] "v"(b[2]), [b3] "v"(b[3])
      : "m0", "scc", "memory");
}

// 4 MFMAs of one K quarter: acc[nj][mi] += B-fragment nj x A-fragment mi
template <int KJ>
__device__ inline void mma_quarter(v16f (&acc)[2][2], const v4i (&bf)[2], const v4i (&af)[2], const int (&bs)[2],
                                   const int (&as)[2]) {
#pragma unroll
  for (int nj = 0; nj < 2; ++nj)
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) acc[nj][mi] = mfma32<KJ, KJ>(bf[nj], af[mi], acc[nj][mi], bs[nj], as[mi]);
}

// scheduling hint: one LDS read after every MFMA, four times
#define AVE_MFMA_DS_4                                         \
  _Pragma("unroll") for (int q_ = 0; q_ < 4; ++q_) {          \
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);        \
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);        \
  }                                                           \
  __builtin_amdgcn_sched_barrier(0);

template <bool SWIGLU, bool QUANT = false, bool SPLITK = false, bool GROUPED = false, bool HALF = false>
__global__ __launch_bounds__(512) void mx_narrow_kernel(MxArgs p, int m_tiles, int n_tiles) {
  using G = Geo<HALF>;
  constexpr int kRowsTile = G::kRows, kOffB = G::kOffB, kStage = G::kStage, kRing = G::kRing, kScaleBase = G::kScaleBase;
  constexpr int kDataLoads = G::kDataLoads;
  static_assert(SWIGLU || !QUANT, "the fused quantiser follows the fused SwiGLU");
  static_assert(!SPLITK || !SWIGLU, "K is split for the plain GEMM");
  static_assert(!SPLITK || !GROUPED, "K is split for the plain GEMM");
  constexpr int kTileN = SWIGLU ? NN / 2 : NN;   // output columns per tile
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int wm = w >> 1, wn = w & 1;   // wave (wm, wn) owns rows 64 wm .., columns 64 wn .. of the tile
  // SPLITK: workgroup pid is tile pid % tiles of K slice pid / tiles; a slice is p.slice_pairs pairs of stages (the
  // last one what is left), its fp32 sums go to p.P[slice][M][N] and launch_splitk_reduce adds the slices up.
  // GROUPED: persistent -- an expert layer at a decode batch is several rounds of tiles with few rows each, so one
  // workgroup per compute unit walks the tiles pid, pid + gridDim.x, ... and requests the next tile's first stages
  // before the finished tile's results leave (a workgroup per tile pays the start of the pipeline once per tile).
  constexpr bool PERSIST = GROUPED;
  // GROUPED, up to 256 experts (what the routing kernel takes): lane l keeps {first m-tile, m-tiles, first row, end
  // row} (clamped to [0, M]) of experts l, l + 64, l + 128 and l + 192 in registers, read once; the list's true length
  // replaces the host's bound (rows / tile + experts).  More experts than that: the caller's table is walked entry by
  // entry for every tile (locate_group_tile).
  constexpr int kExpertSets = 4;
  int g_first[kExpertSets], g_nt[kExpertSets], g_r0[kExpertSets], g_r1[kExpertSets];
  if (GROUPED && p.E <= 64 * kExpertSets) {
    int carry = 0;   // m-tiles of the experts in the sets before
#pragma unroll
    for (int q = 0; q < kExpertSets; ++q) {
      const int e = 64 * q + lane;
      int r0 = 0, r1 = 0;
      if (e < p.E) {
        r0 = p.row_offsets[e];
        r1 = p.row_offsets[e + 1];
        r0 = r0 < 0 ? 0 : (r0 > p.M ? p.M : r0);
        r1 = r1 < 0 ? 0 : (r1 > p.M ? p.M : r1);
      }
      const int nt = r1 > r0 ? (r1 - r0 + kRowsTile - 1) / kRowsTile : 0;
      int incl = nt;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(incl, d);
        if (lane >= d) incl += up;
      }
      g_first[q] = carry + incl - nt;
      g_nt[q] = nt;
      g_r0[q] = r0;
      g_r1[q] = r1;
      carry += __builtin_amdgcn_readlane(incl, 63);
    }
    m_tiles = carry;
  }
  const int total = m_tiles * n_tiles * (SPLITK ? p.slices : 1);
  int pid = blockIdx.x;
  // rows [m_begin, m_end) of A and C: m_end is the end of the matrix, or of the expert
  int tm, tn, slice = 0, m_begin, m_end, expert, n_begin;
  auto locate = [&](int id) {   // false: a slot behind the last tile of the grouped list; uniform for the workgroup
    if (SPLITK) {
      slice = id / (m_tiles * n_tiles);
      id -= slice * (m_tiles * n_tiles);
    }
    map_tile(id, m_tiles, n_tiles, tm, tn);
    m_begin = tm * kRowsTile;
    m_end = p.M;
    expert = 0;
    n_begin = tn * kTileN;
    if (!GROUPED) return true;
    if (p.E <= 64 * kExpertSets) {
#pragma unroll
      for (int q = 0; q < kExpertSets; ++q) {
        const unsigned long long hits = __ballot(tm >= g_first[q] && tm < g_first[q] + g_nt[q]);
        if (hits) {
          const int e = __builtin_ctzll(hits);
          expert = 64 * q + e;
          m_begin = __builtin_amdgcn_readlane(g_r0[q], e) + (tm - __builtin_amdgcn_readlane(g_first[q], e)) * kRowsTile;
          m_end = __builtin_amdgcn_readlane(g_r1[q], e);
          return true;
        }
      }
      return false;
    }
    return locate_group_tile(p.row_offsets, p.E, p.M, kRowsTile, tm, expert, m_begin, m_end);
  };
  {
    bool have = pid < total && locate(pid);
    while (PERSIST && !have && (pid += (int)gridDim.x) < total) have = locate(pid);
    if (!have) return;
  }
  const int k_pair0 = SPLITK ? slice * p.slice_pairs : 0;
  const unsigned row_bytes = (unsigned)p.K / 2, row_scales = (unsigned)p.K / 32;
  const int pairs_left = p.K / (2 * BK) - k_pair0;
  // whole pairs of stages; what K holds behind them (1..15 blocks of 32, never with SPLITK) is multiplied at the end
  const int stages = SPLITK ? 2 * (pairs_left < p.slice_pairs ? pairs_left : p.slice_pairs) : 2 * (p.K / (2 * BK));   // even, >= 2

  // ---- per-lane source offsets of the direct-to-LDS loads (issuing wave wi = w & 3) --------------------------
  // A: instruction i covers tile rows (8 wi + i) * 8 .. + 7; B: (4 wi + i) * 8 .. + 7; lane -> (row, swizzled chunk).
  // Scale rows: lane -> tile row 64 wi + lane of A, and of B as far as the tile's 128 rows go.
  // Rows past the end of a matrix are clamped to its last row: their products land in C elements never stored.
  const int wi = w & 3;
  unsigned a_off[8], b_off[4], as_off, bs_off;
  bool upper_idle;
  int issuers;
  size_t expert_rows;
  const uint8_t *ga, *gb, *gas, *gbs;   // data advance by a stage, scales by a pair per issue
  // row of B behind row `row` (0..127) of the tile's B image, clamped to a valid row
  auto b_image_row = [&](int row) {
    if (SWIGLU) {
      // image rows 64 wn + j: j < 32 the gate row, j >= 32 the up row of output column 32 wn + (j & 31)
      int n = n_begin + 32 * (row >> 6) + (row & 31);
      n = n < p.N ? n : p.N - 1;
      return (row & 32) ? p.N + n : n;
    }
    const int n = n_begin + row;
    return n < p.N ? n : p.N - 1;
  };
  auto setup_tile = [&]() {   // of the tile that locate() has just described
    const int lr = lane >> 3, cprime = lane & 7;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = (wi * G::kALoads + (i % G::kALoads)) * 8 + lr;   // HALF: pieces 4 .. 7 are not issued
      int am = m_begin + row;
      am = am < m_end ? am : m_end - 1;
      a_off[i] = (unsigned)am * row_bytes + (unsigned)((cprime ^ ((row >> 1) & 7)) * 16);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = (wi * 4 + i) * 8 + lr;
      const int bn = b_image_row(row);
      b_off[i] = (unsigned)bn * row_bytes + (unsigned)((cprime ^ ((row >> 1) & 7)) * 16);
    }
    int am = m_begin + wi * 64 + lane;
    am = am < m_end ? am : m_end - 1;
    int brow = wi * 64 + lane;
    brow = brow < NN ? brow : NN - 1;
    const int bn = b_image_row(brow);
    as_off = (unsigned)am * row_scales;
    bs_off = (unsigned)bn * row_scales;
    // Waves 4-7 own rows 128 .. 255 of the tile.  When those rows lie past the end of A (at most 128 rows in all)
    // they multiply nothing, and they take over the loads from waves 0-3: every SIMD then has one wave that
    // multiplies and one that loads, and a stalled load instruction stalls no MFMA.
    upper_idle = HALF || m_begin + 128 >= m_end;
    issuers = __builtin_amdgcn_readfirstlane(upper_idle ? 1 : 0);
    // a pair of stages is 256 bytes of a data row and 16 scale bytes
    expert_rows = (size_t)expert * (SWIGLU ? 2 : 1) * p.N;   // an expert holds N, or N gate + N up rows
    ga = p.A + (size_t)k_pair0 * (2 * kRowBytes);
    gb = p.B + expert_rows * row_bytes + (size_t)k_pair0 * (2 * kRowBytes);
    gas = p.As + (size_t)k_pair0 * 16;
    gbs = p.Bs + expert_rows * row_scales + (size_t)k_pair0 * 16;
  };
  setup_tile();
  const unsigned lds_base = (unsigned)(uintptr_t)lds;
  auto issue_data = [&](unsigned sb) {
    if constexpr (HALF) dma16_stage_half(w >> 2, issuers, sb + (unsigned)wi * 4096, sb + kOffB + (unsigned)wi * 4096, ga, gb, a_off, b_off);
    else dma16_stage_narrow(w >> 2, issuers, sb + (unsigned)wi * 8192, sb + kOffB + (unsigned)wi * 4096, ga, gb, a_off, b_off);
    ga += kRowBytes;
    gb += kRowBytes;
  };
  auto issue_scale_pair = [&](int pair) {
    dma16_scale_rows(w >> 2, issuers, lds_base + kScaleBase + (pair & 1) * kScalePair + (unsigned)wi * 1024, gas, gbs, as_off,
                     bs_off);
    gas += 16;
    gbs += 16;
  };
  auto stage_buffer = [&](int s) { return lds_base + (unsigned)(s % kRing) * kStage; };

  // ---- per-lane fragment read addresses ------------------------------------------------------------------------
  const int rho = lane & 31, h = lane >> 5;
  const int a_row = wm * 64 + rho;            // + 32 mi
  const int b_row = wn * 64 + pi_row(rho);    // + 32 nj
  const unsigned a_frag = a_row * kRowBytes + (((4 * h) ^ ((a_row >> 1) & 7)) * 16);
  const unsigned b_frag = kOffB + b_row * kRowBytes + (((4 * h) ^ ((b_row >> 1) & 7)) * 16);
  const unsigned a_sc = lds_base + kScaleBase + a_row * 16;             // + mi * 512
  const unsigned b_sc = lds_base + kScaleBase + NM * 16 + b_row * 16;   // + nj * 512

  v16f acc[2][2];
  v4i af0[2], bf0[2], af1[2], bf1[2];
  int as_cur[2], bs_cur[2];
  v4i as_pair[2], bs_pair[2];   // the 16 scale bytes of each fragment row for a pair of stages

#define AVE_READ_FRAGS(dst_a, dst_b, sb, KJ)                                                                    \
  _Pragma("unroll") for (int i = 0; i < 2; ++i) dst_a[i] = lds_read16((sb) + (a_frag ^ ((KJ) * 16)) + i * 4096); \
  _Pragma("unroll") for (int i = 0; i < 2; ++i) dst_b[i] = lds_read16((sb) + (b_frag ^ ((KJ) * 16)) + i * 4096);
#define AVE_READ_SCALE_PAIR(pair)                                                                              \
  _Pragma("unroll") for (int i = 0; i < 2; ++i) as_pair[i] = lds_read16(a_sc + ((pair) & 1) * kScalePair + i * 512); \
  _Pragma("unroll") for (int i = 0; i < 2; ++i) bs_pair[i] = lds_read16(b_sc + ((pair) & 1) * kScalePair + i * 512);
  // stage parity P of the pair, lane half h -> dword 2P + h of the row's 16 bytes
#define AVE_PICK_SCALES(P)                                                                                   \
  _Pragma("unroll") for (int i = 0; i < 2; ++i) as_cur[i] = h ? as_pair[i][2 * (P) + 1] : as_pair[i][2 * (P)]; \
  _Pragma("unroll") for (int i = 0; i < 2; ++i) bs_cur[i] = h ? bs_pair[i][2 * (P) + 1] : bs_pair[i][2 * (P)];

  // Issue order of an issuing wave, with R = kRing: S0 D0 D1 [S1 D2 .. D(R-1)], then behind the barrier of stage s:
  // [S((s+R)/2) if s + R is even] D(s+R).  Loads to LDS complete in issue order, so "stage s+1 has landed" is a bound
  // on the number of loads still outstanding: those issued after D(s+1), which are D(s+2) .. D(s+R-1) with the one
  // pair of scale rows that precedes an even stage among them -- fewer at the end of K.
  constexpr int kScaleIssueParity = kRing & 1;   // a stage of this parity issues a pair of scale rows with its data
  constexpr int kWaitEven = (kRing - 2) * kDataLoads + kScaleLoads;
  constexpr int kWaitOdd = (kRing - 2) * kDataLoads + (kRing == 4 ? kScaleLoads : 0);
  constexpr int kWaitTailOdd = kDataLoads;       // in front of the last two stages: D(stages-1) alone
  constexpr bool kTailIssues = kRing == 3;       // four stages from the end, stage s + R still exists for R = 3 only
  auto issue_first_stages = [&]() {
    issue_scale_pair(0);
    issue_data(stage_buffer(0));
    issue_data(stage_buffer(1));
    if (stages > 2) {
      issue_scale_pair(1);
      issue_data(stage_buffer(2));
      if (kRing == 4) issue_data(stage_buffer(3));
    }
  };
  issue_first_stages();
  bool first_tile = true;
  for (;;) {   // one tile per trip; a single trip unless PERSIST
  // Stage 0 has landed when only the loads issued behind it are outstanding.  From the second tile on that count holds
  // for the waves that only load (the 128-row tiles: waves 4-7); a wave that has also stored the previous tile's
  // results waits for everything it has in flight.
  if (first_tile || HALF) {
    if (stages > 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((kRing - 1) * kDataLoads + kScaleLoads) : "memory");
    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kDataLoads) : "memory");
  } else {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  __syncthreads();
  const bool loader = w >= 4 && upper_idle;   // of the tile being computed (setup_tile below is for the next one)
  const int c_m_begin = m_begin, c_m_end = m_end, c_n_begin = n_begin;   // the tile being computed
  // PERSIST, whole groups of four stages and no K tail: the ring does not run dry between two tiles.  Four stages
  // before the tile's end -- where the loads of a single tile stop -- the next tile is looked up and the loading waves
  // send its first four stages out one by one into the buffers as they are consumed, in the order and with the wait
  // counts of the steady state (a tile's stage j then sits in buffer j % 4 and its pair of scales in buffer
  // (j / 2) % 2, as ever).  With 128-row tiles the roles are fixed: waves 0-3 multiply and never load.
  const bool can_cross = PERSIST && HALF && stages >= 4 && (stages & 3) == 0 && p.K % (2 * BK) == 0;
  bool have_next = false, crossed = false;
  auto cross = [&](bool loads) {
    if (can_cross) {
      while (!have_next && (pid += (int)gridDim.x) < total) have_next = locate(pid);
      crossed = true;
      if (loads && have_next) setup_tile();
    }
  };
  if (loader) {
    // the loading waves of a tile without upper rows: the waits, barriers and issues of the stages below, nothing else
#define AVE_LOAD_STAGE(WAIT, ISSUE, PARITY)                                  \
  {                                                                          \
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(WAIT) : "memory");              \
    __syncthreads();                                                         \
    if (ISSUE) {                                                             \
      if ((PARITY) == kScaleIssueParity) issue_scale_pair((s + kRing) >> 1); \
      issue_data(stage_buffer(s));                                           \
    }                                                                        \
  }
    int s = 0;
    for (; s + 1 + kRing < stages; ++s) {
      AVE_LOAD_STAGE(kWaitEven, true, 0)
      ++s;
      AVE_LOAD_STAGE(kWaitOdd, true, 1)
    }
    cross(true);
    if (have_next) {   // only after cross(): the tile's last four stages issue the next tile's first four
      AVE_LOAD_STAGE(kWaitEven, true, 0)
      ++s;
      AVE_LOAD_STAGE(kWaitOdd, true, 1)
      ++s;
      AVE_LOAD_STAGE(kWaitEven, true, 0)
      ++s;
      AVE_LOAD_STAGE(kWaitOdd, true, 1)
    } else {
    if (stages > 2) {
      AVE_LOAD_STAGE(kWaitEven, kTailIssues, 0)
      ++s;
      AVE_LOAD_STAGE(kWaitTailOdd, false, 1)
      ++s;
    }
    AVE_LOAD_STAGE(0, false, 0)
    ++s;
    AVE_LOAD_STAGE(0, false, 1)
    }
#undef AVE_LOAD_STAGE
    if (!PERSIST) return;
  } else {
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = v16f{};
  AVE_READ_SCALE_PAIR(0)
  AVE_READ_FRAGS(af0, bf0, lds_base, 0)
  AVE_PICK_SCALES(0)

  // One stage; PARITY is its position in its pair of stages, WAIT the number of loads that may stay outstanding
  // at its barrier, ISSUE whether stage s + kRing exists, READ_NEXT whether stage s + 1 does.  All four are
  // compile-time constants: a stage must stay one basic block, or the compiler sinks the MFMAs (pure arithmetic
  // to it) out of the loop body to where the accumulators are used.
#define AVE_STAGE(WAIT, ISSUE, READ_NEXT, PARITY)                                                            \
  {                                                                                                          \
    const unsigned sb = stage_buffer(s), sbn = stage_buffer(s + 1);                                          \
    AVE_READ_FRAGS(af1, bf1, sb, 1)                                                                          \
    mma_quarter<0>(acc, bf0, af0, bs_cur, as_cur);                                                           \
    AVE_MFMA_DS_4                                                                                            \
    AVE_READ_FRAGS(af0, bf0, sb, 2)                                                                          \
    mma_quarter<1>(acc, bf1, af1, bs_cur, as_cur);                                                           \
    AVE_MFMA_DS_4                                                                                            \
    AVE_READ_FRAGS(af1, bf1, sb, 3)                                                                          \
    mma_quarter<2>(acc, bf0, af0, bs_cur, as_cur);                                                           \
    AVE_MFMA_DS_4                                                                                            \
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(WAIT) : "memory");                                   \
    __syncthreads();                                                                                         \
    if (ISSUE && !HALF) {   /* 128-row tiles: the waves that run these stages never load */                 \
      if ((PARITY) == kScaleIssueParity) issue_scale_pair((s + kRing) >> 1);                                 \
      issue_data(sb);                                                                                        \
      __builtin_amdgcn_sched_barrier(0);                                                                     \
    }                                                                                                        \
    if (READ_NEXT) {                                                                                         \
      if ((PARITY) == 1) { AVE_READ_SCALE_PAIR((s + 1) >> 1) }                                               \
      AVE_READ_FRAGS(af0, bf0, sbn, 0)                                                                       \
    }                                                                                                        \
    mma_quarter<3>(acc, bf1, af1, bs_cur, as_cur);                                                           \
    if (READ_NEXT) {                                                                                         \
      AVE_MFMA_DS_4                                                                                          \
      AVE_PICK_SCALES((PARITY) ^ 1)                                                                          \
    }                                                                                                        \
    __builtin_amdgcn_sched_barrier(0);                                                                       \
  }

  int s = 0;
  for (; s + 1 + kRing < stages; ++s) {   // stages s + R and s + 1 + R exist
    AVE_STAGE(kWaitEven, true, true, 0)
    ++s;
    AVE_STAGE(kWaitOdd, true, true, 1)
  }
  cross(false);   // the loading waves do the same four stages before their tile's end and issue the next tile's loads
  if (stages > 2) {               // four stages left: with a ring of three the last load goes out in the first of them
    AVE_STAGE(kWaitEven, kTailIssues, true, 0)
    ++s;
    AVE_STAGE(kWaitTailOdd, false, true, 1)
    ++s;
  }
  AVE_STAGE(0, false, true, 0)
  ++s;
  AVE_STAGE(0, false, false, 1)
#undef AVE_STAGE
#undef AVE_READ_FRAGS
#undef AVE_READ_SCALE_PAIR
#undef AVE_PICK_SCALES

  if constexpr (!SPLITK) {
    // K % 512 elements behind the last whole pair of stages: straight from global memory, two blocks of 32 per MFMA
    // (lane half h: block 2j + h), every lane the 16 bytes and the scale byte of its own fragment rows.  A lane half
    // behind the last block fetches block 2j instead (inside the row) and multiplies zeros under the scale 2^0.  The
    // tiles of this kernel are small and few, so the poorly coalesced loads of the tail cost less than the 256 x 256
    // tiling of the kernel that stages its tail would.
    const int tail_blocks = (p.K % (2 * BK)) / 32;
    if (tail_blocks != 0) {
      const unsigned first_block = (unsigned)(p.K / (2 * BK)) * 16u;
      const uint8_t* tB = p.B + expert_rows * row_bytes;
      const uint8_t* tBs = p.Bs + expert_rows * row_scales;
      unsigned ar[2], br[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int am = m_begin + a_row + 32 * i;
        ar[i] = (unsigned)(am < m_end ? am : m_end - 1);
        br[i] = (unsigned)b_image_row(b_row + 32 * i);
      }
      for (int j = 0; 2 * j < tail_blocks; ++j) {
        const bool have = 2 * j + h < tail_blocks;
        const unsigned blk = first_block + (unsigned)(have ? 2 * j + h : 2 * j);
        v4i ta[2], tb[2];
        int tas[2], tbs[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          ta[i] = *reinterpret_cast<const v4i*>(p.A + (size_t)ar[i] * row_bytes + blk * 16u);
          tas[i] = p.As[(size_t)ar[i] * row_scales + blk];
          tb[i] = *reinterpret_cast<const v4i*>(tB + (size_t)br[i] * row_bytes + blk * 16u);
          tbs[i] = tBs[(size_t)br[i] * row_scales + blk];
          if (!have) {
            ta[i] = v4i{0, 0, 0, 0};
            tb[i] = v4i{0, 0, 0, 0};
            tas[i] = 0x7f;
            tbs[i] = 0x7f;
          }
        }
        mma_quarter<0>(acc, tb, ta, tbs, tas);
      }
    }
  }
  // pinned: otherwise the MFMAs of the last stages are sunk below the address arithmetic of the stores
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) asm volatile("" : "+v"(acc[i][j]));
  }   // multiplying waves
  // ---- end of the tile: the next one's first stages go out before this one's results do (unless they already have) --
  if (PERSIST && !crossed) {
    while (!have_next && (pid += (int)gridDim.x) < total) have_next = locate(pid);
    __syncthreads();   // every wave is done reading the ring
    if (have_next) {
      setup_tile();
      issue_first_stages();
    }
  }
  if (!loader) {
  if constexpr (SWIGLU) {
    // acc[0][mi] holds the gate and acc[1][mi] the up values of row m_begin + 64 wm + 32 mi + c, outputs
    // n_begin + 32 wn + 16 piece + 8 q + 0..7 (registers 8 piece .. 8 piece + 7)
    const int c = lane & 31, q = lane >> 5;
    const bool vec_ok = (p.N % 8 == 0) && ((reinterpret_cast<uintptr_t>(p.C) & 15) == 0);
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) {
      const int m = c_m_begin + wm * 64 + 32 * mi + c;
      if (m >= c_m_end) continue;
      uint16_t* crow = QUANT ? nullptr : p.C + (size_t)m * p.N;
      const v16f& g = acc[0][mi];
      const v16f& u = acc[1][mi];
      v4i obits[2];   // QUANT: the 2 x 8 bf16 results of this lane
#pragma unroll
      for (int piece = 0; piece < 2; ++piece) {
        const int n = c_n_begin + 32 * wn + 16 * piece + 8 * q;
        float hv[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) hv[e] = silu(g[8 * piece + e]) * u[8 * piece + e];
        v4i o;
        o[0] = (int)pack_bf16x2(hv[0], hv[1]);
        o[1] = (int)pack_bf16x2(hv[2], hv[3]);
        o[2] = (int)pack_bf16x2(hv[4], hv[5]);
        o[3] = (int)pack_bf16x2(hv[6], hv[7]);
        if constexpr (QUANT) {
          obits[piece] = o;
          continue;
        }
        if (vec_ok && n + 8 <= p.N) {
          *reinterpret_cast<v4i*>(crow + n) = o;
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (n + e < p.N) crow[n + e] = (uint16_t)(((unsigned)o[e >> 1] >> (16 * (e & 1))) & 0xFFFF);
        }
      }
      if constexpr (QUANT) {
        // the stand-alone quantiser's steps on the bf16 values (N % 32 == 0: a block lies inside the matrix or
        // outside it as a whole, so both lanes of the exchange are in the same state)
        float v[2][8];
#pragma unroll
        for (int piece = 0; piece < 2; ++piece)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            v[piece][2 * j] = __builtin_bit_cast(float, (unsigned)obits[piece][j] << 16);
            v[piece][2 * j + 1] = __builtin_bit_cast(float, (unsigned)obits[piece][j] & 0xFFFF0000u);
          }
        unsigned amax = abs_max_bits(v[0]);
        {
          const unsigned second = abs_max_bits(v[1]);
          amax = amax > second ? amax : second;
        }
        amax = lane_xor_max_bits(amax, 32);
        const int byte = mx_scale_byte(amax);
        const float scale = mx_scale_value(byte);
        const int n0 = c_n_begin + 32 * wn;   // first output of the block
        if (n0 < p.N) {
#pragma unroll
          for (int piece = 0; piece < 2; ++piece) {
            unsigned codes = 0;
            codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(codes, v[piece][0], v[piece][1], scale, 0);
            codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(codes, v[piece][2], v[piece][3], scale, 1);
            codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(codes, v[piece][4], v[piece][5], scale, 2);
            codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(codes, v[piece][6], v[piece][7], scale, 3);
            *reinterpret_cast<unsigned*>(p.Q + (size_t)m * (q_row_cols(p) / 2) + (n0 + 16 * piece + 8 * q) / 2) = byte == 0xFF ? 0u : codes;
          }
          if (q == 0) p.Qs[(size_t)m * (q_row_cols(p) / 32) + n0 / 32] = (uint8_t)byte;
        }
      }
    }
  } else if constexpr (SPLITK) {
    store_wave_block_f32<2, 2>(acc, p.P + (size_t)slice * (size_t)p.M * (size_t)p.N, p.N, c_m_begin + wm * 64, p.M,
                               c_n_begin + wn * 64, lane);
  } else {
    store_wave_block<2, 2>(acc, p.C, p.N, c_m_begin + wm * 64, c_m_end, c_n_begin + wn * 64, lane, 1.0f);
  }
  }   // multiplying waves
  if (!PERSIST || !have_next) return;
  first_tile = false;
  }   // next tile
}

}  // namespace

// What the kernel needs: the plain or the SwiGLU-fused GEMM (also grouped) on whole pairs of stages, aligned scale
// rows, 32-bit offsets over the rows of A and over one expert's weight rows (2N of them with SwiGLU).
bool mx_narrow_supports(const MxArgs& p) {
  if (p.row_offsets && p.E <= 0) return false;
  if (p.Q && (!p.swiglu || !p.Qs || p.N % 32 != 0 || (reinterpret_cast<uintptr_t>(p.Q) & 3))) return false;
  if (p.M <= 0 || p.N <= 0 || p.K < 2 * BK || p.K % 32 != 0) return false;
  // a K tail is fetched in 16-byte pieces straight from A and B
  if (p.K % (2 * BK) != 0 && ((reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.B)) & 15) != 0) return false;
  const uint64_t b_rows = (uint64_t)p.N * (p.swiglu ? 2 : 1);
  if ((uint64_t)p.M * (uint64_t)(p.K / 2) >= (1ull << 32) || b_rows * (uint64_t)(p.K / 2) >= (1ull << 32)) return false;
  if ((reinterpret_cast<uintptr_t>(p.As) & 15) || (reinterpret_cast<uintptr_t>(p.Bs) & 15)) return false;
  return true;
}

// Where it pays: more rows than the weight-streaming kernel takes (that kernel has no fused quantiser: with one,
// any number of rows), and no more tiles than compute units -- the shapes whose 256 x 256 tiling would leave half of
// the chip idle.  Grouped: an expert layer at a decode batch, at most 128 rows per expert on average (the host
// does not know the distribution) -- every expert then streams its weights through tiles with few rows, where the
// ring of three stage buffers and the idle upper waves count.
bool mx_narrow_preferred(const MxArgs& p) {
  if (!mx_narrow_supports(p)) return false;
  if (p.row_offsets) return (long)p.M <= 128L * p.E;
  const int cus = compute_units(), tile_n = p.swiglu ? NN / 2 : NN;
  if (p.M <= 64 && !p.Q) {
    // Up to 64 rows belong to the weight-streaming kernel -- except 33..64 rows against so many weight rows that the
    // 128-row tiles make one nearly full round of the compute units: there this kernel is 2-15 % faster (N = 28672 /
    // 32768, K = 4096: 17.6 / 18.8 us at 40 rows against 19.6 / 21+ us; with the fused SwiGLU, 2 x 14336 weight
    // rows: 16.6 against 18.7 us; at three quarters of a round the two are level, below that the rings win).
    if (p.M <= 32) return false;
    const long tiles = (p.N + tile_n - 1) / tile_n;
    return cus > 0 && tiles <= cus && 8 * tiles >= 7L * cus;
  }
  const long tiles = (long)((p.M + NM - 1) / NM) * ((p.N + tile_n - 1) / tile_n);
  return cus > 0 && tiles <= cus;
}

namespace {
template <bool SWIGLU, bool QUANT, bool GROUPED, bool HALF>
hipError_t launch_narrow(const MxArgs& p, hipStream_t s, int n_tiles) {
  // grouped: upper bound of the concatenated tile list, one partly filled tile per expert at most
  const int m_tiles = (p.M + Geo<HALF>::kRows - 1) / Geo<HALF>::kRows + (GROUPED ? p.E : 0);
  if (hipError_t e = allow_dynamic_lds<mx_narrow_kernel<SWIGLU, QUANT, false, GROUPED, HALF>>(kLds<HALF>); e != hipSuccess) return e;
  long grid = (long)m_tiles * n_tiles;
  if (GROUPED) {   // persistent: one workgroup per compute unit (a multiple of 8, so that a workgroup's tiles stay on its XCD)
    const int cus = compute_units();
    if (cus <= 0) return hipErrorInvalidDevice;
    grid = grid < cus ? grid : cus;
  }
  hipLaunchKernelGGL((mx_narrow_kernel<SWIGLU, QUANT, false, GROUPED, HALF>), dim3((unsigned)grid), dim3(512),
                     kLds<HALF>, s, p, m_tiles, n_tiles);
  return hipGetLastError();
}
template <bool GROUPED, bool HALF>
hipError_t launch_narrow_form(const MxArgs& p, hipStream_t s, int n_tiles) {
  if (p.swiglu && p.Q) return launch_narrow<true, true, GROUPED, HALF>(p, s, n_tiles);
  if (p.swiglu) return launch_narrow<true, false, GROUPED, HALF>(p, s, n_tiles);
  return launch_narrow<false, false, GROUPED, HALF>(p, s, n_tiles);
}
}  // namespace

// 128-row tiles (waves 0-3 multiply, waves 4-7 load, a ring of four stages) where no tile would have upper rows
// -- at most 128 rows in all, and every grouped launch (experts with more rows get more tiles) -- and wherever they
// do not outnumber the compute units.
hipError_t launch_mx_narrow(const MxArgs& p, hipStream_t s) {
  const int tile_n = p.swiglu ? NN / 2 : NN;
  const int n_tiles = (p.N + tile_n - 1) / tile_n;
  if (p.row_offsets) return launch_narrow_form<true, true>(p, s, n_tiles);
  // 128-row tiles also for more rows while they do not outnumber the compute units: twice the workgroups
  const int cus = compute_units();
  if (p.M <= 128 || (cus > 0 && (long)((p.M + 127) / 128) * n_tiles <= cus)) return launch_narrow_form<false, true>(p, s, n_tiles);
  return launch_narrow_form<false, false>(p, s, n_tiles);
}

hipError_t launch_mx_narrow_splitk(const MxArgs& p, hipStream_t s) {
  const int n_tiles = (p.N + NN - 1) / NN;
  if (p.M <= 128 || p.half_rows) {
    const int m_tiles = (p.M + 127) / 128;
    if (hipError_t e = allow_dynamic_lds<mx_narrow_kernel<false, false, true, false, true>>(kLds<true>); e != hipSuccess) return e;
    hipLaunchKernelGGL((mx_narrow_kernel<false, false, true, false, true>), dim3((unsigned)(m_tiles * n_tiles * p.slices)),
                       dim3(512), kLds<true>, s, p, m_tiles, n_tiles);
  } else {
    const int m_tiles = (p.M + NM - 1) / NM;
    if (hipError_t e = allow_dynamic_lds<mx_narrow_kernel<false, false, true>>(kLds<false>); e != hipSuccess) return e;
    hipLaunchKernelGGL((mx_narrow_kernel<false, false, true>), dim3((unsigned)(m_tiles * n_tiles * p.slices)), dim3(512),
                       kLds<false>, s, p, m_tiles, n_tiles);
  }
  if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
  return launch_splitk_reduce(p.P, p.C, (size_t)p.M * (size_t)p.N, p.slices, s);
}

}  // namespace ave
