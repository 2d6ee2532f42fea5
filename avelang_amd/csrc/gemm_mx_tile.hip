// MXFP4 GEMM for gfx950, compute-bound shapes: 256x256 output tile per workgroup, EIGHT
// wavefronts (two per SIMD) of 64(m) x 128(n) each, v_mfma_scale_f32_32x32x64_f8f6f4 with the
// E8M0 scales fed through the instruction's scale operands, fp32 accumulation (128 registers
// per lane), bf16 round-to-nearest-even epilogue.  Also serves the grouped (MoE) GEMM: the
// m-tile list is then the concatenation of the experts' tile lists, found from row_offsets on
// the device.
//
// Two waves per SIMD matter on this part: with a single wave, every LDS read and every
// global->LDS load the wave issues sits in the same instruction stream as its MFMAs; with two,
// one wave's MFMAs run under the other's memory instructions.
//
// Data movement per K stage of 256 elements (128 bytes per row):
//   global -> LDS with global_load_lds_dwordx4 (no register staging).  One wave instruction
//   moves 8 rows x 128 B: 8 consecutive lanes fetch one full 128-byte line.  A lane's 16 bytes
//   land at LDS address base + 16*lane, so the LDS image is row-major [256][128 B]; the XOR
//   swizzle that makes the MFMA fragment reads conflict-free is applied on the *source* side:
//   LDS chunk c' of row r holds global chunk c' ^ ((r >> 1) & 7).  (ds_read_b128 is served 16
//   lanes at a time over 64 banks: 16 consecutive rows must map to 16 distinct 16-byte slots
//   of a 256-byte bank line, which (r & 1, (r >> 1) & 7) does.)
//   Scales: per pair of stages as [256 rows][16 B] per operand when K % 512 == 0 (one
//   global_load_lds_dwordx4 per 64 rows and pair), else [256 rows][8 B] per stage as dwords.
//   Two stage buffers; one barrier per stage, placed before the last quarter of the stage so
//   that the MFMAs of that quarter cover the first fragment reads of the next stage.
//   With pair scales, waves 0-3 issue every load of the workgroup, and with more tiles than
//   compute units one persistent workgroup per compute unit walks the tiles and requests the
//   next tile's first stage before the finished tile's C leaves.
//
// K order inside a stage: MFMA kj (0..3) of lane half h consumes the 32-element block
// 4h + kj.  A lane's four blocks are then one contiguous 64-byte run and its four scale bytes
// are one dword, selected per MFMA by the instruction's byte-select (op_sel = kj).
//
// MFMA operand roles: srcA carries rows of B (n), srcB carries rows of A (m), so a lane's 16
// results are 16 values of ONE row of C.  B rows are handed to the fragment in the order
// pi(8u+4q+v) = 16(u/2) + 8q + 4(u%2) + v, which makes those 16 values two runs of 8
// consecutive n: the epilogue stores two 16-byte pieces per 32x32 block.
#include <atomic>

#include "fp4_common.hpp"
#include "kernels.hpp"
#include "tile_common.hpp"
#include "tile_map.hpp"

#ifndef AVE_NO_SC64
#define AVE_NO_SC64 0   // 1: build without the 64-byte scale chunk forms (A/B measurements)
#endif

namespace ave {
namespace {

constexpr int BM = 256, BN = 256, BK = 256;
constexpr int kWaves = 8;
constexpr int kRowBytes = BK / 2;                    // 128
constexpr int kOffA = 0;
constexpr int kOffB = BM * kRowBytes;                // 32768
// Scales, two ways (template parameter SC16 of the kernel):
//  * per stage, inside the stage buffer: [256 rows][8 B] per operand, moved with global_load_lds_dword;
//  * per PAIR of stages (K % 512 == 0), in two buffers of their own behind the stage buffers:
//    [256 rows][16 B] per operand, moved with global_load_lds_dwordx4 -- one instruction per wave and
//    pair of stages instead of four.  The dword form costs far more than its 4 KB per stage suggest:
//    without the scale loads the kernel runs as fast as without any loads at all.
constexpr int kOffAs = kOffB + BN * kRowBytes;       // 65536
constexpr int kOffBs = kOffAs + BM * (BK / 32);      // +2048
constexpr int kStageBytes = kOffBs + BN * (BK / 32); // 69632
constexpr int kLdsBytes = 2 * kStageBytes;           // 139264
constexpr int kDataStage = kOffAs;                   // SC16: a stage buffer holds data only
constexpr int kScaleBase16 = 2 * kDataStage;         // 131072
constexpr int kScalePair16 = (BM + BN) * 16;         // 8192 per pair of stages: A rows, then B rows
constexpr int kTableExperts = 256;   // experts whose tile ranges the grouped forms keep in LDS (what the routing kernel takes)
constexpr int kGroupTable16 = kScaleBase16 + 2 * kScalePair16;   // 147456: kTableExperts entries of 16 bytes, the experts' tile ranges
constexpr int kTouchLead = 8;   // stages between the look-ahead touches of the next tile's panels and the tile's end (even)
constexpr int kTouchSink16 = kGroupTable16 + kTableExperts * 16;   // 151552: 4 x 256 bytes that the look-ahead touches land in
constexpr int kLdsBytes16 = kTouchSink16 + 4 * 256;              // 152576
// CH = 4: scales by chunks of four pairs of stages, [256 rows][64 B] per operand in ONE buffer of 32 KB behind the stage
// buffers -- all of the 160 KB, so only for the forms that need neither the experts' table nor the touches' sink
constexpr int kLdsBytes64 = kScaleBase16 + (BM + BN) * 64;        // 163840


// 8 MFMAs of one K quarter: acc[nj][mi] += B-fragment nj x A-fragment mi
template <int KJ>
__device__ inline void mma_quarter(v16f (&acc)[4][2], const v4i (&bf)[4], const v4i (&af)[2], const int (&bs)[4],
                                   const int (&as)[2]) {
#pragma unroll
  for (int nj = 0; nj < 4; ++nj)
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) acc[nj][mi] = mfma32<KJ, KJ>(bf[nj], af[mi], acc[nj][mi], bs[nj], as[mi]);
}

// scheduling hint: one LDS read after every MFMA, n times
#define AVE_MFMA_DS_PAIRS(n)                                  \
  _Pragma("unroll") for (int q_ = 0; q_ < (n); ++q_) {        \
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);        \
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);        \
  }                                                           \
  __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);          \
  __builtin_amdgcn_sched_barrier(0);

// SC16: scales by pairs of stages, loads issued by waves 0-3, and the persistent form (a workgroup walks the
// tiles pid, pid + gridDim.x, ...); !SC16: scales per stage, every wave loads its share, one tile per workgroup.
// SWIGLU (with SC16 only): B holds the N gate rows followed by the N up rows; a tile is 256 rows of C by 128
// output columns.  The 128 B-image rows of a wave (wm, wn) are the gate rows (first 64) and the up rows (last 64)
// of output columns 64 wn .. 64 wn + 63, so accumulator blocks nj and nj + 2 of a lane hold the gate and the up
// value of the SAME outputs and silu(gate) * up is evaluated in registers, in fp32 on the fp32 accumulators.
// QUANT (with SWIGLU only): the result is rounded to bf16 and then quantised to MXFP4 (p.Q, p.Qs) exactly as the
// stand-alone quantiser would quantise the bf16 output, instead of being stored.
// SPLITK (with SC16 only, plain GEMM): a work item is a tile and a slice of K (p.slice_pairs pairs of stages, the
// last slice what is left); its fp32 sums go to p.P[slice][M][N] and splitk_reduce_kernel adds the slices up in
// slice order.  For shapes with far fewer tiles than compute units and a long K (M of a few hundred rows against
// weights with few rows), where one tile per workgroup leaves most of the chip idle for the whole of K.
// TAIL (with SC16 only, not with SPLITK): K is any multiple of 32 from 512 up.  The whole pairs of stages run as above
// with the true row pitch; the K % 512 elements behind them (1..15 blocks of 32) are copied into the free stage
// buffers through registers, padded with zero codes, and multiplied as one or two more stages.
// GROUPED: the m-tile list is the concatenation of the experts' tile lists (p.row_offsets, p.E).  A template argument
// rather than a test of the pointer, so that the plain GEMM carries none of the lookup.
// BLOCKED (plain pair-scale form only): p.As and p.Bs are in the 128 x 4 blocked layout.  A pair of stages is 16 scale
// columns = four column tiles, which lie back to back in memory: the 256 rows of an operand take 2 row tiles x 2 KB,
// copied as they are (four 1 KB pieces, whole cache lines, where the row-major form gathers 16-byte pieces of 256
// rows).  In LDS a pair is [row tile][column tile d][512 B]; the four scale bytes of fragment row r for stage parity P and
// lane half h are the dword at d = 2 P + h, byte (r % 32) * 16 + (r % 128 / 32) * 4 of that tile.
// TOUCH (ungrouped pair-scale forms, plain or with the fused epilogues): the look-ahead touches of the grouped form for a plain GEMM whose weights come from
// HBM -- a model's layers, each with weights of its own, as opposed to one GEMM replayed on operands that stay in the
// last-level cache.  Same bits; 5 % faster on weights from HBM, 1.6 % slower on cache-resident ones (measured on
// 8192 x 14336 x 4096), so the host chooses (launch_mx_tile).
// CH = 4 (ungrouped pair-scale forms without touches, K % 2048 == 0; 0: 16-byte pieces per pair of stages): the scale
// rows are fetched 64 bytes at a time -- four pairs of stages -- instead of 16.  A row's scales are K / 32 bytes, 128
// for K = 4096: with 16-byte pieces every pair of stages touches a cache line per row (512 lines for 8 KB), which costs
// the load path as much as a tenth of the stage data does; four lanes per row touch each line twice per 4096 elements
// of K instead of eight times (measured: touching half / an eighth as many lines, with wrong scales, is 2.3 / 3.3 %
// faster; this form as built: 1.7-1.9 %).  ONE chunk buffer of 32 KB, [256 rows][64 B] per operand, fills LDS to its
// 160 KB (so not for the forms that keep the experts' table or the touches' sink there): chunk c + 1 is requested
// behind the barrier of the second-to-last stage of chunk c, when every wave has taken chunk c's last pair into
// registers, and is read a stage later -- the lead the stage data has.  16-byte slot j of a row holds its piece
// j ^ ((row >> 2) & 3) (on the source side), so that the 16 rows of a ds_read_b128 fall into 16 bank groups.
template <bool SC16, bool SWIGLU = false, bool QUANT = false, bool SPLITK = false, bool TAIL = false, bool GROUPED = false,
          bool BLOCKED = false, bool TOUCH = false, int CH = 0>
__global__ __launch_bounds__(kWaves * 64) void mx_tile_kernel(MxArgs p, int m_tiles, int n_tiles) {
  constexpr bool SC64 = CH != 0;   // chunked scale rows
  static_assert(CH == 0 || CH == 4, "scale rows per pair of stages, or in chunks of four pairs");
  static_assert(CH != 4 || (!GROUPED && !TOUCH), "four-pair chunks leave no LDS for the experts' table and the touches' sink");
  static_assert(!SC64 || (SC16 && !SPLITK && !TAIL && !BLOCKED), "chunked scale rows: pair-scale forms on whole chunks");
  static_assert(!TOUCH || (SC16 && !SPLITK && !TAIL && !GROUPED && !BLOCKED), "touches: the grouped forms, and the ungrouped ones on whole pairs of stages");
  constexpr bool kTouches = GROUPED || TOUCH;
  static_assert(!BLOCKED || (SC16 && !SWIGLU && !SPLITK && !TAIL && !GROUPED), "blocked scales: the plain GEMM on whole pairs of stages");
  static_assert(!GROUPED || !SPLITK, "K is split for the plain GEMM only");
  static_assert(!TAIL || (SC16 && !SPLITK), "the K tail exists for the pair-scale forms, K not split");
  static_assert(SC16 || !SWIGLU, "the fused SwiGLU epilogue exists for the pair-scale form only");
  static_assert(SWIGLU || !QUANT, "the fused quantiser follows the fused SwiGLU");
  static_assert(!SPLITK || (SC16 && !SWIGLU), "K is split in whole pairs of stages, for the plain GEMM");
  constexpr bool PERSIST = SC16;
  constexpr int kTileN = SWIGLU ? BN / 2 : BN;   // output columns per tile
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int wm = w >> 1, wn = w & 1;   // wave (wm, wn) owns rows 64*wm.., columns 128*wn.. of the tile
  int tiles = m_tiles * n_tiles;   // GROUPED: m_tiles is the host's upper bound until the experts' table is built
  int total = SPLITK ? tiles * p.slices : tiles;
  const unsigned row_bytes = (unsigned)p.K / 2, row_scales = (unsigned)p.K / 32;

  // Tile of workgroup slot `pid`: rows [m_begin, m_end) of A/C (m_end: end of the matrix or of the expert),
  // columns from n_begin, weights of `expert`.  False for a slot behind the last tile of the grouped list.
  // SPLITK: slot pid is tile pid % tiles of slice pid / tiles; the slice covers item_stages stages from pair k_pair0.
  int m_begin, m_end, n_begin, expert;
  // GROUPED with the table in LDS: the experts that own m-tiles of the tile's group of kXcds bands (the tiles of one
  // group and one column of tiles run side by side), and the tile's position in the group; no experts behind the
  // last whole group
  unsigned long long share_experts[kTableExperts / 64] = {0, 0, 0, 0};   // bit e % 64 of word e / 64: expert e
  int share_i = 0;
  int slice = 0, k_pair0 = 0, item_stages = TAIL ? 2 * (p.K / (2 * BK)) : p.K / BK;
  auto locate = [&](int pid) {
    int tm, tn;
    if (SPLITK) {
      slice = pid / tiles;
      pid -= slice * tiles;
      k_pair0 = slice * p.slice_pairs;
      const int left = p.K / (2 * BK) - k_pair0;
      item_stages = 2 * (left < p.slice_pairs ? left : p.slice_pairs);
    }
    map_tile(pid, m_tiles, n_tiles, tm, tn);
    m_begin = tm * BM;
    m_end = p.M;
    expert = 0;
    n_begin = tn * kTileN;
    if (TOUCH) {
      // one "expert": the tiles of a whole group of kXcds bands in one column of tiles share that column's B panel
      constexpr int kGroupTiles = kXcds * kGroupM;
      const int g_first = tm / kGroupTiles * kGroupTiles;
      share_i = tm - g_first;
      share_experts[0] = g_first + kGroupTiles <= m_tiles ? 1ull : 0ull;
    }
    if (!GROUPED) return true;
    // tm indexes the concatenation of per-expert tile lists (table entries clamped to [0, M])
    if (SC16 && p.E <= kTableExperts) {
      // the table in LDS: entry e holds {first tile, tiles, first row, end row} of expert e (no tiles behind the last);
      // lane l looks at experts l, l + 64, l + 128, l + 192
      constexpr int kGroupTiles = kXcds * kGroupM;
      const int g_first = tm / kGroupTiles * kGroupTiles;
      const bool whole_group = g_first + kGroupTiles <= m_tiles;
      share_i = tm - g_first;
      bool found = false;
#pragma unroll
      for (int q = 0; q < kTableExperts / 64; ++q) {
        if (64 * q >= p.E) {   // (uniform) no experts in this set
          share_experts[q] = 0;
          continue;
        }
        const v4i ent = lds_read16((unsigned)(uintptr_t)lds + kGroupTable16 + (unsigned)(64 * q + (threadIdx.x & 63)) * 16);
        const unsigned long long hits = __ballot(tm >= ent[0] && tm < ent[0] + ent[1]);
        if (hits) {
          const int e = __builtin_ctzll(hits);
          expert = 64 * q + e;
          m_begin = __builtin_amdgcn_readlane(ent[2], e) + (tm - __builtin_amdgcn_readlane(ent[0], e)) * BM;
          m_end = __builtin_amdgcn_readlane(ent[3], e);
          found = true;
        }
        share_experts[q] = whole_group ? __ballot(ent[1] > 0 && ent[0] < g_first + kGroupTiles && ent[0] + ent[1] > g_first) : 0ull;
      }
      return found;
    }
    return locate_group_tile(p.row_offsets, p.E, p.M, BM, tm, expert, m_begin, m_end);
  };
  if (GROUPED && SC16 && p.E <= kTableExperts) {
    // Built once per workgroup, by its first wave, with the clamping of locate_group_tile: scanning the caller's table
    // in front of every tile costs 0.8 us per tile with eight experts.
    if (w == 0) {
      int carry = 0;   // tiles of the experts in the sets before
#pragma unroll
      for (int q = 0; q < kTableExperts / 64; ++q) {
        const int e = 64 * q + lane;
        int r0 = 0, r1 = 0;
        if (e < p.E) {
          r0 = p.row_offsets[e];
          r1 = p.row_offsets[e + 1];
          r0 = r0 < 0 ? 0 : (r0 > p.M ? p.M : r0);
          r1 = r1 < 0 ? 0 : (r1 > p.M ? p.M : r1);
        }
        const int nt = r1 > r0 ? (r1 - r0 + BM - 1) / BM : 0;
        int incl = nt;   // inclusive prefix sum over the lanes
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
          const int up = __shfl_up(incl, d);
          if (lane >= d) incl += up;
        }
        *reinterpret_cast<__attribute__((address_space(3))) v4i*>((uintptr_t)((unsigned)(uintptr_t)lds + kGroupTable16 +
                                                                              (unsigned)e * 16)) = v4i{carry + incl - nt, nt, r0, r1};
        carry += __builtin_amdgcn_readlane(incl, 63);
      }
    }
    __syncthreads();
    // The true length of the list replaces the host's bound (rows / 256 + experts): the slots behind the last tile
    // all sit in the last rounds of the walk and left some XCDs four times the tiles of others there.
    const v4i last = lds_read16((unsigned)(uintptr_t)lds + kGroupTable16 + (kTableExperts - 1) * 16);
    m_tiles = __builtin_amdgcn_readfirstlane(last[0] + last[1]);
    tiles = total = m_tiles * n_tiles;
  }
  // first tile of this workgroup (the persistent form walks pid, pid + gridDim.x, ...); the result is
  // uniform for the whole workgroup, so leaving here is safe with respect to the barriers below
  int pid = blockIdx.x;
  if (pid >= total) return;
  {
    bool have = locate(pid);
    while (PERSIST && !have && (pid += gridDim.x) < total) have = locate(pid);
    if (!have) return;
  }

  // ---- per-lane source offsets of the direct-to-LDS loads -----------------------------
  // data: wave w, instruction i covers tile rows (4w+i)*8 .. +7; lane -> (row, swizzled chunk)
  // scales, per stage: wave w covers tile rows 32w .. 32w+31 of both operands; lane -> (row, dword)
  // scales, per pair of stages: wave w covers rows 64w .. 64w+63 of A (w < 4) or 64(w-4) .. of B; lane -> row
  // Rows past the end of the matrix (or of the expert) are clamped to a valid row: their
  // products land in rows of C that are never stored.
  constexpr int kStage = SC16 ? kDataStage : kStageBytes;
  // SC16: waves 0-3 issue all loads of the workgroup (wave w: tile rows 64w .. 64w+63 of both operands and
  // their scale rows); with every wave issuing its share, the waves of a SIMD sit in load issue at the same
  // time and the matrix core idles meanwhile.
  constexpr int kDI = SC16 ? 8 : 4;   // data instructions per operand and issuing wave
  unsigned a_off[kDI], b_off[kDI], as_off, bs_off;
  const uint8_t *ga, *gb, *gas, *gbs;   // data: advance by one stage per issue; scales: by one stage or one pair
  // row of B behind row `row` (0..255) of the tile's B image, clamped to a valid row
  auto b_image_row = [&](int row, int n_begin) {   // n_begin: of the tile in question (a parameter on purpose)
    if (SWIGLU) {
      // image rows 128 wn + j: j < 64 the gate row, j >= 64 the up row of output column 64 wn + (j & 63)
      int n = n_begin + 64 * (row >> 7) + (row & 63);
      n = n < p.N ? n : p.N - 1;
      return (row & 64) ? p.N + n : n;
    }
    const int n = n_begin + row;
    return n < p.N ? n : p.N - 1;
  };
  auto setup_loads = [&](int lane) {
    const int lr = lane >> 3, cprime = lane & 7;
    const int wi = SC16 ? (w & 3) : w;
#pragma unroll
    for (int i = 0; i < kDI; ++i) {
      const int row = (wi * kDI + i) * 8 + lr;
      const int chunk = cprime ^ ((row >> 1) & 7);
      int am = m_begin + row;
      am = am < p.M ? am : p.M - 1;
      const int bn = b_image_row(row, n_begin);
      a_off[i] = (unsigned)am * row_bytes + chunk * 16;
      b_off[i] = (unsigned)bn * row_bytes + chunk * 16;
    }
    if (BLOCKED) {
      // issuing wave wi copies 1 KB per operand and pair: row tile wi / 2 of the tile's two, column tiles 2 (wi % 2) and
      // 2 (wi % 2) + 1 of the pair's four.  A row tile behind the tensor's last (the matrix ends inside the tile's
      // first 128 rows) is replaced by the last: its scales belong to rows that are never stored.
      const unsigned col_tiles = (unsigned)p.K / 128;
      int ta = m_begin / 128 + (wi >> 1), tb = n_begin / 128 + (wi >> 1);
      ta = ta < (p.M + 127) / 128 ? ta : (p.M + 127) / 128 - 1;
      tb = tb < (p.N + 127) / 128 ? tb : (p.N + 127) / 128 - 1;
      as_off = ((unsigned)ta * col_tiles + 2 * (wi & 1)) * 512 + (unsigned)lane * 16;
      bs_off = ((unsigned)tb * col_tiles + 2 * (wi & 1)) * 512 + (unsigned)lane * 16;
    } else if (SC16) {
      const int row = wi * 64 + lane;
      int am = m_begin + row;
      am = am < p.M ? am : p.M - 1;
      const int bn = b_image_row(row, n_begin);
      as_off = (unsigned)am * row_scales;
      bs_off = (unsigned)bn * row_scales;
    } else {
      const int row = w * 32 + (lane >> 1);
      int am = m_begin + row;
      am = am < p.M ? am : p.M - 1;
      int bn = n_begin + row;
      bn = bn < p.N ? bn : p.N - 1;
      as_off = (unsigned)am * row_scales + (lane & 1) * 4;
      bs_off = (unsigned)bn * row_scales + (lane & 1) * 4;
    }
    const size_t expert_rows = (size_t)expert * (SWIGLU ? 2 : 1) * p.N;   // an expert holds N, or N gate + N up rows
    const uint8_t* Bmat = p.B + expert_rows * row_bytes;
    const uint8_t* Bsc = p.Bs + expert_rows * row_scales;
    ga = p.A;
    gb = Bmat;
    gas = p.As;
    gbs = Bsc;
    if (SPLITK) {   // a pair of stages is 256 bytes of a data row and 16 scale bytes
      ga += (size_t)k_pair0 * (2 * kRowBytes);
      gb += (size_t)k_pair0 * (2 * kRowBytes);
      gas += (size_t)k_pair0 * 16;
      gbs += (size_t)k_pair0 * 16;
    }
  };
  setup_loads(lane);
  const unsigned lds_base = (unsigned)(uintptr_t)lds;

  auto issue_stage = [&](unsigned sb) {
    if constexpr (SC16) {
      dma16_stage(w >> 2, 0, sb + (w & 3) * 8192, ga, gb, a_off, b_off);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        dma16(ga, a_off[i], sb + kOffA + (w * 4 + i) * 1024);
        dma16(gb, b_off[i], sb + kOffB + (w * 4 + i) * 1024);
      }
      dma4(gas, as_off, sb + kOffAs + w * 256);
      dma4(gbs, bs_off, sb + kOffBs + w * 256);
      gas += BK / 32;
      gbs += BK / 32;
    }
    ga += kRowBytes;
    gb += kRowBytes;
  };
  // (tile_m, tile_n: of the tile the scales are for -- the tile being computed inside the main loop, the next one when
  // its first loads are requested; SC64 works the row offsets out when it issues, once per eight stages)
  auto issue_scale_pair = [&](int pair, int tile_m, int tile_n) {
    if constexpr (SC64) {
      // pair is a multiple of 4, or enable is 0; wave wi, instruction i: tile rows 64 wi + 16 i .. + 15, lane -> (row, slot)
      const unsigned enable = (pair & 3) == 0 ? 1u : 0u;
      // (the row offsets are worked out at every call: a branch around them that the compiler can see makes it spill
      // 170 registers in the main loop)
      const int wi = w & 3;
      const int piece = (lane & 3) ^ ((lane >> 4) & 3);
      unsigned ao[4], bo[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int row = wi * 64 + 16 * i + (lane >> 2);
        int am = tile_m + row;
        am = am < p.M ? am : p.M - 1;
        ao[i] = (unsigned)am * row_scales + (unsigned)piece * 16;
        bo[i] = (unsigned)b_image_row(row, tile_n) * row_scales + (unsigned)piece * 16;
      }
      dma16_scale_chunk((w >> 2) == 0 ? enable : 0u, lds_base + kScaleBase16 + (unsigned)wi * 4096, gas, gbs, ao, bo);
      if (enable) {
        gas += 64;
        gbs += 64;
      }
    } else {
      dma16_scale_rows(w >> 2, 0, lds_base + kScaleBase16 + (pair & 1) * kScalePair16 + (w & 3) * 1024, gas, gbs, as_off, bs_off);
      gas += BLOCKED ? 2048 : 16;   // blocked: the pair's four column tiles of 512 bytes
      gbs += BLOCKED ? 2048 : 16;
    }
  };

  // ---- per-lane fragment read addresses ------------------------------------------------
  const int rho = lane & 31, h = lane >> 5;
  const int a_row = wm * 64 + rho;             // + 32*mi
  const int b_row = wn * 128 + pi_row(rho);    // + 32*nj
  // chunk (4h + kj) ^ ((row >> 1) & 7): kj only flips bits 4-5 of the byte address
  const unsigned a_frag = kOffA + a_row * kRowBytes + (((4 * h) ^ ((a_row >> 1) & 7)) * 16);
  const unsigned b_frag = kOffB + b_row * kRowBytes + (((4 * h) ^ ((b_row >> 1) & 7)) * 16);
  const unsigned a_sc = kOffAs + a_row * 8 + 4 * h;   // + mi*256
  const unsigned b_sc = kOffBs + b_row * 8 + 4 * h;
  const unsigned a_sc16 = kScaleBase16 + a_row * 16;              // + mi*512
  const unsigned b_sc16 = kScaleBase16 + BM * 16 + b_row * 16;    // + nj*512
  // 64-byte chunks: row * 64, slot (pair & 3) ^ ((row >> 2) & 3); 32 rows further down is 2048 bytes on, same swizzle
  const unsigned a_sc64 = kScaleBase16 + a_row * 64 + (((a_row >> 2) & 3) << 4);               // ^ (pair & 3) << 4, + mi*2048
  const unsigned b_sc64 = kScaleBase16 + BM * 64 + b_row * 64 + (((b_row >> 2) & 3) << 4);     // + nj*2048
  // blocked: row tile, 16-byte row and dword of the fragment row, lane half h -> column tile h (+ 2 for the pair's
  // second stage); 32 rows further down is the next dword
  const unsigned a_blk = kScaleBase16 + (a_row >> 7) * 2048 + (a_row & 31) * 16 + ((a_row >> 5) & 3) * 4 + h * 512;   // + mi*4
  const unsigned b_blk = kScaleBase16 + BM * 16 + (b_row >> 7) * 2048 + (b_row & 31) * 16 + h * 512;                  // + nj*4

  v16f acc[4][2];
  v4i af0[2], bf0[4], af1[2], bf1[4];
  int as_cur[2], bs_cur[4], as_nxt[2], bs_nxt[4];
  v4i as_pair[2], bs_pair[4];   // SC16: the 16 scale bytes of each fragment row for a pair of stages

#define AVE_READ_FRAGS(dst_a, dst_b, sb, KJ)                                                                    \
  _Pragma("unroll") for (int i = 0; i < 2; ++i) dst_a[i] = lds_read16((sb) + (a_frag ^ ((KJ) * 16)) + i * 4096); \
  _Pragma("unroll") for (int i = 0; i < 4; ++i) dst_b[i] = lds_read16((sb) + (b_frag ^ ((KJ) * 16)) + i * 4096);
#define AVE_READ_SCALES(dst_a, dst_b, sb)                                               \
  _Pragma("unroll") for (int i = 0; i < 2; ++i) dst_a[i] = lds_read4((sb) + a_sc + i * 256); \
  _Pragma("unroll") for (int i = 0; i < 4; ++i) dst_b[i] = lds_read4((sb) + b_sc + i * 256);
  // (blocked: elements 0 and 1 of a row's vector hold its dwords for the pair's first and second stage)
#define AVE_READ_SCALE_PAIR(pair)                                                                                     \
  if (SC64) {                                                                                                         \
    const unsigned slot_ = (unsigned)((pair) & 3) << 4;                                                               \
    _Pragma("unroll") for (int i = 0; i < 2; ++i) as_pair[i] = lds_read16(lds_base + ((a_sc64 ^ slot_) + i * 2048));  \
    _Pragma("unroll") for (int i = 0; i < 4; ++i) bs_pair[i] = lds_read16(lds_base + ((b_sc64 ^ slot_) + i * 2048));  \
  } else if (BLOCKED) {                                                                                               \
    _Pragma("unroll") for (int i = 0; i < 2; ++i) {                                                                   \
      as_pair[i][0] = lds_read4(lds_base + ((pair) & 1) * kScalePair16 + a_blk + i * 4);                              \
      as_pair[i][1] = lds_read4(lds_base + ((pair) & 1) * kScalePair16 + a_blk + i * 4 + 1024);                       \
    }                                                                                                                 \
    _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                                                   \
      bs_pair[i][0] = lds_read4(lds_base + ((pair) & 1) * kScalePair16 + b_blk + i * 4);                              \
      bs_pair[i][1] = lds_read4(lds_base + ((pair) & 1) * kScalePair16 + b_blk + i * 4 + 1024);                       \
    }                                                                                                                 \
  } else {                                                                                                            \
    _Pragma("unroll") for (int i = 0; i < 2; ++i) as_pair[i] = lds_read16(lds_base + ((pair) & 1) * kScalePair16 + a_sc16 + i * 512); \
    _Pragma("unroll") for (int i = 0; i < 4; ++i) bs_pair[i] = lds_read16(lds_base + ((pair) & 1) * kScalePair16 + b_sc16 + i * 512); \
  }
  // stage parity P of the pair, lane half h -> dword 2P + h of the row's 16 bytes
#define AVE_PICK_SCALES(dst_a, dst_b, P)                                                                   \
  if (BLOCKED) {                                                                                           \
    _Pragma("unroll") for (int i = 0; i < 2; ++i) dst_a[i] = as_pair[i][(P)];                              \
    _Pragma("unroll") for (int i = 0; i < 4; ++i) dst_b[i] = bs_pair[i][(P)];                              \
  } else {                                                                                                 \
    _Pragma("unroll") for (int i = 0; i < 2; ++i) dst_a[i] = h ? as_pair[i][2 * (P) + 1] : as_pair[i][2 * (P)]; \
    _Pragma("unroll") for (int i = 0; i < 4; ++i) dst_b[i] = h ? bs_pair[i][2 * (P) + 1] : bs_pair[i][2 * (P)]; \
  }

  // One stage.  The barrier sits before the last quarter: by then this wave has read all of the
  // stage's fragments (so the buffer may be refilled) and its loads of the next stage have landed.
  // The loads of the stage after the next are issued right behind the barrier, ahead of the last
  // quarter's MFMAs: the waves of a SIMD do not share the matrix core evenly (the older one is
  // served first), and loads issued behind the MFMAs left the younger wave's data late.
  // PARITY (SC16 only) is the stage's position in its pair: stage 0 issues the next pair's scale
  // loads, stage 1 reads the next pair's scales.
#define AVE_STAGE(ISSUE_NEXT2, READ_NEXT, PARITY)                                       \
  {                                                                                     \
    const unsigned sb = lds_base + (s & 1) * kStage;                                    \
    const unsigned sbn = lds_base + ((s + 1) & 1) * kStage;                             \
    AVE_READ_FRAGS(af1, bf1, sb, 1)                                                     \
    mma_quarter<0>(acc, bf0, af0, bs_cur, as_cur);                                      \
    AVE_MFMA_DS_PAIRS(6)                                                                \
    AVE_READ_FRAGS(af0, bf0, sb, 2)                                                     \
    mma_quarter<1>(acc, bf1, af1, bs_cur, as_cur);                                      \
    AVE_MFMA_DS_PAIRS(6)                                                                \
    AVE_READ_FRAGS(af1, bf1, sb, 3)                                                     \
    mma_quarter<2>(acc, bf0, af0, bs_cur, as_cur);                                      \
    AVE_MFMA_DS_PAIRS(6)                                                                \
    /* pair-scale forms: waves 0-3 issue every stage load; per-stage-scale form: every wave loads its share */ \
    if (kTouches && SC16) wait_loads_if_issuer(w); else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory"); \
    __syncthreads();                                                                    \
    if (ISSUE_NEXT2) {                                                                  \
      issue_stage(sb);                                                                  \
      if (SC16 && (PARITY) == 0) issue_scale_pair((s >> 1) + 1, c_m_begin, c_n_begin);  \
      __builtin_amdgcn_sched_barrier(0);                                                \
    }                                                                                   \
    if (READ_NEXT) {                                                                    \
      if (!SC16) {                                                                      \
        AVE_READ_SCALES(as_nxt, bs_nxt, sbn)                                            \
      } else if ((PARITY) == 1) {                                                       \
        AVE_READ_SCALE_PAIR((s >> 1) + 1)                                               \
      }                                                                                 \
      AVE_READ_FRAGS(af0, bf0, sbn, 0)                                                  \
    }                                                                                   \
    mma_quarter<3>(acc, bf1, af1, bs_cur, as_cur);                                      \
    if (READ_NEXT) { AVE_MFMA_DS_PAIRS(6) }                                             \
    if (SC16) {                                                                         \
      if (READ_NEXT) { AVE_PICK_SCALES(as_cur, bs_cur, (PARITY) ^ 1) }                  \
    } else {                                                                            \
      _Pragma("unroll") for (int i = 0; i < 2; ++i) as_cur[i] = as_nxt[i];              \
      _Pragma("unroll") for (int i = 0; i < 4; ++i) bs_cur[i] = bs_nxt[i];              \
    }                                                                                   \
    __builtin_amdgcn_sched_barrier(0);                                                  \
  }

  // GROUPED: every expert's weights are used by the few m-tiles of that expert only, so unlike the plain GEMM's B they
  // are not in the last-level cache when a tile asks for them, and loads that come from HBM land later than the one
  // stage they are issued ahead (measured: the same launch with every tile on expert 0's weights is 9 % faster). Eight
  // stages before a tile's end, the waves that issue no stage loads touch B panels of the NEXT round of the walk, one
  // 4-byte direct-to-LDS load per 128-byte line into a sink nobody reads.  The 32 tiles of a group in one column of
  // tiles run side by side and use the panels of that column of every expert with m-tiles in the group; each of the 32
  // touches 8 rows of each of these panels (and their scale rows), whichever expert its own tile belongs to, so every
  // panel is whole in the last-level cache when the next round starts -- a panel touched in part is no use, a stage
  // waits for its slowest line -- and no workgroup has more to touch than another.  These waves wait for no loads
  // inside the main loop, so the touches cost them nothing but the issue.  Measured on 8 experts x ~4096 rows, N =
  // 14336, K = 4096, alternately with a build without the touches: 6-7 % faster for even, ragged and band-misaligned
  // row tables alike (4-5 % with the touches at the tile's start, 16 stages ahead); N = 4096, K = 14336: 1-2.5 %
  // faster at 6 to 12 stages ahead, 1 % SLOWER at 24 and 4-6 % slower at the tile's start (56 stages, 115 us ahead: by
  // then the lines have left the cache again and were fetched twice).  (Touching only the panel of the workgroup's own
  // next tile, a part per tile of the same expert, was 6 % faster when every expert's tiles fill whole bands and 2-6 %
  // SLOWER otherwise: a tile whose expert has few tiles in the group then runs on a panel touched in part, falls
  // behind the others for good, and the launch ends with the slowest workgroup.)
  // Before the first round of a group the same is done for the A rows: the eight tiles of one m-tile in that round
  // take 32 rows each (another 0.5-1 %).
  const bool touch_ok = kTouches && (((uintptr_t)p.B | (uintptr_t)p.Bs) & 3) == 0;
  // nrows rows from row r0 of the next tile's B image (of_a: of its A rows), `width` bytes from the row's start, rows
  // `pitch` bytes apart in g (whose first row starts `mis` bytes behind a 4-byte boundary)
  auto touch_rows = [&](const uint8_t* g, unsigned pitch, unsigned width, unsigned mis, int r0, int nrows, bool of_a) {
    const unsigned sink = lds_base + kTouchSink16 + (unsigned)(w & 3) * 256;
    const unsigned per_row = (width + 127) >> 7;
    const unsigned lines = (unsigned)nrows * per_row;
    for (unsigned first = 0; first < lines; first += 256) {
      const unsigned idx = first + (unsigned)(w & 3) * 64 + (unsigned)lane;
      const unsigned r = idx / per_row;
      unsigned off = (idx - r * per_row) * 128;
      off = off + 4 <= width ? off : 0;
      int row = m_begin + r0 + (int)r;
      row = row < p.M ? row : p.M - 1;
      if (!of_a) row = b_image_row(r0 + (int)r, n_begin);
      if (idx < lines) dma4(g, (mis + (unsigned)row * pitch + off) & ~3u, sink);
    }
  };
  auto touch_next_panels = [&](bool on) {   // n_begin, share_experts, share_i describe the next tile here
    if (!on) return;
    for (int q = 0; q < kTableExperts / 64; ++q)
    for (unsigned long long left = share_experts[q]; left; left &= left - 1) {
      const size_t rows = (size_t)(64 * q + __builtin_ctzll(left)) * (SWIGLU ? 2 : 1) * p.N;
      const size_t sc_first = rows * row_scales;
      touch_rows(p.B + rows * row_bytes, row_bytes, row_bytes, 0, 8 * share_i, 8, false);
      touch_rows(p.Bs + (sc_first & ~(size_t)3), row_scales, row_scales, (unsigned)(sc_first & 3), 8 * share_i, 8, false);
    }
    if ((share_experts[0] | share_experts[1] | share_experts[2] | share_experts[3]) && n_begin < 8 * kTileN &&
        (((uintptr_t)p.A | (uintptr_t)p.As) & 3) == 0) {
      const int part = n_begin / kTileN;
      touch_rows(p.A, row_bytes, row_bytes, 0, 32 * part, 32, true);
      touch_rows(p.As, row_scales, row_scales, 0, 32 * part, 32, true);
    }
  };
  if (PERSIST) {
    issue_stage(lds_base);
    issue_scale_pair(0, m_begin, n_begin);
  }
  for (;;) {   // one tile per trip; a single trip unless PERSIST
  const int c_m_begin = m_begin, c_m_end = m_end, c_n_begin = n_begin;   // the tile being computed
  const int c_expert = TAIL ? expert : 0;
  const int stages = (SPLITK || TAIL) ? item_stages : p.K / BK;
  const int c_slice = slice;
  // The next tile is looked up now, while few registers are live; its description stays in scalar registers.
  bool have_next = false;
  if (PERSIST)
    while (!have_next && (pid += gridDim.x) < total) have_next = locate(pid);
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = v16f{};
  int s = 0;
  if (SC16) {
    // stages is even.  Loads in flight: data of the next stage, and from the first stage of a pair on also
    // data of the stage after it and the scales of the next pair.  In the persistent form the first stage
    // and the first pair of scales were issued during the previous tile's epilogue.
    wait_all_loads();
    __syncthreads();
    issue_stage(lds_base + kStage);
    // stage in front of which the look-ahead touches go out: kTouchLead stages before the tile's end
    const int touch_at = stages > kTouchLead ? stages - kTouchLead : 0;
    const bool idle_wave = GROUPED && c_m_begin + wm * 64 >= c_m_end;
    if (idle_wave) {
      // Grouped list, last tile of an expert: this wave's 64 rows lie behind the expert's last row.  It keeps the
      // workgroup's barriers and its share of the loads, reads no fragments and multiplies nothing (its
      // accumulators stay zero and none of its rows is stored), which leaves the matrix core of its SIMD to the
      // wave it shares it with.
#define AVE_IDLE_STAGE(ISSUE_NEXT2, PARITY)                              \
  {                                                                      \
    wait_loads_if_issuer(w);                                             \
    __syncthreads();                                                     \
    if (ISSUE_NEXT2) {                                                   \
      issue_stage(lds_base + (s & 1) * kStage);                          \
      if ((PARITY) == 0) issue_scale_pair((s >> 1) + 1, c_m_begin, c_n_begin); \
    }                                                                    \
  }
      for (; s < stages - 2; ++s) {
        if (kTouches && s == touch_at) touch_next_panels(w >= 4 && have_next && touch_ok);
        AVE_IDLE_STAGE(true, 0)
        ++s;
        AVE_IDLE_STAGE(true, 1)
      }
      AVE_IDLE_STAGE(false, 0)
      ++s;
      AVE_IDLE_STAGE(false, 1)
#undef AVE_IDLE_STAGE
    } else {
      AVE_READ_SCALE_PAIR(0)
      AVE_READ_FRAGS(af0, bf0, lds_base, 0)
      AVE_PICK_SCALES(as_cur, bs_cur, 0)
      for (; s < stages - 2; ++s) {
        if (kTouches && s == touch_at) touch_next_panels(w >= 4 && have_next && touch_ok);
        AVE_STAGE(true, true, 0)
        ++s;
        AVE_STAGE(true, true, 1)
      }
      AVE_STAGE(false, true, 0)
      ++s;
      AVE_STAGE(false, false, 1)
    }
    if constexpr (TAIL) {
      // The K % 512 elements behind the last whole pair of stages: 1..15 blocks of 32.  Behind the last stage's
      // barrier nothing reads the stage and scale buffers any more, so the workgroup copies the tail into them
      // through registers -- chunks behind the end of the row as zeros, their scale bytes as 2^0 -- in the layout
      // of an ordinary pair of stages, and multiplies one or two more stages from there.
      const int tail_blocks = (p.K % (2 * BK)) / 32;
      const int tail_stages = tail_blocks > 8 ? 2 : 1;
      const unsigned k0_bytes = (unsigned)(p.K / (2 * BK)) * (2 * kRowBytes);   // bytes of a row in front of the tail
      const size_t tail_expert_rows = (size_t)c_expert * (SWIGLU ? 2 : 1) * p.N;   // an expert holds N, or N gate + N up rows
      const uint8_t* tB = p.B + tail_expert_rows * row_bytes;
      const uint8_t* tBs = p.Bs + tail_expert_rows * row_scales;
      for (int t = 0; t < tail_stages; ++t) {
        // 2 operands x 256 rows x 8 chunks of 16 bytes; 8 lanes per row.  Every load is issued (a chunk behind the
        // row's end re-reads the tail's first chunk and is replaced by zeros) so that the eight are in flight together.
        v4i v[8];
#pragma unroll
        for (int it = 0; it < 8; ++it) {
          const int q = it * 512 + tid;
          const int opnd = q >> 11, row = (q >> 3) & 255, cc = q & 7;
          int grow = c_m_begin + row;
          grow = grow < p.M ? grow : p.M - 1;
          if (opnd) grow = b_image_row(row, c_n_begin);
          const bool have = 8 * t + cc < tail_blocks;
          v[it] = *reinterpret_cast<const v4i*>((opnd ? tB : p.A) + (size_t)grow * row_bytes + k0_bytes +
                                                (have ? (unsigned)(8 * t + cc) * 16 : 0u));
          if (!have) v[it] = v4i{0, 0, 0, 0};
        }
#pragma unroll
        for (int it = 0; it < 8; ++it) {
          const int q = it * 512 + tid;
          const int opnd = q >> 11, row = (q >> 3) & 255, cc = q & 7;
          *reinterpret_cast<__attribute__((address_space(3))) v4i*>((uintptr_t)(
              lds_base + (unsigned)t * kStage + (opnd ? kOffB : kOffA) + (unsigned)row * kRowBytes +
              (unsigned)((cc ^ ((row >> 1) & 7)) * 16))) = v[it];
        }
      }
      {
        // scales: lane -> one row of one operand.  The 16 bytes that END at the row's end are fetched (K >= 512: they
        // lie inside the row) and moved down so that the tail's first block comes first; 0x7f fills the rest.
        const int opnd = tid >> 8, row = tid & 255;
        int grow = c_m_begin + row;
        grow = grow < p.M ? grow : p.M - 1;
        if (opnd) grow = b_image_row(row, c_n_begin);
        const uint8_t* src = (opnd ? tBs : p.As) + (size_t)grow * row_scales + row_scales - 16;
        v4i e;
        __builtin_memcpy(&e, src, 16);   // any byte alignment
        const int shift = 16 - tail_blocks;   // bytes to drop in front, 1..15
        const unsigned fill = 0x7f7f7f7fu;
        const unsigned x[8] = {(unsigned)e[0], (unsigned)e[1], (unsigned)e[2], (unsigned)e[3], fill, fill, fill, fill};
        v4i o;
        const unsigned r = (unsigned)shift & 3u;
        switch (shift >> 2) {
          case 0:
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = (int)__builtin_amdgcn_alignbyte(x[j + 1], x[j], r);
            break;
          case 1:
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = (int)__builtin_amdgcn_alignbyte(x[j + 2], x[j + 1], r);
            break;
          case 2:
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = (int)__builtin_amdgcn_alignbyte(x[j + 3], x[j + 2], r);
            break;
          default:
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = (int)__builtin_amdgcn_alignbyte(j + 4 < 8 ? x[j + 4] : fill, x[j + 3], r);
            break;
        }
        *reinterpret_cast<__attribute__((address_space(3))) v4i*>((uintptr_t)(
            lds_base + kScaleBase16 + (opnd ? BM * 16 : 0) + (unsigned)row * 16)) = o;
      }
      __syncthreads();
      if (!idle_wave) {
        AVE_READ_SCALE_PAIR(0)
        for (int t = 0; t < tail_stages; ++t) {
          const unsigned sb = lds_base + (unsigned)t * kStage;
          if (t == 0) {
            AVE_PICK_SCALES(as_cur, bs_cur, 0)
          } else {
            AVE_PICK_SCALES(as_cur, bs_cur, 1)
          }
          AVE_READ_FRAGS(af0, bf0, sb, 0)
          AVE_READ_FRAGS(af1, bf1, sb, 1)
          mma_quarter<0>(acc, bf0, af0, bs_cur, as_cur);
          AVE_READ_FRAGS(af0, bf0, sb, 2)
          mma_quarter<1>(acc, bf1, af1, bs_cur, as_cur);
          AVE_READ_FRAGS(af1, bf1, sb, 3)
          mma_quarter<2>(acc, bf0, af0, bs_cur, as_cur);
          mma_quarter<3>(acc, bf1, af1, bs_cur, as_cur);
        }
      }
    }
  } else {
    issue_stage(lds_base);
    wait_all_loads();
    __syncthreads();
    if (stages > 1) issue_stage(lds_base + kStage);
    AVE_READ_SCALES(as_cur, bs_cur, lds_base)
    AVE_READ_FRAGS(af0, bf0, lds_base, 0)
    for (; s < stages - 2; ++s) AVE_STAGE(true, true, 0)
    if (s < stages - 1) {
      AVE_STAGE(false, true, 0)
      ++s;
    }
    AVE_STAGE(false, false, 0)
  }
#undef AVE_STAGE
#undef AVE_READ_FRAGS
#undef AVE_READ_SCALES
#undef AVE_READ_SCALE_PAIR
#undef AVE_PICK_SCALES

  // ---- epilogue: fp32 -> bf16 (RNE) ----------------------------------------------------
  // Full-width tiles go through LDS (free after the last stage) so that every store instruction
  // writes whole rows of the tile: 512 contiguous bytes per row, four full 128-byte lines,
  // instead of 32-byte pieces per row straight from the accumulator layout.
  const bool row_store = (c_n_begin + BN <= p.N) && (p.N % 8 == 0) && ((reinterpret_cast<uintptr_t>(p.C) & 15) == 0);
  if (!PERSIST) {
    if (!row_store) {
      store_wave_block<2>(acc, p.C, p.N, c_m_begin + wm * 64, c_m_end, c_n_begin + wn * 128, lane, 1.0f);
      return;
    }
    constexpr int kCRow = BN * 2 + 16;   // bytes per staged row; the 16-byte pad spreads rows over the banks
    __syncthreads();                      // every wave is done reading the stage buffers
    {
      const int c = lane & 31, q = lane >> 5;
#pragma unroll
      for (int mi = 0; mi < 2; ++mi) {
        const unsigned row_addr = lds_base + (unsigned)(wm * 64 + 32 * mi + c) * kCRow + (unsigned)(wn * 128 + 8 * q) * 2;
#pragma unroll
        for (int nj = 0; nj < 4; ++nj) {
          const v16f& d = acc[nj][mi];
#pragma unroll
          for (int piece = 0; piece < 2; ++piece) {
            v4i o;
            o[0] = (int)pack_bf16x2(d[8 * piece + 0], d[8 * piece + 1]);
            o[1] = (int)pack_bf16x2(d[8 * piece + 2], d[8 * piece + 3]);
            o[2] = (int)pack_bf16x2(d[8 * piece + 4], d[8 * piece + 5]);
            o[3] = (int)pack_bf16x2(d[8 * piece + 6], d[8 * piece + 7]);
            *reinterpret_cast<__attribute__((address_space(3))) v4i*>((uintptr_t)(row_addr + (32 * nj + 16 * piece) * 2)) = o;
          }
        }
      }
    }
    __syncthreads();
    {
      // wave w stores tile rows 32w .. 32w+31, two rows per instruction
      const int half = lane >> 5, col16 = lane & 31;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int row = w * 32 + 2 * i + half;
        const int m = c_m_begin + row;
        const v4i o = lds_read16(lds_base + (unsigned)row * kCRow + (unsigned)col16 * 16);
        if (m < c_m_end) *reinterpret_cast<v4i*>(p.C + (size_t)m * p.N + c_n_begin + col16 * 8) = o;
      }
    }
    return;
  }

  // The accumulators are pinned here: the MFMAs are pure arithmetic to the compiler, which otherwise sinks
  // those of the last stages below the barrier and the loads that follow, far from their operands.
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) asm volatile("" : "+v"(acc[i][j]));
  // Persistent form: the next tile's first stage and first pair of scales are requested BEFORE this tile's
  // C leaves, into stage buffer 0 and scale buffer 0, so their latency (3 us when every workgroup of the
  // chip starts a tile at the same moment) runs under the stores.  C is staged through stage buffer 1 alone,
  // 128 rows at a time: [128 rows][512 B], 16-byte chunk c of row r at position c ^ (r & 15) (16 consecutive
  // rows of one column chunk then fall into 16 different bank groups).
  __syncthreads();   // every wave is done reading the stage and scale buffers
  // Everything below is addressed from an opaque copy of the lane number: the addresses of the epilogue do
  // not change from tile to tile, and hoisted out of the tile loop they would occupy registers that the
  // main loop has no room for.
  int elane = lane;
  asm volatile("" : "+v"(elane));
  auto request_next_tile = [&]() {
    if (have_next) {
      setup_loads(elane);
      issue_stage(lds_base);
      issue_scale_pair(0, m_begin, n_begin);
    }
  };
  if constexpr (SWIGLU) {
    // silu(gate) * up in registers, rounded to bf16 and staged through stage buffer 1 as one [256 rows][256 B] tile
    // (16-byte chunk ch of row r at position ch ^ (r & 15)), then written out as whole 256-byte rows -- or, with
    // QUANT, quantised on the way out: the four lanes that hold a 32-element block are neighbours, as in the
    // stand-alone quantiser.
    request_next_tile();
    const unsigned cbuf = lds_base + kStage;
    {
      const int c = elane & 31, q = elane >> 5;
#pragma unroll
      for (int mi = 0; mi < 2; ++mi) {
        const int r = wm * 64 + 32 * mi + c;
        const unsigned row_addr = cbuf + (unsigned)r * 256;
#pragma unroll
        for (int nj = 0; nj < 2; ++nj) {
          const v16f& g = acc[nj][mi];
          const v16f& u = acc[nj + 2][mi];
#pragma unroll
          for (int piece = 0; piece < 2; ++piece) {
            float h[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) h[e] = silu(g[8 * piece + e]) * u[8 * piece + e];
            v4i o;
            o[0] = (int)pack_bf16x2(h[0], h[1]);
            o[1] = (int)pack_bf16x2(h[2], h[3]);
            o[2] = (int)pack_bf16x2(h[4], h[5]);
            o[3] = (int)pack_bf16x2(h[6], h[7]);
            const unsigned chunk = (unsigned)(wn * 8 + 4 * nj + 2 * piece + q);
            *reinterpret_cast<__attribute__((address_space(3))) v4i*>((uintptr_t)(row_addr + ((chunk ^ (r & 15)) * 16))) = o;
          }
        }
      }
    }
    __syncthreads();
    {
      // wave w writes out rows 32w .. 32w+31, four rows per instruction: lane -> (row, 16-byte chunk = 8 outputs)
      const bool vec_ok = (p.N % 8 == 0) && ((reinterpret_cast<uintptr_t>(p.C) & 15) == 0);
      const int ch = elane & 15;
      v4i o[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int r = 32 * w + 4 * i + (elane >> 4);
        o[i] = lds_read16(cbuf + (unsigned)r * 256 + (unsigned)((ch ^ (r & 15)) * 16));
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int m = c_m_begin + 32 * w + 4 * i + (elane >> 4);
        const int n = c_n_begin + 8 * ch;
        if constexpr (QUANT) {
          // the stand-alone quantiser's steps on the bf16 values (N % 32 == 0: a block is inside the matrix or
          // outside it as a whole, so the exchange below is between lanes in the same state)
          float v[8];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            v[2 * j] = __builtin_bit_cast(float, (unsigned)o[i][j] << 16);
            v[2 * j + 1] = __builtin_bit_cast(float, (unsigned)o[i][j] & 0xFFFF0000u);
          }
          const unsigned amax = lane_xor_max_bits(lane_xor_max_bits(abs_max_bits(v), 1), 2);
          const int byte = mx_scale_byte(amax);
          const float scale = mx_scale_value(byte);
          unsigned codes = 0;
          codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(codes, v[0], v[1], scale, 0);
          codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(codes, v[2], v[3], scale, 1);
          codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(codes, v[4], v[5], scale, 2);
          codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(codes, v[6], v[7], scale, 3);
          if (m < c_m_end && n < p.N) {
            *reinterpret_cast<unsigned*>(p.Q + (size_t)m * (q_row_cols(p) / 2) + n / 2) = byte == 0xFF ? 0u : codes;
            if ((ch & 3) == 0) p.Qs[(size_t)m * (q_row_cols(p) / 32) + n / 32] = (uint8_t)byte;
          }
        } else if (m < c_m_end) {
          uint16_t* crow = p.C + (size_t)m * p.N;
          if (vec_ok && n + 8 <= p.N) {
            *reinterpret_cast<v4i*>(crow + n) = o[i];
          } else {
#pragma unroll
            for (int e = 0; e < 8; ++e)
              if (n + e < p.N) crow[n + e] = (uint16_t)(((unsigned)o[i][e >> 1] >> (16 * (e & 1))) & 0xFFFF);
          }
        }
      }
    }
  } else if constexpr (SPLITK) {
    request_next_tile();
    store_wave_block_f32<2>(acc, p.P + (size_t)c_slice * (size_t)p.M * (size_t)p.N, p.N, c_m_begin + wm * 64, c_m_end,
                            c_n_begin + wn * 128, elane);
  } else if (!row_store) {
    request_next_tile();
    store_wave_block<2>(acc, p.C, p.N, c_m_begin + wm * 64, c_m_end, c_n_begin + wn * 128, elane, 1.0f);
  } else {
    const unsigned cbuf = lds_base + kStage;
    auto stage_rows = [&]() {   // this wave's 64 rows of C into their half of the staging buffer
      const int c = elane & 31, q = elane >> 5;
#pragma unroll
      for (int mi = 0; mi < 2; ++mi) {
        const int r = (wm & 1) * 64 + 32 * mi + c;
        const unsigned row_addr = cbuf + (unsigned)r * 512;
#pragma unroll
        for (int nj = 0; nj < 4; ++nj) {
          const v16f& d = acc[nj][mi];
#pragma unroll
          for (int piece = 0; piece < 2; ++piece) {
            v4i o;
            o[0] = (int)pack_bf16x2(d[8 * piece + 0], d[8 * piece + 1]);
            o[1] = (int)pack_bf16x2(d[8 * piece + 2], d[8 * piece + 3]);
            o[2] = (int)pack_bf16x2(d[8 * piece + 4], d[8 * piece + 5]);
            o[3] = (int)pack_bf16x2(d[8 * piece + 6], d[8 * piece + 7]);
            const unsigned chunk = (unsigned)(wn * 16 + 4 * nj + 2 * piece + q);
            *reinterpret_cast<__attribute__((address_space(3))) v4i*>((uintptr_t)(row_addr + ((chunk ^ (r & 15)) * 16))) = o;
          }
        }
      }
    };
    auto store_rows = [&](int hh, int first) {   // rows first .. first + 15 of half hh, two per instruction
      const int half = elane >> 5, col16 = elane & 31;
      v4i o[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int r = first + 2 * i + half;
        o[i] = lds_read16(cbuf + (unsigned)r * 512 + (unsigned)((col16 ^ (r & 15)) * 16));
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int m = c_m_begin + hh * 128 + first + 2 * i + half;
        if (m < c_m_end) *reinterpret_cast<v4i*>(p.C + (size_t)m * p.N + c_n_begin + col16 * 8) = o[i];
      }
    };
    request_next_tile();
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      if (hh == 1) __syncthreads();   // the first half has been read
      if ((wm >> 1) == hh) stage_rows();
      __syncthreads();
      store_rows(hh, w * 16);   // wave w stores rows 16w .. 16w+15 of this half
    }
  }
  if (!have_next) return;
  }   // next tile
}

// C = bf16(P[0] + P[1] + ... + P[slices-1]), added in that order in fp32; P[s] is [mn] floats.
// A lane owns 8 consecutive elements (VEC: two 16-byte loads per slice, one 16-byte store) or one.
template <bool VEC>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ P, uint16_t* __restrict__ C,
                                                            size_t mn, int slices) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  if constexpr (VEC) {
    const size_t groups = mn / 8;   // mn % 8 == 0
    for (size_t g = (size_t)blockIdx.x * blockDim.x + threadIdx.x; g < groups; g += stride) {
      const v4f* src = reinterpret_cast<const v4f*>(P) + 2 * g;
      const size_t step = mn / 4;
      v4f lo = src[0], hi = src[1];
      int sl = 1;
      for (; sl + 4 <= slices; sl += 4) {   // four slices' loads in flight, added in slice order
        v4f l[4], h[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          l[u] = src[(size_t)(sl + u) * step];
          h[u] = src[(size_t)(sl + u) * step + 1];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          lo += l[u];
          hi += h[u];
        }
      }
      for (; sl < slices; ++sl) {
        lo += src[(size_t)sl * step];
        hi += src[(size_t)sl * step + 1];
      }
      v4i o;
      o[0] = (int)pack_bf16x2(lo[0], lo[1]);
      o[1] = (int)pack_bf16x2(lo[2], lo[3]);
      o[2] = (int)pack_bf16x2(hi[0], hi[1]);
      o[3] = (int)pack_bf16x2(hi[2], hi[3]);
      reinterpret_cast<v4i*>(C)[g] = o;
    }
  } else {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < mn; i += stride) {
      float sum = P[i];
      for (int sl = 1; sl < slices; ++sl) sum += P[(size_t)sl * mn + i];
      C[i] = to_bf16(sum);
    }
  }
}

}  // namespace

// K of any multiple of 32 from 512 up: whole pairs of stages plus a tail copied in behind them.  The scale rows are
// fetched in 16-byte pieces from rows whose pitch is K / 32 bytes.  The plain GEMM keeps its per-stage-scale form for
// K = 256 * odd; the fused forms have no such form and take the tail for every K that is no multiple of 512.
static bool tail_form(const MxArgs& p) {
  return p.K % (p.swiglu ? 2 * BK : BK) != 0 && p.K % 32 == 0 && p.K >= 2 * BK && (reinterpret_cast<uintptr_t>(p.A) & 15) == 0 &&
         (reinterpret_cast<uintptr_t>(p.B) & 15) == 0;
}

bool mx_tile_swiglu_supports(const MxArgs& p) {
  if (!p.swiglu) return false;
  if (p.Q && (!p.Qs || p.N % 32 != 0 || (reinterpret_cast<uintptr_t>(p.Q) & 3))) return false;
  if (p.M <= 0 || p.N <= 0) return false;
  if ((uint64_t)p.M * (uint64_t)(p.K / 2) >= (1ull << 32)) return false;
  if (2 * (uint64_t)p.N * (uint64_t)(p.K / 2) >= (1ull << 32)) return false;   // gate and up rows
  if (tail_form(p)) return true;
  if (p.K % (2 * BK) != 0) return false;
  // 16-byte pieces of the scale rows
  if ((reinterpret_cast<uintptr_t>(p.As) & 15) || (reinterpret_cast<uintptr_t>(p.Bs) & 15)) return false;
  return true;
}

bool mx_tile_supports(const MxArgs& p) {
  if (p.swiglu) return mx_tile_swiglu_supports(p);
  if ((p.K % BK != 0 && !tail_form(p)) || p.M <= 0 || p.N <= 0) return false;
  // 32-bit byte offsets inside A and inside one expert's B
  if ((uint64_t)p.M * (uint64_t)(p.K / 2) >= (1ull << 32)) return false;
  if ((uint64_t)p.N * (uint64_t)(p.K / 2) >= (1ull << 32)) return false;
  // scale rows are fetched as aligned dwords
  if ((reinterpret_cast<uintptr_t>(p.As) & 3) || (reinterpret_cast<uintptr_t>(p.Bs) & 3)) return false;
  return true;
}

namespace {
// compute units of the current device, a multiple of 8 (one share per XCD); 0 if the query fails
int persistent_workgroups() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    if (n >= 8) n -= n % 8;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}
}  // namespace

SplitPlan mx_tile_split_plan(int M, int N, int K, size_t max_workspace_bytes) {
  return mx_tile_split_plan_for(M, N, K, persistent_workgroups(), max_workspace_bytes);
}

SplitPlan mx_tile_split_plan_for(int M, int N, int K, int cus, size_t max_workspace_bytes) {
  SplitPlan plan;
  // The weight-streaming kernel owns M <= 64 -- except 33..64 rows over a long K (from 12288 elements): its four blocks
  // of activation rows per K panel then cost more than the split does (N = 4096, K = 14336: 17.0 us at 33..64 rows
  // against 14.4 us at 65 with the split; at K = 8192 the rings win, 10.9 against 12.5-14.5 us).  K is split in whole
  // pairs of stages.
  if (M <= 32 || (M <= 64 && K < 12288) || N <= 0 || K <= 0 || K % (2 * BK) != 0) return plan;
  if ((uint64_t)M * (uint64_t)(K / 2) >= (1ull << 32) || (uint64_t)N * (uint64_t)(K / 2) >= (1ull << 32)) return plan;
  const long tiles = (long)((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  if (cus <= 0 || tiles * 2 > cus) return plan;
  // Estimated time in microseconds, from measurements on MI355X with the weights streamed from HBM: 1.65 per stage
  // when a workgroup streams a weight panel of its own, 5 of prologue and epilogue; a split adds the second launch
  // and the slices' first-stage latency (9 in all), and its partial sums cross the memory system twice at 5.9 TB/s.
  const int pairs = K / (2 * BK);
  const long narrow_tiles = (long)((M + BM - 1) / BM) * ((N + 127) / 128);   // 256 x 128 tiles
  const long half_tiles = (long)((M + 127) / 128) * ((N + 127) / 128);       // 128 x 128 tiles
  // per stage: 1.65 on 256 x 256 tiles, 0.85 on 256 x 128 tiles (three stage buffers), 0.72 on 128 x 128 tiles
  // (four, and waves of their own for the loads); the unsplit call takes the best tiling that fits the compute units
  const double unsplit = (half_tiles <= cus ? 0.72 : (narrow_tiles <= cus ? 0.85 : 1.65)) * 2 * pairs + 5.0;
  double best = unsplit * 0.85;   // a split must save 15 %
  // the slices run on 256 x 256 tiles, or on the 256 x 128 or 128 x 128 tiles of the narrow-tile kernel
  for (int tiling = 0; tiling < 3; ++tiling) {
    const long t_tiles = tiling == 0 ? tiles : (tiling == 1 ? narrow_tiles : half_tiles);
    if (tiling > 0 && t_tiles > cus) continue;
    const double stage_us = tiling == 0 ? 1.65 : (tiling == 1 ? 0.85 : 0.72);
    const int max_slices = (int)(cus / t_tiles);
    for (int per = 1; per < pairs; ++per) {
      const int slices = (pairs + per - 1) / per;
      if (slices > max_slices) continue;
      if ((size_t)slices * (size_t)M * (size_t)N * sizeof(float) > max_workspace_bytes) continue;
      const double bytes = 2.0 * slices * (double)M * (double)N * 4.0;
      const double t = stage_us * 2 * per + 9.0 + bytes / 5.9e6;
      if (t < best) {
        best = t;
        plan.slices = slices;
        plan.slice_pairs = per;
        plan.narrow = tiling > 0;
        plan.half = tiling == 2;
      }
    }
  }
  if (plan.slices > 1) plan.workspace_bytes = (size_t)plan.slices * (size_t)M * (size_t)N * sizeof(float);
  else plan = SplitPlan{};
  return plan;
}

hipError_t launch_splitk_reduce(const float* P, uint16_t* C, size_t mn, int slices, hipStream_t s) {
  const bool vec = mn % 8 == 0 && (reinterpret_cast<uintptr_t>(C) & 15) == 0 && (reinterpret_cast<uintptr_t>(P) & 15) == 0;
  const size_t lanes = vec ? mn / 8 : mn;
  size_t grid = (lanes + 255) / 256;
  if (grid > 256 * 16) grid = 256 * 16;
  if (vec) hipLaunchKernelGGL(splitk_reduce_kernel<true>, dim3((unsigned)grid), dim3(256), 0, s, P, C, mn, slices);
  else hipLaunchKernelGGL(splitk_reduce_kernel<false>, dim3((unsigned)grid), dim3(256), 0, s, P, C, mn, slices);
  return hipGetLastError();
}

hipError_t launch_mx_tile_splitk(const MxArgs& p, hipStream_t s) {
  const int m_tiles = (p.M + BM - 1) / BM, n_tiles = (p.N + BN - 1) / BN;
  const int total = m_tiles * n_tiles * p.slices, cus = persistent_workgroups();
  if (cus <= 0) return hipErrorInvalidDevice;
  if (hipError_t e = allow_dynamic_lds<mx_tile_kernel<true, false, false, true>>(kLdsBytes16); e != hipSuccess) return e;
  hipLaunchKernelGGL((mx_tile_kernel<true, false, false, true>), dim3((unsigned)(total < cus ? total : cus)),
                     dim3(kWaves * 64), kLdsBytes16, s, p, m_tiles, n_tiles);
  if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
  return launch_splitk_reduce(p.P, p.C, (size_t)p.M * (size_t)p.N, p.slices, s);
}

int compute_units() { return persistent_workgroups(); }

namespace {
// one form of the kernel, plain or grouped
template <bool SC16, bool SWIGLU, bool QUANT, bool TAIL>
hipError_t launch_form(const MxArgs& p, unsigned grid, int lds_bytes, hipStream_t s, int m_tiles, int n_tiles) {
  const dim3 block(kWaves * 64);
  if (p.row_offsets) {
    if (hipError_t e = allow_dynamic_lds<mx_tile_kernel<SC16, SWIGLU, QUANT, false, TAIL, true>>(lds_bytes); e != hipSuccess) return e;
    hipLaunchKernelGGL((mx_tile_kernel<SC16, SWIGLU, QUANT, false, TAIL, true>), dim3(grid), block, lds_bytes, s, p, m_tiles, n_tiles);
  } else {
    if (hipError_t e = allow_dynamic_lds<mx_tile_kernel<SC16, SWIGLU, QUANT, false, TAIL, false>>(lds_bytes); e != hipSuccess) return e;
    hipLaunchKernelGGL((mx_tile_kernel<SC16, SWIGLU, QUANT, false, TAIL, false>), dim3(grid), block, lds_bytes, s, p, m_tiles, n_tiles);
  }
  return hipGetLastError();
}
}  // namespace

// Blocked scale tensors: the plain GEMM on whole pairs of stages, 16-byte aligned scale tensors, 32-bit offsets.
bool mx_tile_blocked_supports(const MxArgs& p) {
  if (!p.blocked_scales || p.swiglu || p.row_offsets || p.Q || p.M <= 0 || p.N <= 0 || p.K <= 0 || p.K % (2 * BK) != 0) return false;
  if ((uint64_t)((p.M + 127) / 128 * 128) * (uint64_t)(p.K / 2) >= (1ull << 32)) return false;
  if ((uint64_t)((p.N + 127) / 128 * 128) * (uint64_t)(p.K / 2) >= (1ull << 32)) return false;
  return (reinterpret_cast<uintptr_t>(p.As) & 15) == 0 && (reinterpret_cast<uintptr_t>(p.Bs) & 15) == 0;
}

namespace {
// one pair-scale form on whole pairs of stages: SWIGLU / QUANT epilogue, grouped or not, with or without touches, scale
// rows in chunks of CH pairs (0: per pair)
template <bool SWIGLU, bool QUANT, bool GROUPED, bool TOUCH, int CH>
hipError_t launch_pair_form(const MxArgs& p, unsigned grid, hipStream_t s, int m_tiles, int n_tiles) {
  constexpr int lds_bytes = CH == 4 ? kLdsBytes64 : kLdsBytes16;
  if (hipError_t e = allow_dynamic_lds<mx_tile_kernel<true, SWIGLU, QUANT, false, false, GROUPED, false, TOUCH, CH>>(lds_bytes); e != hipSuccess) return e;
  hipLaunchKernelGGL((mx_tile_kernel<true, SWIGLU, QUANT, false, false, GROUPED, false, TOUCH, CH>), dim3(grid), dim3(kWaves * 64), lds_bytes, s,
                     p, m_tiles, n_tiles);
  return hipGetLastError();
}
// ... picked by what the launch needs: the grouped forms and the forms with touches keep the experts' table and the
// touches' sink in LDS and fetch their scale rows per pair of stages (chunks of two pairs in the place of the two pair
// buffers measured no faster there: 970-976 against 971-973 us on the 8-expert benchmark); the others take chunks of four
// pairs when K is a multiple of 2048
template <bool SWIGLU, bool QUANT>
hipError_t launch_pairs(const MxArgs& p, unsigned grid, hipStream_t s, int m_tiles, int n_tiles, bool touch) {
  if (p.row_offsets) return launch_pair_form<SWIGLU, QUANT, true, false, 0>(p, grid, s, m_tiles, n_tiles);
  if (touch) return launch_pair_form<SWIGLU, QUANT, false, true, 0>(p, grid, s, m_tiles, n_tiles);
  if (p.K % (8 * BK) == 0 && !AVE_NO_SC64) return launch_pair_form<SWIGLU, QUANT, false, false, 4>(p, grid, s, m_tiles, n_tiles);
  return launch_pair_form<SWIGLU, QUANT, false, false, 0>(p, grid, s, m_tiles, n_tiles);
}
}  // namespace

hipError_t launch_mx_tile(const MxArgs& p, hipStream_t s) {
  if (p.blocked_scales) {
    const int m_tiles = (p.M + BM - 1) / BM, n_tiles = (p.N + BN - 1) / BN;
    const int total = m_tiles * n_tiles, cus = persistent_workgroups();
    if (cus <= 0) return hipErrorInvalidDevice;
    if (hipError_t e = allow_dynamic_lds<mx_tile_kernel<true, false, false, false, false, false, true>>(kLdsBytes16); e != hipSuccess) return e;
    hipLaunchKernelGGL((mx_tile_kernel<true, false, false, false, false, false, true>), dim3((unsigned)(total < cus ? total : cus)),
                       dim3(kWaves * 64), kLdsBytes16, s, p, m_tiles, n_tiles);
    return hipGetLastError();
  }
  const int m_tiles = (p.M + BM - 1) / BM + (p.row_offsets ? p.E : 0);
  const int n_tiles = p.swiglu ? (p.N + BN / 2 - 1) / (BN / 2) : (p.N + BN - 1) / BN;
  const int total = m_tiles * n_tiles;
  // scales by pairs of stages: whole pairs, and 16-byte pieces of the scale rows must be aligned
  const bool pairs = p.K % (2 * BK) == 0 && (reinterpret_cast<uintptr_t>(p.As) & 15) == 0 &&
                     (reinterpret_cast<uintptr_t>(p.Bs) & 15) == 0;
  if (!p.swiglu && !tail_form(p) && !pairs) return launch_form<false, false, false, false>(p, (unsigned)total, kLdsBytes, s, m_tiles, n_tiles);
  // the persistent forms: one workgroup per compute unit walks the tiles (a single tile each when there are no more
  // tiles than units)
  const int cus = persistent_workgroups();
  if (cus <= 0) return hipErrorInvalidDevice;
  const unsigned grid = (unsigned)(total < cus ? total : cus);
  const bool touch = p.touch && !p.row_offsets && total > cus;   // more than one round of tiles: there is a next round to touch for
  if (p.swiglu) {
    if (tail_form(p)) {
      if (p.Q) return launch_form<true, true, true, true>(p, grid, kLdsBytes16, s, m_tiles, n_tiles);
      return launch_form<true, true, false, true>(p, grid, kLdsBytes16, s, m_tiles, n_tiles);
    }
    if (p.Q) return launch_pairs<true, true>(p, grid, s, m_tiles, n_tiles, touch);
    return launch_pairs<true, false>(p, grid, s, m_tiles, n_tiles, touch);
  }
  if (tail_form(p)) return launch_form<true, false, false, true>(p, grid, kLdsBytes16, s, m_tiles, n_tiles);
  return launch_pairs<false, false>(p, grid, s, m_tiles, n_tiles, touch);
}

}  // namespace ave
