// MXFP4 GEMM for decode-time shapes (few activation rows) on gfx950: the weights B are streamed
// from HBM exactly once; only the activation panel is re-read.  The kernels are bound by HBM
// bandwidth, so the design is about keeping enough weight bytes of a workgroup in flight.
//
// Two kernels share the arithmetic (v_mfma_scale_f32_16x16x128_f8f6f4 with srcA = weight rows,
// srcB = activation rows, so a lane ends with 4 consecutive n of one row m; K split over the waves
// of a workgroup, partial tiles summed through LDS, bf16 RNE store):
//
//   * mx_decode_ring_kernel (further down): weights staged through an LDS ring with
//     global_load_lds; M <= 64, K % 512 == 0.  The one that matters for throughput.  It also has an
//     NVFP4 form (M <= 32): the same rings and items, fragments converted to f16 in registers.
//   * mx_decode_kernel (first): weights loaded straight into MFMA operand registers; M <= 16,
//     K % 128 == 0.  A workgroup owns T consecutive 16-column tiles of C and splits K over its
//     WAVES wavefronts: wave w handles K steps (128 elements each) SPW*w .. SPW*w+SPW-1 of every
//     chunk of WAVES*SPW steps; per step a lane issues one 16-byte load per tile (row l%16 of the
//     tile, 32 consecutive k = one E8M0 block) and all loads of a chunk are issued before the
//     first MFMA.
//
// Scale bytes: a lane needs byte (4*step + l/16) of its row.  Each lane loads the row's 4
// bytes of a step as one dword and rotates it by l/16 bytes, so the byte select of the
// instruction is the same for all lanes.
#include "fp4_common.hpp"
#include "kernels.hpp"

namespace ave {
namespace {

constexpr int kMaxT = 7;

template <int WAVES, int T, int SPW>
__global__ __launch_bounds__(WAVES * 64) void mx_decode_kernel(MxArgs p, int n_tiles16) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int r = lane & 15, g = lane >> 4;
  const int tile0 = blockIdx.x * T;
  const unsigned row_bytes = (unsigned)p.K / 2, row_scales = (unsigned)p.K / 32;
  const int blocks = p.K / 32, steps = (blocks + 3) / 4;   // a step is 128 elements: one block of 32 per lane group g

  // Buffer resources give 32-bit offsets and make rows past M / N read as zeros
  // (zero codes contribute nothing whatever the scale byte is).  Only the per-lane offset is compared with the
  // buffer size, not the scalar offset operand: a tile's row displacement therefore sits in the per-lane offset and
  // the scalar operand carries the position inside the row alone.
  const __amdgpu_buffer_rsrc_t ra = make_rsrc(p.A, (unsigned)p.M * row_bytes);
  const __amdgpu_buffer_rsrc_t ras = make_rsrc(p.As, (unsigned)p.M * row_scales);
  const __amdgpu_buffer_rsrc_t rb = make_rsrc(p.B, (unsigned)p.N * row_bytes);
  const __amdgpu_buffer_rsrc_t rbs = make_rsrc(p.Bs, (unsigned)p.N * row_scales);
  const unsigned a_off = (unsigned)r * row_bytes + 16 * g;
  const unsigned as_off = (unsigned)r * row_scales;
  const unsigned b_off = (unsigned)(tile0 * 16 + r) * row_bytes + 16 * g;   // + t*16*row_bytes
  const unsigned bs_off = (unsigned)(tile0 * 16 + r) * row_scales;          // + t*16*row_scales

  v4f acc[T];
#pragma unroll
  for (int t = 0; t < T; ++t) acc[t] = v4f{0, 0, 0, 0};

  for (int c0 = 0; c0 < steps; c0 += WAVES * SPW) {
    const int s0 = c0 + w * SPW;
    v4i af[SPW], bf[T][SPW];
    int asc[SPW], bsc[T][SPW];
#pragma unroll
    for (int j = 0; j < SPW; ++j) {
      const int s = s0 + j;
      if (s < steps) {
        // K % 128 != 0: the last step holds fewer than four blocks.  A dword of scales would then reach into the
        // next row -- behind the buffer's end for the last row, where the whole dword reads as zero -- so each lane
        // group fetches the one byte of its own block.
        const bool partial = s == steps - 1 && (blocks & 3) != 0;
        // a lane group behind the row's last block fetches the step's first block instead (its product is replaced
        // by zeros below): every address stays inside the row, also in the last row of the buffer, where the range
        // check -- which sees the per-lane offset only -- would let a few bytes behind the end through
        const int gl = 4 * s + g < blocks ? g : 0;
        const unsigned back = 16u * (unsigned)(g - gl);
#pragma unroll
        for (int t = 0; t < T; ++t) {
          bf[t][j] = __builtin_amdgcn_raw_buffer_load_b128(rb, b_off + t * 16 * row_bytes - back, s * 64, 0);
          bsc[t][j] = partial ? (int)__builtin_amdgcn_raw_buffer_load_b8(rbs, bs_off + t * 16 * row_scales + gl, s * 4, 0)
                              : __builtin_amdgcn_raw_buffer_load_b32(rbs, bs_off + t * 16 * row_scales, s * 4, 0);
        }
        af[j] = __builtin_amdgcn_raw_buffer_load_b128(ra, a_off - back, s * 64, 0);
        asc[j] = partial ? (int)__builtin_amdgcn_raw_buffer_load_b8(ras, as_off + gl, s * 4, 0)
                         : __builtin_amdgcn_raw_buffer_load_b32(ras, as_off, s * 4, 0);
      }
    }
#pragma unroll
    for (int j = 0; j < SPW; ++j) {
      const int s = s0 + j;
      if (s < steps) {
        // K % 128 != 0: in the last step the lane groups behind the row's last block multiply zeros under the scale
        // 2^0 (what they loaded belongs to the next row)
        const bool have = 4 * s + g < blocks;
        const bool partial = s == steps - 1 && (blocks & 3) != 0;   // the scale is then a single byte
        const int sa = have ? (partial ? asc[j] : rotr_bytes(asc[j], g)) : 0x7f;
        const v4i a = have ? af[j] : v4i{0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < T; ++t)
          acc[t] = mfma16<0, 0>(have ? bf[t][j] : v4i{0, 0, 0, 0}, a, acc[t],
                                have ? (partial ? bsc[t][j] : rotr_bytes(bsc[t][j], g)) : 0x7f, sa);
      }
    }
  }

  // ---- sum the WAVES partial tiles through LDS ------------------------------------------
  v4f* part = reinterpret_cast<v4f*>(lds);  // [WAVES][T][64]
#pragma unroll
  for (int t = 0; t < T; ++t) part[(w * T + t) * 64 + lane] = acc[t];
  __syncthreads();
  for (int u = tid; u < T * 64; u += WAVES * 64) {
    v4f s = part[u];
#pragma unroll
    for (int ww = 1; ww < WAVES; ++ww) s += part[ww * T * 64 + u];
    const int t = u >> 6, l = u & 63;
    const int m = l & 15, n = (tile0 + t) * 16 + 4 * (l >> 4);
    if (m < p.M && n < p.N) {
      uint16_t* dst = p.C + (size_t)m * p.N + n;
      if (n + 4 <= p.N && (p.N % 4 == 0) && ((reinterpret_cast<uintptr_t>(p.C) & 7) == 0)) {
        v2i o = {(int)pack_bf16x2(s[0], s[1]), (int)pack_bf16x2(s[2], s[3])};
        *reinterpret_cast<v2i*>(dst) = o;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n + e < p.N) dst[e] = to_bf16(s[e]);
      }
    }
  }
}

template <int WAVES, int T, int SPW>
hipError_t launch_t(const MxArgs& p, hipStream_t s, int n_tiles16) {
  constexpr int lds_bytes = WAVES * T * 64 * 16;
  if (hipError_t e = allow_dynamic_lds<mx_decode_kernel<WAVES, T, SPW>>(lds_bytes); e != hipSuccess) return e;
  const unsigned grid = (unsigned)((n_tiles16 + T - 1) / T);
  hipLaunchKernelGGL((mx_decode_kernel<WAVES, T, SPW>), dim3(grid), dim3(WAVES * 64), lds_bytes, s, p, n_tiles16);
  return hipGetLastError();
}


// ---------------------------------------------------------------------------------------------
// Weight streaming through LDS rings (whole units of 512 elements of K; plain MXFP4 takes up to 15 more blocks of 32
// behind them straight from global memory at the end).
//
// Loading B straight into MFMA operand order costs one 64-byte segment per row and instruction:
// the texture path then spends its time on address coalescing instead of moving data, and the
// waves sit in load issue.  Here the rows are copied to LDS with global_load_lds_dwordx4, 1 KB per
// wave instruction, without touching VGPRs, several items ahead of the MFMAs, and the fragments
// are then read from LDS in operand order.
//
// K is cut into NP panels of KP = 512*SPW elements (SPW = 1, 2, 4 or 8).  Four waves; wave w owns the
// K steps [w*SPW, (w+1)*SPW) of every panel -- 64*SPW bytes of every row -- for loading AND for the
// MFMAs.  Each wave therefore has a ring of its own in LDS, fills it with its own loads, waits for
// them with its own vmcnt and refills a slot as soon as it has read it: the main loop has no barrier
// at all.  (A version in which the four waves shared one ring, each loading whole rows, needed two
// barriers per item and measured 14.4 us per launch on the M=16, N=28672, K=4096 GEMM.)  The four
// partial tiles are summed through LDS at the end, the only point where the waves meet.
//
// The unit of a ring (an "item") is this wave's part of 16 rows: 16 x 64*SPW bytes of codes plus
// 16 x 4*SPW scale bytes.  Per panel a wave consumes the activation items first (their fragments
// go to registers and stay there for the panel) and then one item per 16-column tile; the fp32
// accumulators of all tiles live in registers across panels.  The activation rows take the same
// path as the weights: all loads are then of one kind and complete in issue order, which the vmcnt
// arithmetic relies on (loads that return to VGPRs may overtake loads into LDS).
//
// LDS chunk c' (16 bytes) of row r of an item holds the wave's chunk c' ^ f(r) of that row (applied on
// the source side), with f chosen so that the 16 rows a ds_read_b128 touches fall into 16 different
// bank groups: r & 15 for rows of 256 bytes or more, (r >> 1) & 7 for 128, (r >> 2) & 3 for 64.
//
// A K that is no whole number of panels ends with a SHORT panel of rem units (rem < SPW; 0: none): its items are loaded
// with the same instructions, wave w owning the K steps [w*rem, (w+1)*rem) of it, and the lanes whose chunk lies
// behind those steps fetch one of the wave's valid chunks again (source chunk (c' ^ f(r)) % (4*rem), so that LDS chunk
// (4j + g) ^ f(r) still holds source chunk 4j + g for every step j < rem); the MFMAs of the steps from rem on are
// skipped.  Hidden sizes such as 11008, 13824 or 17920 (21.5, 27 and 35 units) thereby run on panels of 2048 elements
// with one short panel at the end instead of on panels of 512.
//
// M up to 16*MB (MB = 1, 2 or 4): the activation rows of a panel are MB items of 16 rows each, every
// weight fragment is multiplied with MB activation fragments, and a tile has MB accumulators.
// NV: the operands are NVFP4 -- one E4M3 scale byte per 16 elements, twice as many scale bytes per row.
template <int SPW, bool NV = false>
struct Ring {
  static_assert(SPW == 1 || SPW == 2 || SPW == 4 || SPW == 8, "panel lengths are 512, 1024, 2048 or 4096 elements");
  static constexpr int kChunks = 4 * SPW;                                  // 16-byte chunks per item row (this wave's part)
  static constexpr int kRowBytes = 64 * SPW;
  static constexpr int kSlotData = 16 * kRowBytes;
  static constexpr int kScaleRowBytes = (NV ? 8 : 4) * SPW;                // scale bytes per item row (this wave's part)
  static constexpr int kScaleDwords = 16 * kScaleRowBytes / 4;             // per item: one lane of a scale load each
  static constexpr int kScaleLoads = (kScaleDwords + 63) / 64;             // global_load_lds_dword instructions: 256 B each
  static constexpr int kSlotBytes = kSlotData + 256 * kScaleLoads;         // one wave's slot
  static constexpr int kSlots = SPW <= 2 ? 16 : (SPW == 4 ? 8 : 4);
  static constexpr int kWaveBytes = kSlots * kSlotBytes;                   // one wave's ring
  static constexpr int kLds = 4 * kWaveBytes;                              // 81920 .. 147456; the first 28672*MB bytes are
                                                                           // reused as [4 waves][7 tiles][MB][64 lanes][16 B]
  static constexpr int kLoadsPerItem = SPW + kScaleLoads;
  static constexpr int kMaxDepth = kSlots < 7 ? kSlots : 7;                // bounded by the vmcnt immediates below
  static_assert(kMaxDepth * kLoadsPerItem < 64, "vmcnt immediate");
  __device__ static int swizzle(int row) { return SPW >= 4 ? (row & 15) : (SPW == 2 ? ((row >> 1) & 7) : ((row >> 2) & 3)); }
};

__device__ inline void dec_dma16(const void* gbase, unsigned voff, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(
                   __builtin_amdgcn_readfirstlane(lds_addr)),
               "v"(voff), "s"(gbase)
               : "m0");
}
__device__ inline void dec_dma4(const void* gbase, unsigned voff, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(
                   __builtin_amdgcn_readfirstlane(lds_addr)),
               "v"(voff), "s"(gbase)
               : "m0");
}

// waits until at most `items` (0..7) of this wave's newest items are still in flight (never more than the
// ring holds, so the immediates that would not fit the 6-bit counter are never reached)
template <int LOADS>
__device__ inline void wait_items(int items) {
  constexpr auto imm = [](int k) { return k * LOADS < 64 ? k * LOADS : 63; };
  switch (items) {
    case 0: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    case 1: asm volatile("s_waitcnt vmcnt(%0)" ::"n"(imm(1)) : "memory"); break;
    case 2: asm volatile("s_waitcnt vmcnt(%0)" ::"n"(imm(2)) : "memory"); break;
    case 3: asm volatile("s_waitcnt vmcnt(%0)" ::"n"(imm(3)) : "memory"); break;
    case 4: asm volatile("s_waitcnt vmcnt(%0)" ::"n"(imm(4)) : "memory"); break;
    case 5: asm volatile("s_waitcnt vmcnt(%0)" ::"n"(imm(5)) : "memory"); break;
    case 6: asm volatile("s_waitcnt vmcnt(%0)" ::"n"(imm(6)) : "memory"); break;
    default: asm volatile("s_waitcnt vmcnt(%0)" ::"n"(imm(7)) : "memory"); break;
  }
}

// SWIGLU: B holds 2*p.N rows, gate projections first, then up projections, and the result is
// C[m, n] = silu(gate[m, n]) * up[m, n].  A tile is then 8 gate rows and the 8 up rows of the same
// output columns, so that both halves of every output value meet in the workgroup's final reduction.

// NV: NVFP4 operands (scale_a, scale_b: the two per-tensor scales).  The items travel and are consumed in the same
// way; a fragment's 32 elements are two scale blocks, converted to f16 in registers (E2M1 x E4M3 is exact in f16) and
// fed 8 at a time to four v_mfma_f32_16x16x32_f16; the activation fragments of a panel are kept converted.
// QUANT (with SWIGLU): the bf16 result is not stored but quantised to MXFP4 (p.Q, p.Qs) exactly as the stand-alone
// quantiser would quantise it.  A block of 32 outputs is four tiles, so a workgroup owns a multiple of four tiles (up to
// eight: kTiles) and every block is complete in its final reduction.
// REM: K ends with a short panel of `rem` units (a template argument so that the forms for a whole number of panels
// carry none of it: the second set of load offsets and the step test cost the M = 16 benchmark 7 %).
template <int SPW, bool SWIGLU, int MB, bool NV = false, bool QUANT = false, bool REM = false>
__global__ __launch_bounds__(256) void mx_decode_ring_kernel(MxArgs p, int n_tiles16, int T, int NP, int depth,
                                                             const float* scale_a, const float* scale_b, int rem_units) {
  const int rem = REM ? rem_units : 0;
  static_assert(!NV || !SWIGLU, "the fused SwiGLU exists for MXFP4");
  static_assert(!QUANT || SWIGLU, "the fused quantiser follows the fused SwiGLU");
  constexpr int kTiles = QUANT ? 8 : kMaxT;   // most tiles a workgroup owns
  static_assert(!NV || MB * SPW <= 8, "converted activation fragments: 16 registers per row block and K step");
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  using R = Ring<SPW, NV>;
  constexpr int kRing = R::kSlots, kSlotBytes = R::kSlotBytes, kSlotData = R::kSlotData, NC = R::kChunks;
  constexpr unsigned panel_bytes = 256 * SPW;   // KP / 2, of which this wave owns R::kRowBytes
  constexpr unsigned panel_scales = 4 * R::kScaleRowBytes;   // the panel's scale bytes per row, a quarter of them this wave's
  // partial sums of a (tile, row block): 64 lanes x 16 bytes; the plain form pads each to 69 so that the row-wise
  // read-back below spreads over the banks
  constexpr int kBlk = SWIGLU ? 64 : 69;
  static_assert(4 * kTiles * MB * kBlk * 16 <= R::kLds, "reduction buffer");
  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int r = lane & 15, g = lane >> 4;
  const int tile0 = blockIdx.x * T;
  const int my_tiles = (n_tiles16 - tile0) < T ? (n_tiles16 - tile0) : T;   // >= 1 by grid construction
  const unsigned row_bytes = (unsigned)p.K / 2, row_scales = (unsigned)p.K / (NV ? 16 : 32);
  const unsigned ring_base = (unsigned)(uintptr_t)lds + (unsigned)w * R::kWaveBytes;   // this wave's ring
  const int per_panel = my_tiles + MB;          // MB activation items + one item per tile
  const int total = NP * per_panel;

  // ---- per-lane load coordinates inside an item -----------------------------------------------
  // data: instruction i fills LDS chunks 64i .. 64i+63 of the slot, i.e. rows 64i/NC ..; the lane fetches
  // chunk c' ^ f(row) of this wave's 64*SPW bytes of that row
  int d_row[SPW];
  unsigned d_col[SPW];
#pragma unroll
  for (int i = 0; i < SPW; ++i) {
    const int P = 64 * i + lane;
    const int rr = P / NC, cp = P % NC;
    d_row[i] = rr;
    d_col[i] = (unsigned)w * R::kRowBytes + (unsigned)((cp ^ R::swizzle(rr)) * 16);
  }
  // scales: 16 rows x SPW dwords = 16*SPW lanes of one load (two loads of 64 lanes for SPW = 8); lanes past
  // that repeat the last dword and land in the padding of the slot's scale area
  int s_row[R::kScaleLoads];
  unsigned s_col[R::kScaleLoads];
#pragma unroll
  for (int i = 0; i < R::kScaleLoads; ++i) {
    constexpr int kRowDwords = R::kScaleRowBytes / 4;
    int P = 64 * i + lane;
    P = P < R::kScaleDwords ? P : R::kScaleDwords - 1;
    s_row[i] = P / kRowDwords;
    s_col[i] = (unsigned)w * R::kScaleRowBytes + (unsigned)(P % kRowDwords) * 4;
  }

  // the same for the short last panel (rem != 0): this wave's part of a row is 64*rem bytes and 4*rem (NVFP4: 8*rem)
  // scale bytes, and what a lane would fetch from behind it wraps around onto the part's start
  unsigned d_col2[REM ? SPW : 1], s_col2[REM ? R::kScaleLoads : 1];
  if constexpr (REM) {
    const int valid = rem ? 4 * rem : NC;                                  // 16-byte chunks of this wave's part
    const int valid_dw = rem ? (NV ? 2 : 1) * rem : R::kScaleRowBytes / 4;   // scale dwords of this wave's part
#pragma unroll
    for (int i = 0; i < SPW; ++i) {
      const int P = 64 * i + lane;
      const int rr = P / NC, cp = P % NC;
      d_col2[i] = (unsigned)w * (unsigned)(16 * valid) + (unsigned)(((cp ^ R::swizzle(rr)) % valid) * 16);
    }
#pragma unroll
    for (int i = 0; i < R::kScaleLoads; ++i) {
      constexpr int kRowDwords = R::kScaleRowBytes / 4;
      int P = 64 * i + lane;
      P = P < R::kScaleDwords ? P : R::kScaleDwords - 1;
      s_col2[i] = (unsigned)w * (unsigned)(4 * valid_dw) + (unsigned)((P % kRowDwords) % valid_dw) * 4;
    }
  }

  int blocked = p.blocked_scales;
  const unsigned col_tiles = (unsigned)p.K / 128;
  asm volatile("" : "+s"(blocked));
  // copies this wave's part of rows row0 .. row0+15 (of a matrix with `rows` rows), K panel kp, and of their
  // scales into slot `sb`; item rows 8..15 are taken `jump` matrix rows further down (the up projections of a
  // SWIGLU tile).  Rows past the end of the matrix are clamped onto its last row -- also when the whole item
  // lies past the end (an activation block beyond M): their products land in rows of C that are never stored.
  // Offsets are absolute row numbers times the row pitch, which the host has checked to fit 32 bits.
  auto issue_rows = [&](const uint8_t* data, const uint8_t* scales, int row0, int rows, int kp, unsigned sb,
                        unsigned jump) {
    const uint8_t* gd = data + (size_t)kp * panel_bytes;
    const bool short_panel = REM && kp == NP - 1;   // uniform
#pragma unroll
    for (int i = 0; i < SPW; ++i) {
      const int row = row0 + d_row[i] < rows ? row0 + d_row[i] : rows - 1;
      const unsigned src_row = SWIGLU ? (unsigned)row + (d_row[i] >= 8 ? jump : 0u) : (unsigned)row;
      dec_dma16(gd, src_row * row_bytes + (short_panel ? d_col2[REM ? i : 0] : d_col[i]), sb + i * 1024);
    }
    if (!SWIGLU && !NV && blocked) {
      // 128 x 4 blocked scale tensors: a K step's four scale bytes of a row are one dword of the 512-byte tile
      // (row / 128, step); the panel's 4 * SPW column tiles lie back to back
      const uint8_t* gs = scales + (size_t)kp * (4 * SPW * 512);
#pragma unroll
      for (int i = 0; i < R::kScaleLoads; ++i) {
        const unsigned row = (unsigned)(row0 + s_row[i] < rows ? row0 + s_row[i] : rows - 1);
        dec_dma4(gs, ((row >> 7) * col_tiles + ((short_panel ? s_col2[REM ? i : 0] : s_col[i]) >> 2)) * 512 + (row & 31) * 16 +
                         ((row >> 5) & 3) * 4,
                 sb + kSlotData + i * 256);
      }
      return;
    }
    const uint8_t* gs = scales + (size_t)kp * panel_scales;
#pragma unroll
    for (int i = 0; i < R::kScaleLoads; ++i) {
      const int row = row0 + s_row[i] < rows ? row0 + s_row[i] : rows - 1;
      const unsigned src_row = SWIGLU ? (unsigned)row + (s_row[i] >= 8 ? jump : 0u) : (unsigned)row;
      dec_dma4(gs, src_row * row_scales + (short_panel ? s_col2[REM ? i : 0] : s_col[i]), sb + kSlotData + i * 256);
    }
  };
  v4i af[NV ? 1 : MB][NV ? 1 : SPW];   // MXFP4: the panel's activation fragments as loaded, and their scale bytes
  int asc[NV ? 1 : MB][NV ? 1 : SPW];
  v8h a8[NV ? MB : 1][NV ? SPW : 1][4];   // NVFP4: the same converted to f16, 8 elements per MFMA of a K step
  v4f acc[kTiles][MB];
#pragma unroll
  for (int t = 0; t < kTiles; ++t)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[t][mb] = v4f{0, 0, 0, 0};

  // Kernel arguments used on the issue path, pinned in scalar registers: left to itself the compiler
  // re-reads them from the argument segment in front of every issue and waits for that load.
  const uint8_t *gA = p.A, *gAs = p.As, *gB = p.B, *gBs = p.Bs;
  int rowsA = p.M, rowsB = p.N;
  asm volatile("" : "+s"(gA), "+s"(gAs), "+s"(gB), "+s"(gBs), "+s"(rowsA), "+s"(rowsB));

  // Items are issued in consumption order: per panel the activation rows (pos < MB), then the tiles.
  int issued = 0;                 // items handed to the loader so far; item j lives in slot j % kRing
  int next_kp = 0, next_pos = 0;  // panel and position of item number `issued`
  auto issue_next = [&]() {
    if (issued < total) {
      const unsigned sb = ring_base + (unsigned)(issued & (kRing - 1)) * kSlotBytes;
      const bool act = next_pos < MB;   // activation rows 16*next_pos .. +15
      if (SWIGLU) {
        // tile j: gate rows 8j .. 8j+7 and up rows N + 8j .. N + 8j+7; N % 8 == 0, so tiles are never ragged
        const int row0 = act ? 16 * next_pos : (tile0 + next_pos - MB) * 8;
        issue_rows(act ? gA : gB, act ? gAs : gBs, row0, act ? rowsA : row0 + 16, next_kp, sb,
                   act ? 0u : (unsigned)rowsB - 8u);
      } else {
        issue_rows(act ? gA : gB, act ? gAs : gBs, act ? 16 * next_pos : (tile0 + next_pos - MB) * 16,
                   act ? rowsA : rowsB, next_kp, sb, 0u);
      }
      ++issued;
      if (++next_pos == per_panel) {
        next_pos = 0;
        ++next_kp;
      }
    }
  };
  for (int j = 0; j < depth; ++j) issue_next();   // depth >= MB + 1: the activation items and at least one tile

  // fragment read address inside a slot: row r, chunk (4*step + g) ^ f(r); scale dword of (row r, step)
  const unsigned frag_base = (unsigned)r * R::kRowBytes;
  const int fr = R::swizzle(r);
  const unsigned sc_addr = kSlotData + (unsigned)r * R::kScaleRowBytes;
  // NVFP4: the two E4M3 bytes of this lane's 32 elements of (row r, step j) as f16
  auto nv_scales = [&](unsigned slot, int j) {
    const v2i eight = *reinterpret_cast<const __attribute__((address_space(3))) v2i*>((uintptr_t)(slot + sc_addr + j * 8));
    return scale_pair((g & 2 ? eight[1] : eight[0]) >> (16 * (g & 1)));
  };

  int i = 0;   // item being consumed
  for (int kp = 0; kp < NP; ++kp) {
    const int steps = REM && kp == NP - 1 ? rem : SPW;   // K steps of this wave in the panel
    i += MB;   // the activation items of the panel are consumed together with the first tile
#pragma unroll
    for (int pos = 1; pos <= kTiles; ++pos) {
      if (pos <= my_tiles) {
        wait_items<R::kLoadsPerItem>(issued - 1 - i);   // loads complete in issue order: item i and all before it have landed
        if (pos == 1) {
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) {
            const unsigned sa = ring_base + (unsigned)((i - MB + mb) & (kRing - 1)) * kSlotBytes;
#pragma unroll
            for (int j = 0; j < SPW; ++j) {
              const v4i raw = *reinterpret_cast<const __attribute__((address_space(3))) v4i*>(
                  (uintptr_t)(sa + frag_base + (unsigned)(((4 * j + g) ^ fr) * 16)));
              if constexpr (NV) {
                const v2h sc = nv_scales(sa, j);
#pragma unroll
                for (int d = 0; d < 4; ++d) a8[mb][j][d] = dequant8((unsigned)raw[d], sc[d >> 1]);
              } else {
                af[mb][j] = raw;
                asc[mb][j] = rotr_bytes(
                    *reinterpret_cast<const __attribute__((address_space(3))) int*>((uintptr_t)(sa + sc_addr + j * 4)), g);
              }
            }
          }
        }
        const unsigned sb = ring_base + (unsigned)(i & (kRing - 1)) * kSlotBytes;
        v4i bf[SPW];
        int bsc[NV ? 1 : SPW];
        v2h bsh[NV ? SPW : 1];
#pragma unroll
        for (int j = 0; j < SPW; ++j) {
          bf[j] = *reinterpret_cast<const __attribute__((address_space(3))) v4i*>(
              (uintptr_t)(sb + frag_base + (unsigned)(((4 * j + g) ^ fr) * 16)));
          if constexpr (NV) {
            bsh[j] = nv_scales(sb, j);
          } else {
            bsc[j] = rotr_bytes(
                *reinterpret_cast<const __attribute__((address_space(3))) int*>((uintptr_t)(sb + sc_addr + j * 4)), g);
          }
        }
#pragma unroll
        for (int j = 0; j < SPW; ++j) {
          if (REM && j >= steps) continue;   // (uniform) behind the end of a short panel
          if constexpr (NV) {
#pragma unroll
            for (int d = 0; d < 4; ++d) {
              const v8h b8 = dequant8((unsigned)bf[j][d], bsh[j][d >> 1]);
#pragma unroll
              for (int mb = 0; mb < MB; ++mb)
                acc[pos - 1][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b8, a8[mb][j][d], acc[pos - 1][mb], 0, 0, 0);
            }
          } else {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
              acc[pos - 1][mb] = mfma16<0, 0>(bf[j], af[mb][j], acc[pos - 1][mb], bsc[j], asc[mb][j]);
          }
        }
        // The slots just read are this wave's own and their contents are in registers (the MFMAs above depend
        // on them and issue in order): refill at once.
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int q = 0; q < MB + 1; ++q)   // MB + 1 at the first tile of a panel: the activation items' slots are free as well
          if (issued - (i + 1) < depth) issue_next();
        ++i;
      }
    }
  }

  // ---- K % 512 elements behind the last whole unit of 512 (MXFP4): up to 15 blocks of 32 ---------------------------
  // Wave w multiplies tail blocks 4w .. 4w+3 (lane group g: block 4w + g) straight from global memory, every lane
  // the 16 bytes and the scale byte of its own fragment rows; a lane group behind the last block fetches the wave's
  // first block instead (inside the row) and multiplies zeros under the scale 2^0.  All ring loads have landed by now
  // (the last item has been consumed), so these loads into registers are alone in flight.
  if constexpr (!NV) {
    const int tail_blocks = (p.K % 512) / 32;
    if (4 * w < tail_blocks) {   // uniform per wave
      const bool have = 4 * w + g < tail_blocks;
      const unsigned blk = (unsigned)(p.K / 512) * 16u + (unsigned)(have ? 4 * w + g : 4 * w);
      v4i ta[MB];
      int tas[MB];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const unsigned arow = (unsigned)(16 * mb + r < rowsA ? 16 * mb + r : rowsA - 1);
        ta[mb] = *reinterpret_cast<const v4i*>(gA + (size_t)arow * row_bytes + blk * 16u);
        tas[mb] = gAs[(size_t)arow * row_scales + blk];
        if (!have) {
          ta[mb] = v4i{0, 0, 0, 0};
          tas[mb] = 0x7f;
        }
      }
#pragma unroll
      for (int t = 0; t < kTiles; ++t)
        if (t < my_tiles) {
          // SWIGLU: rows 0-7 of a tile are gate rows 8 tile .., rows 8-15 the up rows of the same outputs (N % 8 == 0)
          const int n = SWIGLU ? (tile0 + t) * 8 + r + (r >= 8 ? rowsB - 8 : 0) : (tile0 + t) * 16 + r;
          const unsigned brow = (unsigned)(SWIGLU || n < rowsB ? n : rowsB - 1);
          v4i tb = *reinterpret_cast<const v4i*>(gB + (size_t)brow * row_bytes + blk * 16u);
          int tbs = gBs[(size_t)brow * row_scales + blk];
          if (!have) {
            tb = v4i{0, 0, 0, 0};
            tbs = 0x7f;
          }
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) acc[t][mb] = mfma16<0, 0>(tb, ta[mb], acc[t][mb], tbs, tas[mb]);
        }
    }
  } else {
    // NVFP4: the same tail, a block of 32 elements being two scale blocks of 16 (two E4M3 bytes) and four MFMAs of
    // 8 elements per lane; a lane group without a block multiplies zeros under the scale 1.0
    const int tail_blocks = (p.K % 512) / 32;
    if (4 * w < tail_blocks) {
      const bool have = 4 * w + g < tail_blocks;
      const unsigned blk = (unsigned)(p.K / 512) * 16u + (unsigned)(have ? 4 * w + g : 4 * w);
      const v2h one = {(_Float16)1.0f, (_Float16)1.0f};
      v8h ta8[MB][4];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const unsigned arow = (unsigned)(16 * mb + r < rowsA ? 16 * mb + r : rowsA - 1);
        v4i raw = *reinterpret_cast<const v4i*>(gA + (size_t)arow * row_bytes + blk * 16u);
        v2h sc = scale_pair(*reinterpret_cast<const unsigned short*>(gAs + (size_t)arow * row_scales + blk * 2u));
        if (!have) {
          raw = v4i{0, 0, 0, 0};
          sc = one;
        }
#pragma unroll
        for (int d = 0; d < 4; ++d) ta8[mb][d] = dequant8((unsigned)raw[d], sc[d >> 1]);
      }
#pragma unroll
      for (int t = 0; t < kTiles; ++t)
        if (t < my_tiles) {
          const int n = (tile0 + t) * 16 + r;
          const unsigned brow = (unsigned)(n < rowsB ? n : rowsB - 1);
          v4i raw = *reinterpret_cast<const v4i*>(gB + (size_t)brow * row_bytes + blk * 16u);
          v2h sc = scale_pair(*reinterpret_cast<const unsigned short*>(gBs + (size_t)brow * row_scales + blk * 2u));
          if (!have) {
            raw = v4i{0, 0, 0, 0};
            sc = one;
          }
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            const v8h b8 = dequant8((unsigned)raw[d], sc[d >> 1]);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
              acc[t][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b8, ta8[mb][d], acc[t][mb], 0, 0, 0);
          }
        }
    }
  }

  // ---- sum the four partial tiles through LDS and store bf16 ---------------------------------
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();   // every wave is done with its ring; the reduction buffer overlays them
  v4f* part = reinterpret_cast<v4f*>(lds);   // [4 waves][kTiles][MB][kBlk]
#pragma unroll
  for (int t = 0; t < kTiles; ++t)
    if (t < my_tiles)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) part[((w * kTiles + t) * MB + mb) * kBlk + lane] = acc[t][mb];
  __syncthreads();
  constexpr int kWaveStride = kTiles * MB * kBlk;   // v4f elements between the partial sums of two waves
  if constexpr (QUANT) {
    // thread -> (row block, block of 32 outputs, row, position p of 8): the block's four tiles are 4 b .. 4 b + 3, and
    // position p holds the four outputs of lane half p & 1 of tile 4 b + p / 2 -- the eight positions of a block are
    // neighbouring lanes, so its amax is three exchanges; then the stand-alone quantiser's steps on the bf16 values.
    const int blocks = my_tiles >> 2;   // my_tiles % 4 == 0: N % 32 == 0 and a multiple of four tiles per workgroup
    for (int u = tid; u < MB * blocks * 16 * 8; u += 256) {
      const int pos = u & 7, m16 = (u >> 3) & 15, rest = u >> 7;
      const int bb = rest % blocks, mb = rest / blocks;
      const int t = 4 * bb + (pos >> 1), gh = pos & 1, l = m16 + 16 * gh;
      const int tb = t * MB + mb;
      v4f gate = part[tb * 64 + l], up = part[tb * 64 + 32 + l];
#pragma unroll
      for (int ww = 1; ww < 4; ++ww) {
        gate += part[ww * kWaveStride + tb * 64 + l];
        up += part[ww * kWaveStride + tb * 64 + 32 + l];
      }
      float v[8];
#pragma unroll
      for (int e = 0; e < 4; ++e)   // rounded to bf16 first: the quantiser sees what the unfused call would have stored
        v[e] = __builtin_bit_cast(float, (unsigned)to_bf16(silu(gate[e]) * up[e]) << 16);
#pragma unroll
      for (int e = 4; e < 8; ++e) v[e] = 0.0f;
      const unsigned amax = lane_xor_max_bits(lane_xor_max_bits(lane_xor_max_bits(abs_max_bits(v), 1), 2), 4);
      const int byte = mx_scale_byte(amax);
      const float scale = mx_scale_value(byte);
      unsigned codes = 0;
      codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(codes, v[0], v[1], scale, 0);
      codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(codes, v[2], v[3], scale, 1);
      const int m = 16 * mb + m16, n = (tile0 + t) * 8 + 4 * gh;
      if (m < p.M) {
        *reinterpret_cast<uint16_t*>(p.Q + (size_t)m * (q_row_cols(p) / 2) + n / 2) = byte == 0xFF ? (uint16_t)0 : (uint16_t)(codes & 0xFFFFu);
        if (pos == 0) p.Qs[(size_t)m * (q_row_cols(p) / 32) + n / 32] = (uint8_t)byte;
      }
    }
    return;
  }
  if (SWIGLU) {
    // lanes 0-31 of a tile hold the gate values of output columns 8*tile + 4*(l/16) .. +3, lanes 32-63 the
    // up values of the same columns
    for (int u = tid; u < my_tiles * MB * 32; u += 256) {
      const int tb = u >> 5, l = u & 31;   // tb = tile * MB + row block
      v4f gate = part[tb * 64 + l], up = part[tb * 64 + 32 + l];
#pragma unroll
      for (int ww = 1; ww < 4; ++ww) {
        gate += part[ww * kWaveStride + tb * 64 + l];
        up += part[ww * kWaveStride + tb * 64 + 32 + l];
      }
      const int t = tb / MB, mb = tb % MB;
      const int m = 16 * mb + (l & 15), n = (tile0 + t) * 8 + 4 * (l >> 4);
      if (m < p.M) {   // N % 8 == 0: the four columns exist
        uint16_t* dst = p.C + (size_t)m * p.N + n;
        const float h0 = silu(gate[0]) * up[0], h1 = silu(gate[1]) * up[1];
        const float h2 = silu(gate[2]) * up[2], h3 = silu(gate[3]) * up[3];
        if ((reinterpret_cast<uintptr_t>(p.C) & 7) == 0) {
          v2i o = {(int)pack_bf16x2(h0, h1), (int)pack_bf16x2(h2, h3)};
          *reinterpret_cast<v2i*>(dst) = o;
        } else {
          dst[0] = to_bf16(h0);
          dst[1] = to_bf16(h1);
          dst[2] = to_bf16(h2);
          dst[3] = to_bf16(h3);
        }
      }
    }
    return;
  }
  const float tensor_scale = NV ? scale_a[0] * scale_b[0] : 1.0f;
  if (p.N % 8 == 0 && (tile0 + my_tiles) * 16 <= p.N && (reinterpret_cast<uintptr_t>(p.C) & 15) == 0) {
    // Whole tiles, aligned rows: a lane adds up eight consecutive outputs of one row (lanes r + 16 g and r + 16 (g + 1)
    // of a tile) and consecutive lanes walk along the row, so that the workgroup's 32 * my_tiles bytes of a row of C
    // leave as one run of 16-byte stores instead of separate 8-byte pieces per tile.  Same order of addition as below.
    const int chunks = 2 * my_tiles;
    for (int v = tid; v < MB * 16 * chunks; v += 256) {
      const int rr = v / chunks, c = v - rr * chunks;
      const int mb = rr >> 4, r16 = rr & 15, t = c >> 1, g0 = (c & 1) * 2;
      const int at = (t * MB + mb) * kBlk + r16 + 16 * g0;
      v4f s0 = part[at], s1 = part[at + 16];
#pragma unroll
      for (int ww = 1; ww < 4; ++ww) {
        s0 += part[ww * kWaveStride + at];
        s1 += part[ww * kWaveStride + at + 16];
      }
      if constexpr (NV) {
        s0 *= tensor_scale;
        s1 *= tensor_scale;
      }
      const int m = 16 * mb + r16;
      if (m < p.M) {
        const v4i o = {(int)pack_bf16x2(s0[0], s0[1]), (int)pack_bf16x2(s0[2], s0[3]), (int)pack_bf16x2(s1[0], s1[1]),
                       (int)pack_bf16x2(s1[2], s1[3])};
#ifdef AVE_EXP_STORE_WT
        store16_write_through(p.C + (size_t)m * p.N + (size_t)(tile0 + t) * 16 + 4 * g0, o);
#else
        // written through: C is not left as modified lines in eight L2s for the kernel's end to write back
        store16_write_through(p.C + (size_t)m * p.N + (size_t)(tile0 + t) * 16 + 4 * g0, o);
#endif
      }
    }
    return;
  }
  for (int u = tid; u < my_tiles * MB * 64; u += 256) {
    const int tb = u >> 6, l = u & 63;
    v4f s = part[tb * kBlk + l];
#pragma unroll
    for (int ww = 1; ww < 4; ++ww) s += part[ww * kWaveStride + tb * kBlk + l];
    if constexpr (NV) s *= tensor_scale;
    const int t = tb / MB, mb = tb % MB;
    const int m = 16 * mb + (l & 15), n = (tile0 + t) * 16 + 4 * (l >> 4);
    if (m < p.M && n < p.N) {
      uint16_t* dst = p.C + (size_t)m * p.N + n;
      if (n + 4 <= p.N && (p.N % 4 == 0) && ((reinterpret_cast<uintptr_t>(p.C) & 7) == 0)) {
        v2i o = {(int)pack_bf16x2(s[0], s[1]), (int)pack_bf16x2(s[2], s[3])};
        *reinterpret_cast<v2i*>(dst) = o;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n + e < p.N) dst[e] = to_bf16(s[e]);
      }
    }
  }
}

template <int SPW, bool SWIGLU, int MB, bool NV = false, bool QUANT = false, bool REM = false>
hipError_t launch_ring(const MxArgs& p, hipStream_t s, int n_tiles16, int T, int NP, int depth, const float* scale_a = nullptr,
                       const float* scale_b = nullptr, int rem = 0) {
  using R = Ring<SPW, NV>;
  if constexpr (!REM && SPW > 1) {   // the forms with a short last panel exist on panels of 1024 elements and more
    if (rem != 0) return launch_ring<SPW, SWIGLU, MB, NV, QUANT, true>(p, s, n_tiles16, T, NP, depth, scale_a, scale_b, rem);
  }
  if (!REM && rem != 0) return hipErrorInvalidValue;
  if (hipError_t e = allow_dynamic_lds<mx_decode_ring_kernel<SPW, SWIGLU, MB, NV, QUANT, REM>>(R::kLds); e != hipSuccess) return e;
  // at least MB + 1: the first tile of a panel is consumed together with the MB activation items in front of it
  static_assert(MB + 1 <= R::kMaxDepth, "ring too short for this many activation items");
  depth = depth < MB + 1 ? MB + 1 : (depth > R::kMaxDepth ? R::kMaxDepth : depth);
  const unsigned grid = (unsigned)((n_tiles16 + T - 1) / T);
  hipLaunchKernelGGL((mx_decode_ring_kernel<SPW, SWIGLU, MB, NV, QUANT, REM>), dim3(grid), dim3(256), R::kLds, s, p, n_tiles16, T, NP,
                     depth, scale_a, scale_b, rem);
  return hipGetLastError();
}

}  // namespace

static bool regs_supports(const MxArgs& p) {
  if (p.row_offsets) return false;
  if (p.M < 1 || p.M > 16 || p.N < 1) return false;
  if (p.K % 32 != 0) return false;
  // rows whose scales are not whole dwords are fetched at odd addresses: fine for a few MB of weights (N = K = 2880:
  // 10 us against 17 us on the generic kernel), twice as slow as that kernel for 59 MB
  if (p.K % 128 != 0 && (uint64_t)p.N * (uint64_t)(p.K / 2) > (16ull << 20)) return false;
  if ((reinterpret_cast<uintptr_t>(p.As) & 3) || (reinterpret_cast<uintptr_t>(p.Bs) & 3)) return false;
  if ((uint64_t)p.N * (uint64_t)(p.K / 2) >= (1ull << 32)) return false;   // 32-bit buffer offsets
  return true;
}

static hipError_t launch_regs(const MxArgs& p, hipStream_t s) {
  const int n_tiles16 = (p.N + 15) / 16;
  const int t = tiles_per_workgroup(n_tiles16, compute_units(), kMaxT);
  switch (t) {
    case 1: return launch_t<16, 1, 2>(p, s, n_tiles16);
    case 2: return launch_t<16, 2, 2>(p, s, n_tiles16);
    case 3: return launch_t<16, 3, 2>(p, s, n_tiles16);
    case 4: return launch_t<16, 4, 2>(p, s, n_tiles16);
    case 5: return launch_t<16, 5, 2>(p, s, n_tiles16);
    case 6: return launch_t<16, 6, 2>(p, s, n_tiles16);
    default: return launch_t<16, 7, 2>(p, s, n_tiles16);
  }
}

}  // namespace ave

namespace ave {

// Shape of the rings for a GEMM, from measurements on M=16 GEMMs (time per launch, weights from HBM):
//   N=28672, K=4096 (7 tiles per workgroup): panels of 2048 elements with 3 items in flight 14.1 us,
//     2 in flight 15.1, 4: 14.3, 5: 14.5, 6: 14.7, 7: 14.8; panels of 4096: 14.7; of 1024: 15.4; of 512: 21.3
//     (an item costs a wave a fixed sequence of wait, LDS reads, MFMAs and load issue, so short items are slow;
//     deeper queues stall the waves in load issue).
//   N=4096, K=14336 (1 tile per workgroup, every other item is activation rows served by L2): 4 in flight.
struct RingShape {
  int spw, depth;
  int np, rem;   // panels (the last one of rem units when rem != 0)
};
// row blocks of 16 activation rows: 1, 2 or 4
static int ring_row_blocks(int M) { return M <= 16 ? 1 : (M <= 32 ? 2 : 4); }

// Panel length (512 * spw elements) and items kept in flight.  spw == 0: nothing fits (four row blocks
// need 112 KB for the partial sums, which the shortest panel's rings do not provide).
static RingShape ring_shape(int K, int tiles_per_wg, int mb) {
  const int units = K / 512;
  static const int few_tiles[4] = {8, 4, 2, 1};
  static const int many_tiles[4] = {4, 8, 2, 1};
  const int* order = tiles_per_wg == 1 && mb == 1 ? few_tiles : many_tiles;
  int spw = 0;
  for (int i = 0; i < 4 && !spw; ++i) {
    if (mb == 4 && (order[i] == 1 || order[i] == 8)) continue;   // too little LDS / too short a ring
    if (units % order[i] == 0) spw = order[i];
  }
  // No long panel divides K (hidden sizes such as 11008, 13824, 17920: 21, 27 and 35 units): panels of 2048 elements
  // -- of 1024 for two or three units -- and a short panel at the end (16 x 5120 x 13824: 26.7 us on panels of 512)
  if (spw < 4 && units >= 4) spw = 4;
  else if (spw < 2 && units >= 2) spw = 2;
  if (spw == 0) return {0, 0, 0, 0};
  return {spw, tiles_per_wg == 1 ? 4 : 3, (units + spw - 1) / spw, units % spw};
}

// K: whole units of 512 through the rings; up to 15 more blocks of 32 behind them are multiplied from global memory at
// the end (MXFP4 plain and with the fused SwiGLU, and NVFP4: nv_ring_supports below)
static bool ring_supports(const MxArgs& p) {
  if (p.row_offsets) return false;
  if (p.M < 1 || p.M > 64 || p.N < 1) return false;
  if (p.K < 512 || p.K % 32 != 0) return false;
  if ((uint64_t)p.N * (uint64_t)(p.K / 2) >= (1ull << 32)) return false;   // 32-bit offsets
  const uintptr_t bits = reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.As) |
                         reinterpret_cast<uintptr_t>(p.B) | reinterpret_cast<uintptr_t>(p.Bs);
  if ((bits & 15) != 0) return false;
  return true;   // every K has a panel length for one or two row blocks; four on an odd number of units run as two launches
}

bool mx_decode_supports(const MxArgs& p) { return !p.swiglu && !p.blocked_scales && (regs_supports(p) || ring_supports(p)); }

// blocked scale tensors: the rings only, whole units of 512 (the K tail reads scale bytes row-major)
bool mx_decode_blocked_supports(const MxArgs& p) {
  if (!p.blocked_scales || p.swiglu || p.K % 512 != 0) return false;
  if ((uint64_t)((p.N + 127) / 128 * 128) * (uint64_t)(p.K / 2) >= (1ull << 32)) return false;
  // 33..64 rows over an odd number of units run as two launches on row ranges, which a blocked tensor cannot be cut into
  if (p.M > 32 && ring_shape(p.K, 2, 4).spw == 0) return false;
  return ring_supports(p);
}

// SWIGLU runs on the ring kernel only: 2N weight rows within 32-bit offsets, whole 8-column tiles
bool mx_decode_swiglu_supports(const MxArgs& p) {
  if (!p.swiglu || p.N % 8 != 0 || p.N > (1 << 30)) return false;
  MxArgs q = p;
  q.N = 2 * p.N;
  return ring_supports(q);
}

template <bool SWIGLU, int MB>
static hipError_t launch_ring_mb(const MxArgs& p, hipStream_t s) {
  const int n_tiles = SWIGLU ? p.N / 8 : (p.N + 15) / 16;   // tiles of 16 weight rows
  const int t = tiles_per_workgroup(n_tiles, compute_units(), kMaxT);
  const RingShape shape = ring_shape(p.K / 512 * 512, t, MB);
  const int np = shape.np, depth = shape.depth, rem = shape.rem;
  switch (shape.spw) {
    case 1:
      if constexpr (MB < 4) return launch_ring<1, SWIGLU, MB>(p, s, n_tiles, t, np, depth, nullptr, nullptr, rem);
      return hipErrorInvalidValue;   // excluded by ring_shape
    case 2: return launch_ring<2, SWIGLU, MB>(p, s, n_tiles, t, np, depth, nullptr, nullptr, rem);
    case 4: return launch_ring<4, SWIGLU, MB>(p, s, n_tiles, t, np, depth, nullptr, nullptr, rem);
    case 8:
      if constexpr (MB < 4) return launch_ring<8, SWIGLU, MB>(p, s, n_tiles, t, np, depth, nullptr, nullptr, rem);
      return hipErrorInvalidValue;   // excluded by ring_shape
    default: return hipErrorInvalidValue;   // no panel length: excluded by the callers
  }
}

// The fused SwiGLU + quantiser on the rings: up to 32 rows (from 33 the narrow-tile kernel's fused quantiser is the
// faster one), whole blocks of 32 outputs.
bool mx_decode_swiglu_quant_supports(const MxArgs& p) {
  if (!p.Q || !p.Qs || p.M > 32 || p.N % 32 != 0 || (reinterpret_cast<uintptr_t>(p.Q) & 1)) return false;
  return mx_decode_swiglu_supports(p);
}

template <int MB>
static hipError_t launch_ring_quant_mb(const MxArgs& p, hipStream_t s) {
  const int n_tiles = p.N / 8;   // a multiple of 4: tiles of 8 outputs, blocks of 32
  // four tiles (one block of 32 outputs) or eight per workgroup
  const int t = tiles_per_workgroup(n_tiles, compute_units(), 8, 4);
  const RingShape shape = ring_shape(p.K / 512 * 512, t, MB);
  const int np = shape.np, depth = shape.depth, rem = shape.rem;
  switch (shape.spw) {
    case 1: return launch_ring<1, true, MB, false, true>(p, s, n_tiles, t, np, depth, nullptr, nullptr, rem);
    case 2: return launch_ring<2, true, MB, false, true>(p, s, n_tiles, t, np, depth, nullptr, nullptr, rem);
    case 4: return launch_ring<4, true, MB, false, true>(p, s, n_tiles, t, np, depth, nullptr, nullptr, rem);
    default: return launch_ring<8, true, MB, false, true>(p, s, n_tiles, t, np, depth, nullptr, nullptr, rem);
  }
}

template <bool SWIGLU>
static hipError_t launch_ring_any(const MxArgs& p, hipStream_t s) {
  if constexpr (SWIGLU) {
    if (p.Q) return p.M <= 16 ? launch_ring_quant_mb<1>(p, s) : launch_ring_quant_mb<2>(p, s);
  }
  switch (ring_row_blocks(p.M)) {
    case 1: return launch_ring_mb<SWIGLU, 1>(p, s);
    case 2: return launch_ring_mb<SWIGLU, 2>(p, s);
    default: break;
  }
  if (ring_shape(p.K / 512 * 512, 2, 4).spw != 0) return launch_ring_mb<SWIGLU, 4>(p, s);
  // Four row blocks want an even number of 512-element units (their partial sums need the LDS of the longer panels'
  // rings).  With an odd number the rows go in two launches of two row blocks each: twice the weight traffic, still
  // several times faster than the shape-agnostic kernel.
  MxArgs q = p;
  q.M = 32;
  if (hipError_t e = launch_ring_mb<SWIGLU, 2>(q, s); e != hipSuccess) return e;
  q.A += (size_t)32 * (size_t)(p.K / 2);
  q.As += (size_t)32 * (size_t)(p.K / 32);
  q.C += (size_t)32 * (size_t)p.N;
  q.M = p.M - 32;
  return launch_ring_mb<SWIGLU, 2>(q, s);
}

// NVFP4 on the rings: at most 64 rows (the converted activation fragments of a panel live in registers: 16 per row
// block and K step, so four row blocks -- 33..64 rows -- take panels of 1024 elements and an even number of
// 512-element units; up to 32 rows take panels of 2048 and any number of units, the last panel a short one), K a
// multiple of 32 from 512 up (whole units through the rings, the rest from global memory at the end), 16-byte aligned
// operands, 32-bit offsets.
bool nv_ring_supports(const NvArgs& p) {
  if (p.M < 1 || p.M > 64 || p.N < 1 || p.K < 512 || p.K % 32 != 0) return false;
  // four row blocks: whole panels of 1024 elements (with a short panel at the end the loads into registers of
  // nv_decode_kernel are the faster choice there: 48 x 5120 x 13824 40 against 45 us)
  if (p.M > 32 && (p.K / 512) % 2 != 0) return false;
  if ((uint64_t)p.N * (uint64_t)(p.K / 2) >= (1ull << 32)) return false;
  const uintptr_t bits = reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.As) |
                         reinterpret_cast<uintptr_t>(p.B) | reinterpret_cast<uintptr_t>(p.Bs);
  return (bits & 15) == 0;
}

hipError_t launch_nv_ring(const NvArgs& p, hipStream_t s) {
  const MxArgs q{p.A, p.As, p.B, p.Bs, p.C, p.M, p.N, p.K, nullptr, 0, 0};
  const int mb = p.M <= 16 ? 1 : (p.M <= 32 ? 2 : 4);
  const int n_tiles = (p.N + 15) / 16;
  const int t = tiles_per_workgroup(n_tiles, compute_units(), kMaxT);
  const int units = p.K / 512, depth = t == 1 ? 4 : 3;
  // Panels of 512 * spw elements, as long as the registers of the converted activation fragments allow (16 per row
  // block and K step: spw 4, 4 and 2 for one, two and four row blocks) and K holds; a K that is no whole number of
  // panels ends with a short one.
  int spw = mb == 4 ? 2 : 4;
  while (spw > units) spw /= 2;
  const int np = (units + spw - 1) / spw, rem = units % spw;
  switch (mb * 10 + spw) {
    case 14: return launch_ring<4, false, 1, true>(q, s, n_tiles, t, np, depth, p.Ag, p.Bg, rem);
    case 12: return launch_ring<2, false, 1, true>(q, s, n_tiles, t, np, depth, p.Ag, p.Bg, rem);
    case 11: return launch_ring<1, false, 1, true>(q, s, n_tiles, t, np, depth, p.Ag, p.Bg, rem);
    case 24: return launch_ring<4, false, 2, true>(q, s, n_tiles, t, np, depth, p.Ag, p.Bg, rem);
    case 22: return launch_ring<2, false, 2, true>(q, s, n_tiles, t, np, depth, p.Ag, p.Bg, rem);
    case 21: return launch_ring<1, false, 2, true>(q, s, n_tiles, t, np, depth, p.Ag, p.Bg, rem);
    case 42: return launch_ring<2, false, 4, true>(q, s, n_tiles, t, np, depth, p.Ag, p.Bg, rem);
    default: return hipErrorInvalidValue;   // four row blocks on a single unit: excluded by nv_ring_supports
  }
}

hipError_t launch_mx_decode(const MxArgs& p, hipStream_t s) {
  if (p.swiglu) return launch_ring_any<true>(p, s);
  if (!ring_supports(p) && !p.blocked_scales) return launch_regs(p, s);
  return launch_ring_any<false>(p, s);
}

}  // namespace ave
