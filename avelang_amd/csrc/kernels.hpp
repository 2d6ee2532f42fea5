// Host-side launch interface shared by the kernel translation units and the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace ave {

struct MxArgs {
  const uint8_t* A;        // [M, K/2] packed E2M1
  const uint8_t* As;       // [M, K/32] E8M0
  const uint8_t* B;        // [N, K/2] or [E, N, K/2]
  const uint8_t* Bs;       // [N, K/32] or [E, N, K/32]
  uint16_t* C;             // [M, N] bf16
  int M, N, K;
  const int32_t* row_offsets;  // nullptr for a plain GEMM; else device [E+1]
  int E;
  int swiglu;                  // 1: B holds 2N rows (gate rows, then up rows) and C[m,n] = silu(gate) * up
  uint8_t* Q = nullptr;        // swiglu only: when set, the bf16 result is not stored but quantised to MXFP4:
  uint8_t* Qs = nullptr;       //   Q [M, q_n/2] packed E2M1, Qs [M, q_n/32] E8M0 (N % 32 == 0)
  int q_n = 0;                 //   columns that a row of Q and Qs is laid out for: 0 = N; more (a multiple of 32): the
                               //   rows are padded for a consumer that wants K % 512 == 0, columns N.. are not written
  float* P = nullptr;          // split K only: partial sums [slices][M][N]
  int slices = 1;              //   K slices of slice_pairs x 512 elements each (the last one what is left)
  int slice_pairs = 0;
  int half_rows = 0;           //   narrow-tile kernel only: 1 = the slices run on its 128-row tiles
  int touch = 0;               // 256 x 256 kernel, plain GEMM: 1 = look-ahead touches of the next round's panels (weights
                               //   expected to come from HBM rather than from the last-level cache)
  int blocked_scales = 0;      // 1: As and Bs are in the 128 x 4 blocked layout (plain GEMM, K % 512 == 0): padded to
                               //   128 rows and 4 columns, 512-byte tiles in row-major tile order, scale (r, c) of a
                               //   tile at byte (r % 32) * 16 + (r / 32) * 4 + c
};

__host__ __device__ inline int q_row_cols(const MxArgs& p) { return p.q_n > 0 ? p.q_n : p.N; }

// How launch_mx_tile_splitk would cut K for a shape on the current device; slices == 1: it would not.
struct SplitPlan {
  int slices = 1;
  int slice_pairs = 0;
  size_t workspace_bytes = 0;
  bool narrow = false;   // the slices run on the narrow-tile kernel (launch_mx_narrow_splitk) ...
  bool half = false;     // ... on its 128 x 128 tiles (four stage buffers) rather than 256 x 128
};
// max_workspace_bytes: only splits whose partial sums fit are considered (the best of those, or no split)
SplitPlan mx_tile_split_plan(int M, int N, int K, size_t max_workspace_bytes = ~(size_t)0);
SplitPlan mx_tile_split_plan_for(int M, int N, int K, int compute_units,
                                 size_t max_workspace_bytes = ~(size_t)0);   // host arithmetic only
// the NVFP4 tile kernel's split: slice_pairs holds the 256-element stages per slice
SplitPlan nv_tile_split_plan(int M, int N, int K);
SplitPlan nv_tile_split_plan_for(int M, int N, int K, int compute_units);

struct NvArgs {
  const uint8_t* A;        // [M, K/2]
  const uint8_t* As;       // [M, K/16] E4M3
  const float* Ag;         // [1]
  const uint8_t* B;        // [N, K/2]
  const uint8_t* Bs;       // [N, K/16]
  const float* Bg;         // [1]
  uint16_t* C;
  int M, N, K;
  float* P = nullptr;      // split K only: partial sums [slices][M][N]
  int slices = 1;          //   K slices of slice_stages x 256 elements each (the last one what is left)
  int slice_stages = 0;
};

// Raises a kernel's dynamic-LDS limit above the 64 KB default, once per kernel and device (the
// attribute is per device; bit d of the mask records that device d has it).  Thread-safe; devices past
// the 64th set it on every launch.
template <auto Kernel>
hipError_t allow_dynamic_lds(int bytes) {
  static std::atomic<uint64_t> done{0};
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
  if (dev >= 0 && dev < 64 && ((done.load(std::memory_order_acquire) >> dev) & 1)) return hipSuccess;
  const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(Kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess && dev >= 0 && dev < 64) done.fetch_or(1ull << dev, std::memory_order_release);
  return e;
}

// Tiles per workgroup for a weight-streaming launch: n_tiles tiles, workgroups of t tiles (t a multiple of `step`, at
// most t_max) that run in rounds of `cus` at a time.  A workgroup costs about one tile's time to start and to
// finish on top of its tiles, so the choice minimises rounds * (t + 1): one round of ceil(n_tiles / cus) tiles when
// that fits t_max (N = 28672: 7 tiles of 16 rows on each of 256 compute units), and balanced rounds beyond it
// (N = 32768: two rounds of 4 tiles, where 7 tiles per workgroup would run a second round for a seventh of the chip).
inline int tiles_per_workgroup(int n_tiles, int cus, int t_max, int step = 1) {
  if (cus <= 0) cus = 256;
  int best = step;
  long best_cost = -1;
  for (int t = step; t <= t_max; t += step) {
    const long wgs = (n_tiles + t - 1) / t;
    const long cost = (wgs + cus - 1) / cus * (t + 1);
    if (best_cost < 0 || cost < best_cost || (cost == best_cost && t > best)) {
      best = t;
      best_cost = cost;
    }
  }
  return best;
}

// Each launcher validates nothing: callers (the C ABI) check shapes and alignment first.
// grid.x of the shape-agnostic kernels for a matrix with N columns and m_tiles tiles of 32 rows (host arithmetic):
// ceil(N / 128) * m_tiles, or 0 when that does not fit one grid dimension
unsigned generic_grid(int N, uint64_t m_tiles, unsigned* n_blocks);
hipError_t launch_mx_generic(const MxArgs& p, hipStream_t s);
hipError_t launch_nv_generic(const NvArgs& p, hipStream_t s);
hipError_t launch_mx_tile(const MxArgs& p, hipStream_t s);
hipError_t launch_mx_tile_splitk(const MxArgs& p, hipStream_t s);   // p.P, p.slices, p.slice_pairs from a SplitPlan
hipError_t launch_mx_narrow_splitk(const MxArgs& p, hipStream_t s);
// C = bf16(P[0] + ... + P[slices-1]) in slice order; P[s] is [mn] floats
hipError_t launch_splitk_reduce(const float* P, uint16_t* C, size_t mn, int slices, hipStream_t s);
hipError_t launch_mx_narrow(const MxArgs& p, hipStream_t s);
hipError_t launch_mx_decode(const MxArgs& p, hipStream_t s);
hipError_t launch_nv_tile(const NvArgs& p, hipStream_t s);
hipError_t launch_nv_f16_tile(const NvArgs& p, hipStream_t s);   // any K % 16 == 0: every element dequantised once per workgroup
hipError_t launch_nv_decode(const NvArgs& p, hipStream_t s);
hipError_t launch_nv_ring(const NvArgs& p, hipStream_t s);          // the LDS-ring weight-streaming kernel, M <= 64
hipError_t launch_nv_tile_splitk(const NvArgs& p, hipStream_t s);   // p.P, p.slices, p.slice_stages from nv_tile_split_plan

// x: [rows, k] fp32 or bf16 -> packed [rows, k_padded/2] bytes, scales [rows, k_padded/32] bytes; the blocks behind
// column k of a row are written as blocks of zeros (k_padded >= k, both multiples of 32)
hipError_t launch_quantize_mx(const void* x, int is_bf16, uint8_t* packed, uint8_t* scales, size_t rows, int k,
                              int k_padded, hipStream_t s);

// x: [n_blocks*16] fp32 or bf16, global_scale: device [1] -> packed [n_blocks*8] bytes, scales [n_blocks] E4M3 bytes
hipError_t launch_quantize_nv(const void* x, int is_bf16, const float* global_scale, uint8_t* packed, uint8_t* scales,
                              size_t n_blocks, hipStream_t s);

// MoE routing (one workgroup) and row gather; see moe_route.hip
int route_top2_max_experts();
hipError_t launch_route_top2(const float* logits, int T, int E, int32_t* token_of_row, int32_t* row_offsets,
                             float* row_weight, int32_t* rows_of_token, hipStream_t s);
hipError_t launch_combine_top2(const uint16_t* rows, const int32_t* rows_of_token, const float* row_weight, int T, int H,
                               int n_rows, int renormalize, uint16_t* out, hipStream_t s);
hipError_t launch_gather_rows(const uint8_t* src, const uint8_t* src_s, const int32_t* index, int rows, int src_rows,
                              int K, uint8_t* dst, uint8_t* dst_s, hipStream_t s);

// row-major [rows, cols] scale bytes <-> 128 x 4 blocked layout; see scale_layout.hip
hipError_t launch_scale_layout(const uint8_t* src, uint8_t* dst, int rows, int cols, bool to_blocked, hipStream_t s);

// Diagnostic: `workgroups` x 8 waves each issue `iters` x 8 scaled FP4 MFMAs on operand fragments taken from
// `codes` (`bytes` >= 16, 16-byte aligned); `sink` is one float that is practically never written.
hipError_t launch_mfma_rate(const uint8_t* codes, size_t bytes, int workgroups, int iters, float* sink, hipStream_t s);
double mfma_rate_flop(int workgroups, int iters);
// the same with v_mfma_f32_32x32x16_f16 on the codes dequantised to f16 (the NVFP4 kernels' matrix instruction)
hipError_t launch_mfma_rate_f16(const uint8_t* codes, size_t bytes, int workgroups, int iters, float* sink, hipStream_t s);
double mfma_rate_f16_flop(int workgroups, int iters);
// Diagnostic: `workgroups` x 256 lanes read `bytes` (a multiple of 16) once, 16 bytes per lane and trip, and write
// nothing; `sink` is one int that is practically never written.
hipError_t launch_stream_read(const void* src, size_t bytes, int workgroups, int* sink, void* dst, size_t dst_bytes,
                              hipStream_t s);

// compute units of the current device rounded down to a multiple of 8 (one share per XCD); 0 if the query fails
int compute_units();

bool mx_tile_supports(const MxArgs& p);
bool mx_tile_blocked_supports(const MxArgs& p);     // p.blocked_scales: the 256 x 256 kernel reads blocked scale tensors for this shape
bool mx_decode_blocked_supports(const MxArgs& p);   // ... the weight-streaming kernel does
bool mx_narrow_supports(const MxArgs& p);    // the 256 x 128 tile kernel can run the shape
bool mx_narrow_preferred(const MxArgs& p);   // ... and shape-based dispatch picks it
bool mx_decode_supports(const MxArgs& p);
bool mx_decode_swiglu_supports(const MxArgs& p);
bool mx_decode_swiglu_quant_supports(const MxArgs& p);   // ... with the fused quantiser (p.Q, p.Qs): up to 32 rows
bool nv_tile_supports(const NvArgs& p);
bool nv_f16_tile_supports(const NvArgs& p);
bool nv_decode_supports(const NvArgs& p);
bool nv_ring_supports(const NvArgs& p);

}  // namespace ave
