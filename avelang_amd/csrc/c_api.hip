// C ABI of libave_fp4.so: argument checks, kernel selection, error text.  No allocation,
// no synchronisation, nothing but kernel launches on the caller's stream.
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include <atomic>
#include <mutex>

#include "../../include/ave_fp4.h"
#include "../../include/ave_fp4_debug.h"
#include "kernels.hpp"
#include "tile_map.hpp"

// Scratch of ave_fp4_gemm_mxfp4_noalloc: the fp32 partial sums of a GEMM whose K is split over the compute units, for
// callers that cannot allocate a workspace.  Every GPU the library runs on holds its own copy of the array, at its
// own address, until the process ends.  In host code the array's name is only a handle for hipGetSymbolAddress, not
// a device address: kernels get the pointer that scratch_pointer() returns.
static __device__ __align__(256) unsigned char scratch[AVE_FP4_NOALLOC_SCRATCH_BYTES];

namespace {

thread_local char g_err[512] = "";

int fail_inval(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return AVE_FP4_EINVAL;
}

int finish(hipError_t e, const char* what) {
  if (e == hipSuccess) return 0;
  // same wording the reference uses for HIP failures (backends/amdgpu/driver.py:125-138)
  snprintf(g_err, sizeof(g_err), "ave-lang Error [HIP]: %s (%s)", hipGetErrorString(e), what);
  return (int)e;
}

bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// Whether a GEMM's weights are likely to come from HBM rather than from the 256 MB last-level cache: a small model
// of that cache's contents, kept per device -- the weight tensors of the latest shape-dispatched MXFP4 GEMMs, most
// recent first.  Weights found among the latest ones whose sizes add up to 192 MB at most are taken to be resident (one
// GEMM replayed on the same operands, a small block replayed in a graph); anything else is taken to be cold (a model's
// layers, each with weights of its own, whose turn comes again after the whole model has passed through the cache).
// The 256 x 256 kernel then runs with or without its look-ahead touches (7 % faster from HBM, 1 % slower from the
// cache, the same bits either way).  A hint only: a wrong guess costs a few per cent.  Decided when the call is made, so
// a captured launch keeps its form on every replay.
bool weights_likely_from_hbm(const void* B, size_t bytes) {
  struct Recent {
    const void* ptr[8];
    size_t bytes[8];
    int n = 0;
  };
  static Recent recent[64];
  static std::mutex mu;
  constexpr size_t kWindow = 192u << 20;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;   // no device (host-side tests): one list
  std::lock_guard<std::mutex> lock(mu);
  Recent& r = recent[dev];
  int at = -1;
  size_t seen = 0;
  for (int i = 0; i < r.n && at < 0; ++i) {
    seen += r.bytes[i];
    if (r.ptr[i] == B) at = i;
  }
  const bool resident = at >= 0 && seen <= kWindow;
  // move (or put) B to the front
  const int last = at >= 0 ? at : (r.n < 8 ? r.n++ : 7);
  for (int i = last; i > 0; --i) {
    r.ptr[i] = r.ptr[i - 1];
    r.bytes[i] = r.bytes[i - 1];
  }
  r.ptr[0] = B;
  r.bytes[0] = bytes;
  return !resident;
}

// Device address of `scratch` on the current device, looked up once per device (with that device current) and
// kept.  Null with *err set when the lookup fails.
void* scratch_pointer(hipError_t* err) {
  static std::atomic<void*> cached[64];
  *err = hipSuccess;
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) {
    *err = e;
    return nullptr;
  }
  const bool slot = dev >= 0 && dev < 64;
  if (slot) {
    if (void* p = cached[dev].load(std::memory_order_acquire)) return p;
  }
  void* ptr = nullptr;
  if (hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)); e != hipSuccess || !ptr) {
    *err = e != hipSuccess ? e : hipErrorInvalidSymbol;
    return nullptr;
  }
  if (slot) cached[dev].store(ptr, std::memory_order_release);
  return ptr;
}

int check_common(const void* A, const void* As, const void* B, const void* Bs, const void* C, int M, int N, int K,
                 int kblock, size_t data_align) {
  if (M < 0) return fail_inval("M must be non-negative, got %d.", M);
  if (N < 0) return fail_inval("N must be non-negative, got %d.", N);
  if (K <= 0 || K % kblock != 0) return fail_inval("K must be a positive multiple of %d, got %d.", kblock, K);
  if (M == 0 || N == 0) return 0;
  if (!A || !As || !B || !Bs || !C) return fail_inval("null device pointer.");
  if (!aligned(A, data_align) || !aligned(B, data_align))
    return fail_inval("A and B must be %zu-byte aligned.", data_align);
  if (!aligned(C, 2)) return fail_inval("C must be 2-byte aligned.");
  return 0;
}

}  // namespace

extern "C" {

const char* ave_fp4_last_error(void) { return g_err; }

int ave_fp4_abi_version(void) { return 1; }

int ave_fp4_debug_tiles_per_workgroup(int n_tiles, int compute_units, int t_max, int step) {
  if (n_tiles < 1 || t_max < 1 || step < 1 || step > t_max) return 0;
  return ave::tiles_per_workgroup(n_tiles, compute_units, t_max, step);
}

int ave_fp4_debug_weights_from_hbm(const void* B, size_t bytes) { return weights_likely_from_hbm(B, bytes) ? 1 : 0; }

int ave_fp4_debug_map_tile(int pid, int m_tiles, int n_tiles, int* tm, int* tn) {
  g_err[0] = 0;
  if (m_tiles <= 0 || n_tiles <= 0 || pid < 0 || pid >= m_tiles * n_tiles || !tm || !tn)
    return fail_inval("pid %d outside a %d x %d tile grid.", pid, m_tiles, n_tiles);
  ave::map_tile(pid, m_tiles, n_tiles, *tm, *tn);
  return 0;
}

int ave_fp4_debug_locate_group_tile(const int32_t* row_offsets, int E, int total_M, int tile_rows, int tm, int* expert,
                                    int* m_begin, int* m_end) {
  g_err[0] = 0;
  if (!row_offsets || !expert || !m_begin || !m_end) return fail_inval("null pointer.");
  if (E <= 0 || total_M < 0 || tile_rows <= 0 || tm < 0)
    return fail_inval("E and tile_rows must be positive, total_M and tm non-negative (got %d, %d, %d, %d).", E, tile_rows,
                      total_M, tm);
  return ave::locate_group_tile(row_offsets, E, total_M, tile_rows, tm, *expert, *m_begin, *m_end) ? 1 : 0;
}

int ave_fp4_debug_generic_grid(int M, int N, int E, unsigned* workgroups) {
  g_err[0] = 0;
  if (!workgroups) return fail_inval("null pointer.");
  if (M <= 0 || N <= 0 || E < 0) return fail_inval("M and N must be positive and E non-negative (got %d, %d, %d).", M, N, E);
  unsigned n_blocks;
  *workgroups = ave::generic_grid(N, ((uint64_t)M + 31) / 32 + (uint64_t)E, &n_blocks);
  return 0;
}

int ave_fp4_debug_mfma_rate(const uint8_t* codes, size_t bytes, int workgroups, int iters, float* sink,
                            void* hip_stream, double* flop) {
  g_err[0] = 0;
  if (!codes || !sink || !flop) return fail_inval("codes, sink and flop must not be null.");
  if (bytes < 16 || !aligned(codes, 16)) return fail_inval("codes must hold at least 16 bytes, 16-byte aligned.");
  if (workgroups <= 0 || workgroups > (1 << 20) || iters <= 0)
    return fail_inval("workgroups must be in 1..2^20 and iters positive (got %d, %d).", workgroups, iters);
  *flop = ave::mfma_rate_flop(workgroups, iters);
  return finish(ave::launch_mfma_rate(codes, bytes, workgroups, iters, sink, static_cast<hipStream_t>(hip_stream)),
                "matrix-core rate probe");
}

int ave_fp4_debug_mfma_rate_f16(const uint8_t* codes, size_t bytes, int workgroups, int iters, float* sink,
                                void* hip_stream, double* flop) {
  g_err[0] = 0;
  if (!codes || !sink || !flop) return fail_inval("codes, sink and flop must not be null.");
  if (bytes < 16 || !aligned(codes, 16)) return fail_inval("codes must hold at least 16 bytes, 16-byte aligned.");
  if (workgroups <= 0 || workgroups > (1 << 20) || iters <= 0)
    return fail_inval("workgroups must be in 1..2^20 and iters positive (got %d, %d).", workgroups, iters);
  *flop = ave::mfma_rate_f16_flop(workgroups, iters);
  return finish(ave::launch_mfma_rate_f16(codes, bytes, workgroups, iters, sink, static_cast<hipStream_t>(hip_stream)),
                "f16 matrix-core rate probe");
}

int ave_fp4_debug_stream_read(const void* src, size_t bytes, int workgroups, int32_t* sink, void* hip_stream) {
  g_err[0] = 0;
  if (!src || !sink) return fail_inval("src and sink must not be null.");
  if (bytes < 16 || bytes % 16 != 0 || !aligned(src, 16)) return fail_inval("src must hold a multiple of 16 bytes, 16-byte aligned.");
  if (workgroups <= 0 || workgroups > (1 << 20)) return fail_inval("workgroups must be in 1..2^20, got %d.", workgroups);
  return finish(ave::launch_stream_read(src, bytes, workgroups, sink, nullptr, 0, static_cast<hipStream_t>(hip_stream)),
                "streaming-read probe");
}

int ave_fp4_debug_stream_read_write(const void* src, size_t bytes, void* dst, size_t dst_bytes, int workgroups,
                                    int32_t* sink, void* hip_stream) {
  g_err[0] = 0;
  if (!src || !sink || !dst) return fail_inval("src, dst and sink must not be null.");
  if (bytes < 16 || bytes % 16 != 0 || !aligned(src, 16)) return fail_inval("src must hold a multiple of 16 bytes, 16-byte aligned.");
  if (dst_bytes % 16 != 0 || !aligned(dst, 16)) return fail_inval("dst must hold a multiple of 16 bytes, 16-byte aligned.");
  if (workgroups <= 0 || workgroups > (1 << 20)) return fail_inval("workgroups must be in 1..2^20, got %d.", workgroups);
  return finish(ave::launch_stream_read(src, bytes, workgroups, sink, dst, dst_bytes, static_cast<hipStream_t>(hip_stream)),
                "streaming-read-and-write probe");
}

int ave_fp4_gemm_mxfp4_ex(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B, const uint8_t* B_scale,
                          uint16_t* C, int M, int N, int K, void* hip_stream, int variant) {
  g_err[0] = 0;
  if (int rc = check_common(A, A_scale, B, B_scale, C, M, N, K, 32, 16)) return rc;
  if (M == 0 || N == 0) return 0;
  ave::MxArgs p{A, A_scale, B, B_scale, C, M, N, K, nullptr, 0};
  hipStream_t s = static_cast<hipStream_t>(hip_stream);
  switch (variant) {
    case AVE_FP4_AUTO:
      // (33..64 rows against a nearly full round of 128-row tiles: the narrow-tile kernel ahead of the rings)
      if (M > 32 && M <= 64 && ave::mx_narrow_preferred(p)) return finish(ave::launch_mx_narrow(p, s), "mxfp4 narrow-tile kernel");
      if (ave::mx_decode_supports(p)) return finish(ave::launch_mx_decode(p, s), "mxfp4 decode kernel");
      if (ave::mx_narrow_preferred(p)) return finish(ave::launch_mx_narrow(p, s), "mxfp4 narrow-tile kernel");
      // (a K that is no multiple of 256 costs the tile kernel a tail read straight from global memory: with at most
      // 64 rows the generic kernel is as fast or faster)
      if (ave::mx_tile_supports(p) && (M > 64 || K % 256 == 0)) {
        p.touch = weights_likely_from_hbm(B, (size_t)N * (size_t)(K / 2 + K / 32)) ? 1 : 0;
        return finish(ave::launch_mx_tile(p, s), "mxfp4 tile kernel");
      }
      return finish(ave::launch_mx_generic(p, s), "mxfp4 generic kernel");
    case AVE_FP4_GENERIC:
      return finish(ave::launch_mx_generic(p, s), "mxfp4 generic kernel");
    case AVE_FP4_TILE:
    case AVE_FP4_TILE_STREAMED:
      if (!ave::mx_tile_supports(p)) return fail_inval("tile kernel does not support M=%d N=%d K=%d.", M, N, K);
      p.touch = variant == AVE_FP4_TILE_STREAMED ? 1 : 0;
      return finish(ave::launch_mx_tile(p, s), "mxfp4 tile kernel");
    case AVE_FP4_DECODE:
      if (!ave::mx_decode_supports(p)) return fail_inval("decode kernel does not support M=%d N=%d K=%d.", M, N, K);
      return finish(ave::launch_mx_decode(p, s), "mxfp4 decode kernel");
    case AVE_FP4_NARROW:
      if (!ave::mx_narrow_supports(p)) return fail_inval("narrow-tile kernel does not support M=%d N=%d K=%d.", M, N, K);
      return finish(ave::launch_mx_narrow(p, s), "mxfp4 narrow-tile kernel");
    default:
      return fail_inval("unknown kernel variant %d.", variant);
  }
}

int ave_fp4_gemm_mxfp4(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B, const uint8_t* B_scale,
                       uint16_t* C, int M, int N, int K, void* hip_stream) {
  return ave_fp4_gemm_mxfp4_ex(A, A_scale, B, B_scale, C, M, N, K, hip_stream, AVE_FP4_AUTO);
}

int ave_fp4_gemm_mxfp4_blocked_scales(const uint8_t* A, const uint8_t* A_scale_blocked, const uint8_t* B,
                                      const uint8_t* B_scale_blocked, uint16_t* C, int M, int N, int K, void* hip_stream) {
  g_err[0] = 0;
  if (int rc = check_common(A, A_scale_blocked, B, B_scale_blocked, C, M, N, K, 32, 16)) return rc;
  if (M == 0 || N == 0) return 0;
  if (K % 512 != 0)
    return fail_inval("blocked scale tensors are read by the kernels that work on whole 512-element units of K (got K = %d): "
                      "convert them with ave_fp4_scales_from_blocked and call ave_fp4_gemm_mxfp4.", K);
  if (!aligned(A_scale_blocked, 16) || !aligned(B_scale_blocked, 16)) return fail_inval("blocked scale tensors must be 16-byte aligned.");
  ave::MxArgs p{A, A_scale_blocked, B, B_scale_blocked, C, M, N, K, nullptr, 0};
  p.blocked_scales = 1;
  hipStream_t s = static_cast<hipStream_t>(hip_stream);
  if (ave::mx_decode_blocked_supports(p)) return finish(ave::launch_mx_decode(p, s), "mxfp4 decode kernel, blocked scales");
  if (ave::mx_tile_blocked_supports(p)) return finish(ave::launch_mx_tile(p, s), "mxfp4 tile kernel, blocked scales");
  return fail_inval("no kernel reads blocked scale tensors for M=%d N=%d K=%d (operands of 4 GB and more): convert them with "
                    "ave_fp4_scales_from_blocked and call ave_fp4_gemm_mxfp4.", M, N, K);
}

size_t ave_fp4_gemm_mxfp4_workspace_bytes(int M, int N, int K) { return ave::mx_tile_split_plan(M, N, K).workspace_bytes; }

int ave_fp4_debug_split_plan_capped(int M, int N, int K, int compute_units, size_t max_workspace_bytes, int* slices,
                                    int* slice_pairs, int* narrow_tiles, size_t* workspace_bytes) {
  g_err[0] = 0;
  if (!slices || !slice_pairs || !narrow_tiles || !workspace_bytes) return fail_inval("null output pointer.");
  if (compute_units <= 0) return fail_inval("compute_units must be positive, got %d.", compute_units);
  const ave::SplitPlan plan = ave::mx_tile_split_plan_for(M, N, K, compute_units, max_workspace_bytes);
  *slices = plan.slices;
  *slice_pairs = plan.slice_pairs;
  *narrow_tiles = plan.narrow ? (plan.half ? 2 : 1) : 0;
  *workspace_bytes = plan.workspace_bytes;
  return 0;
}

int ave_fp4_debug_split_plan(int M, int N, int K, int compute_units, int* slices, int* slice_pairs, int* narrow_tiles,
                             size_t* workspace_bytes) {
  return ave_fp4_debug_split_plan_capped(M, N, K, compute_units, ~(size_t)0, slices, slice_pairs, narrow_tiles, workspace_bytes);
}

static int gemm_mxfp4_split(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B, const uint8_t* B_scale,
                            uint16_t* C, int M, int N, int K, void* workspace, size_t workspace_bytes,
                            const ave::SplitPlan& plan, void* hip_stream) {
  ave::MxArgs p{A, A_scale, B, B_scale, C, M, N, K, nullptr, 0};
  p.P = static_cast<float*>(workspace);
  p.slices = plan.slices;
  p.slice_pairs = plan.slice_pairs;
  p.half_rows = plan.half ? 1 : 0;
  if (plan.narrow)
    return finish(ave::launch_mx_narrow_splitk(p, static_cast<hipStream_t>(hip_stream)), "mxfp4 narrow-tile kernel, split K");
  return finish(ave::launch_mx_tile_splitk(p, static_cast<hipStream_t>(hip_stream)), "mxfp4 tile kernel, split K");
}

int ave_fp4_gemm_mxfp4_ws(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B, const uint8_t* B_scale,
                          uint16_t* C, int M, int N, int K, void* workspace, size_t workspace_bytes, void* hip_stream) {
  g_err[0] = 0;
  if (int rc = check_common(A, A_scale, B, B_scale, C, M, N, K, 32, 16)) return rc;
  if (M == 0 || N == 0) return 0;
  if (workspace_bytes > 0 && !workspace) return fail_inval("null workspace with workspace_bytes = %zu.", workspace_bytes);
  if (workspace && !aligned(workspace, 16)) return fail_inval("workspace must be 16-byte aligned.");
  const ave::SplitPlan plan = ave::mx_tile_split_plan(M, N, K);
  if (plan.slices > 1 && workspace_bytes >= plan.workspace_bytes && aligned(A_scale, 16) && aligned(B_scale, 16))
    return gemm_mxfp4_split(A, A_scale, B, B_scale, C, M, N, K, workspace, workspace_bytes, plan, hip_stream);
  return ave_fp4_gemm_mxfp4_ex(A, A_scale, B, B_scale, C, M, N, K, hip_stream, AVE_FP4_AUTO);
}

int ave_fp4_gemm_mxfp4_noalloc(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B, const uint8_t* B_scale,
                               uint16_t* C, int M, int N, int K, void* hip_stream) {
  g_err[0] = 0;
  if (int rc = check_common(A, A_scale, B, B_scale, C, M, N, K, 32, 16)) return rc;
  if (M == 0 || N == 0) return 0;
  // the best split whose partial sums fit the scratch (for nearly every shape the plan of ave_fp4_gemm_mxfp4_ws; a few
  // hundred rows against a K of 30000 and more would want up to twice the scratch and get fewer, longer slices here)
  const ave::SplitPlan plan = ave::mx_tile_split_plan(M, N, K, (size_t)AVE_FP4_NOALLOC_SCRATCH_BYTES);
  if (plan.slices > 1 && aligned(A_scale, 16) && aligned(B_scale, 16)) {
    hipError_t e;
    void* scratch = scratch_pointer(&e);
    if (!scratch) return finish(e, "address of the library's scratch buffer");
    return gemm_mxfp4_split(A, A_scale, B, B_scale, C, M, N, K, scratch, plan.workspace_bytes, plan, hip_stream);
  }
  return ave_fp4_gemm_mxfp4_ex(A, A_scale, B, B_scale, C, M, N, K, hip_stream, AVE_FP4_AUTO);
}

int ave_fp4_debug_gemm_mxfp4_splitk(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B, const uint8_t* B_scale,
                                    uint16_t* C, int M, int N, int K, void* workspace, size_t workspace_bytes,
                                    int slice_pairs, int narrow_tiles, void* hip_stream) {
  g_err[0] = 0;
  if (int rc = check_common(A, A_scale, B, B_scale, C, M, N, K, 32, 16)) return rc;
  if (M == 0 || N == 0) return 0;
  if (K % 512 != 0 || !aligned(A_scale, 16) || !aligned(B_scale, 16))
    return fail_inval("split K needs K %% 512 == 0 and 16-byte aligned scale tensors (K = %d).", K);
  if ((uint64_t)M * (uint64_t)(K / 2) >= (1ull << 32) || (uint64_t)N * (uint64_t)(K / 2) >= (1ull << 32))
    return fail_inval("operand too large for the tile kernel (M=%d N=%d K=%d).", M, N, K);
  const int pairs = K / 512;
  if (slice_pairs <= 0 || slice_pairs > pairs) return fail_inval("slice_pairs must be in 1..%d, got %d.", pairs, slice_pairs);
  ave::SplitPlan plan;
  plan.slice_pairs = slice_pairs;
  plan.slices = (pairs + slice_pairs - 1) / slice_pairs;
  plan.narrow = narrow_tiles != 0;
  plan.half = narrow_tiles == 2;
  plan.workspace_bytes = (size_t)plan.slices * (size_t)M * (size_t)N * sizeof(float);
  if (!workspace || !aligned(workspace, 16) || workspace_bytes < plan.workspace_bytes)
    return fail_inval("workspace must be 16-byte aligned and hold %zu bytes, got %zu.", plan.workspace_bytes, workspace_bytes);
  return gemm_mxfp4_split(A, A_scale, B, B_scale, C, M, N, K, workspace, workspace_bytes, plan, hip_stream);
}

int ave_fp4_gemm_nvfp4_ex(const uint8_t* A, const uint8_t* A_scale, const float* A_global, const uint8_t* B,
                          const uint8_t* B_scale, const float* B_global, uint16_t* C, int M, int N, int K,
                          void* hip_stream, int variant) {
  g_err[0] = 0;
  if (int rc = check_common(A, A_scale, B, B_scale, C, M, N, K, 16, 8)) return rc;
  if (M == 0 || N == 0) return 0;
  if (!A_global || !B_global) return fail_inval("null per-tensor scale pointer.");
  ave::NvArgs p{A, A_scale, A_global, B, B_scale, B_global, C, M, N, K};
  hipStream_t s = static_cast<hipStream_t>(hip_stream);
  switch (variant) {
    case AVE_FP4_AUTO:
      if (ave::nv_decode_supports(p)) return finish(ave::launch_nv_decode(p, s), "nvfp4 decode kernel");
      if (ave::nv_tile_supports(p)) return finish(ave::launch_nv_tile(p, s), "nvfp4 tile kernel");
      // What is left is every other K (a multiple of 16).  The f16-staged kernel converts and multiplies
      // whole 256 x 256 tiles at about 1 us per 64 elements of K whatever the tile holds; the shape-agnostic kernel
      // runs one wave per 32 x 32 block.  Measured crossover (N = 4096 and 28672, K = 320 / 2112 / 4160, 20..300
      // rows): up to about 1500 such blocks the one-wave kernel is faster (300 x 4096 x 2112: 38 against 46 us; 20 x
      // 28672 x 4160: 79 against 86), above it the tile kernel (65 x 28672 x 4160: 90 against 131 us).
      if (ave::nv_f16_tile_supports(p) && ((long)(M + 31) / 32) * ((long)(N + 31) / 32) > 1536)
        return finish(ave::launch_nv_f16_tile(p, s), "nvfp4 f16-staged tile kernel");
      return finish(ave::launch_nv_generic(p, s), "nvfp4 generic kernel");
    case AVE_FP4_TILE_F16:
      if (!ave::nv_f16_tile_supports(p))
        return fail_inval("f16-staged tile kernel does not support M=%d N=%d K=%d (16-byte aligned A and B and 4-byte aligned scales for K %% 64 == 0, 8-byte aligned A and B otherwise).", M, N, K);
      return finish(ave::launch_nv_f16_tile(p, s), "nvfp4 f16-staged tile kernel");
    case AVE_FP4_DECODE:
      if (!ave::nv_decode_supports(p)) return fail_inval("nvfp4 decode kernel does not support M=%d N=%d K=%d.", M, N, K);
      return finish(ave::launch_nv_decode(p, s), "nvfp4 decode kernel");
    case AVE_FP4_GENERIC:
      return finish(ave::launch_nv_generic(p, s), "nvfp4 generic kernel");
    case AVE_FP4_TILE:
      if (!ave::nv_tile_supports(p)) return fail_inval("tile kernel does not support M=%d N=%d K=%d.", M, N, K);
      return finish(ave::launch_nv_tile(p, s), "nvfp4 tile kernel");
    default:
      return fail_inval("unknown kernel variant %d.", variant);
  }
}

size_t ave_fp4_gemm_nvfp4_workspace_bytes(int M, int N, int K) { return ave::nv_tile_split_plan(M, N, K).workspace_bytes; }

int ave_fp4_gemm_nvfp4_ws(const uint8_t* A, const uint8_t* A_scale, const float* A_global, const uint8_t* B,
                          const uint8_t* B_scale, const float* B_global, uint16_t* C, int M, int N, int K, void* workspace,
                          size_t workspace_bytes, void* hip_stream) {
  g_err[0] = 0;
  if (int rc = check_common(A, A_scale, B, B_scale, C, M, N, K, 16, 8)) return rc;
  if (M == 0 || N == 0) return 0;
  if (!A_global || !B_global) return fail_inval("null per-tensor scale pointer.");
  if (workspace_bytes > 0 && !workspace) return fail_inval("null workspace with workspace_bytes = %zu.", workspace_bytes);
  if (workspace && !aligned(workspace, 16)) return fail_inval("workspace must be 16-byte aligned.");
  ave::NvArgs p{A, A_scale, A_global, B, B_scale, B_global, C, M, N, K};
  const ave::SplitPlan plan = ave::nv_tile_split_plan(M, N, K);
  if (plan.slices > 1 && workspace_bytes >= plan.workspace_bytes && ave::nv_tile_supports(p)) {
    p.P = static_cast<float*>(workspace);
    p.slices = plan.slices;
    p.slice_stages = plan.slice_pairs;
    return finish(ave::launch_nv_tile_splitk(p, static_cast<hipStream_t>(hip_stream)), "nvfp4 tile kernel, split K");
  }
  return ave_fp4_gemm_nvfp4_ex(A, A_scale, A_global, B, B_scale, B_global, C, M, N, K, hip_stream, AVE_FP4_AUTO);
}

int ave_fp4_gemm_nvfp4(const uint8_t* A, const uint8_t* A_scale, const float* A_global, const uint8_t* B,
                       const uint8_t* B_scale, const float* B_global, uint16_t* C, int M, int N, int K,
                       void* hip_stream) {
  return ave_fp4_gemm_nvfp4_ex(A, A_scale, A_global, B, B_scale, B_global, C, M, N, K, hip_stream, AVE_FP4_AUTO);
}

static int quantize_common(const void* x, int is_bf16, uint8_t* packed, uint8_t* scales, int rows, int K, int K_padded,
                           void* hip_stream) {
  g_err[0] = 0;
  if (rows < 0) return fail_inval("rows must be non-negative, got %d.", rows);
  if (K <= 0 || K % 32 != 0) return fail_inval("K must be a positive multiple of 32, got %d.", K);
  if (K_padded < K || K_padded % 32 != 0)
    return fail_inval("K_padded must be a multiple of 32 and at least K = %d, got %d.", K, K_padded);
  if (rows == 0) return 0;
  if (!x || !packed || !scales) return fail_inval("null device pointer.");
  if (!aligned(x, 16) || !aligned(packed, 4)) return fail_inval("x must be 16-byte and packed 4-byte aligned.");
  return finish(ave::launch_quantize_mx(x, is_bf16, packed, scales, (size_t)rows, K, K_padded,
                                        static_cast<hipStream_t>(hip_stream)),
                "mxfp4 quantiser");
}

int ave_fp4_quantize_mxfp4_f32(const float* x, uint8_t* packed, uint8_t* scales, int rows, int K, void* hip_stream) {
  return quantize_common(x, 0, packed, scales, rows, K, K, hip_stream);
}

int ave_fp4_quantize_mxfp4_bf16(const uint16_t* x, uint8_t* packed, uint8_t* scales, int rows, int K,
                                void* hip_stream) {
  return quantize_common(x, 1, packed, scales, rows, K, K, hip_stream);
}

int ave_fp4_quantize_mxfp4_f32_padded(const float* x, uint8_t* packed, uint8_t* scales, int rows, int K, int K_padded,
                                      void* hip_stream) {
  return quantize_common(x, 0, packed, scales, rows, K, K_padded, hip_stream);
}

int ave_fp4_quantize_mxfp4_bf16_padded(const uint16_t* x, uint8_t* packed, uint8_t* scales, int rows, int K, int K_padded,
                                       void* hip_stream) {
  return quantize_common(x, 1, packed, scales, rows, K, K_padded, hip_stream);
}

static int quantize_nv_common(const void* x, int is_bf16, const float* global_scale, uint8_t* packed, uint8_t* scales,
                              int rows, int K, void* hip_stream) {
  g_err[0] = 0;
  if (rows < 0) return fail_inval("rows must be non-negative, got %d.", rows);
  if (K <= 0 || K % 16 != 0) return fail_inval("K must be a positive multiple of 16, got %d.", K);
  if (rows == 0) return 0;
  if (!x || !global_scale || !packed || !scales) return fail_inval("null device pointer.");
  if (!aligned(x, 16) || !aligned(packed, 4) || !aligned(global_scale, 4))
    return fail_inval("x must be 16-byte, packed and global_scale 4-byte aligned.");
  return finish(ave::launch_quantize_nv(x, is_bf16, global_scale, packed, scales, (size_t)rows * (size_t)(K / 16),
                                        static_cast<hipStream_t>(hip_stream)),
                "nvfp4 quantiser");
}

int ave_fp4_quantize_nvfp4_f32(const float* x, const float* global_scale, uint8_t* packed, uint8_t* scales, int rows,
                               int K, void* hip_stream) {
  return quantize_nv_common(x, 0, global_scale, packed, scales, rows, K, hip_stream);
}

int ave_fp4_quantize_nvfp4_bf16(const uint16_t* x, const float* global_scale, uint8_t* packed, uint8_t* scales, int rows,
                                int K, void* hip_stream) {
  return quantize_nv_common(x, 1, global_scale, packed, scales, rows, K, hip_stream);
}

int ave_fp4_gemm_mxfp4_swiglu_ex(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B, const uint8_t* B_scale,
                                 uint16_t* C, int M, int N, int K, void* hip_stream, int variant) {
  g_err[0] = 0;
  if (int rc = check_common(A, A_scale, B, B_scale, C, M, N, K, 32, 16)) return rc;
  if (M == 0 || N == 0) return 0;
  if (N > (1 << 30)) return fail_inval("N must not exceed 2^30, got %d.", N);
  ave::MxArgs p{A, A_scale, B, B_scale, C, M, N, K, nullptr, 0, 1};
  hipStream_t s = static_cast<hipStream_t>(hip_stream);
  switch (variant) {
    case AVE_FP4_AUTO:
      // (33..64 rows against a nearly full round of 128-row tiles: the narrow-tile kernel ahead of the rings)
      if (M > 32 && M <= 64 && ave::mx_narrow_preferred(p)) return finish(ave::launch_mx_narrow(p, s), "mxfp4 swiglu narrow-tile kernel");
      if (ave::mx_decode_swiglu_supports(p)) return finish(ave::launch_mx_decode(p, s), "mxfp4 swiglu decode kernel");
      if (ave::mx_narrow_preferred(p)) return finish(ave::launch_mx_narrow(p, s), "mxfp4 swiglu narrow-tile kernel");
      if (ave::mx_tile_supports(p)) {
        p.touch = weights_likely_from_hbm(B, 2 * (size_t)N * (size_t)(K / 2 + K / 32)) ? 1 : 0;
        return finish(ave::launch_mx_tile(p, s), "mxfp4 swiglu tile kernel");
      }
      return finish(ave::launch_mx_generic(p, s), "mxfp4 swiglu generic kernel");
    case AVE_FP4_GENERIC:
      return finish(ave::launch_mx_generic(p, s), "mxfp4 swiglu generic kernel");
    case AVE_FP4_TILE:
    case AVE_FP4_TILE_STREAMED:
      p.touch = variant == AVE_FP4_TILE_STREAMED ? 1 : 0;
      if (!ave::mx_tile_supports(p))
        return fail_inval("swiglu tile kernel does not support M=%d N=%d K=%d (K a multiple of 32 from 512 up; K %% 512 == 0 wants 16-byte aligned scales).", M, N, K);
      return finish(ave::launch_mx_tile(p, s), "mxfp4 swiglu tile kernel");
    case AVE_FP4_DECODE:
      if (!ave::mx_decode_swiglu_supports(p))
        return fail_inval("swiglu decode kernel does not support M=%d N=%d K=%d.", M, N, K);
      return finish(ave::launch_mx_decode(p, s), "mxfp4 swiglu decode kernel");
    case AVE_FP4_NARROW:
      if (!ave::mx_narrow_supports(p))
        return fail_inval("swiglu narrow-tile kernel does not support M=%d N=%d K=%d (K a multiple of 32 from 512 up, 16-byte aligned scales).", M, N, K);
      return finish(ave::launch_mx_narrow(p, s), "mxfp4 swiglu narrow-tile kernel");
    default:
      return fail_inval("unknown or unsupported kernel variant %d.", variant);
  }
}

int ave_fp4_gemm_mxfp4_swiglu_quant(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B, const uint8_t* B_scale,
                                    uint8_t* Q, uint8_t* Q_scale, int M, int N, int K, void* hip_stream) {
  return ave_fp4_gemm_mxfp4_swiglu_quant_padded(A, A_scale, B, B_scale, Q, Q_scale, M, N, N, K, hip_stream);
}

int ave_fp4_gemm_mxfp4_swiglu_quant_padded(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B,
                                           const uint8_t* B_scale, uint8_t* Q, uint8_t* Q_scale, int M, int N,
                                           int N_padded, int K, void* hip_stream) {
  g_err[0] = 0;
  // Q stands in for C in the common checks (non-null, 2-byte aligned is implied by the 16 bytes asked below)
  if (int rc = check_common(A, A_scale, B, B_scale, Q, M, N, K, 32, 16)) return rc;
  if (M == 0 || N == 0) return 0;
  if (N > (1 << 30)) return fail_inval("N must not exceed 2^30, got %d.", N);
  if (N % 32 != 0) return fail_inval("N must be a multiple of 32 (whole scale blocks per row), got %d.", N);
  if (!Q_scale) return fail_inval("null device pointer.");
  if (!aligned(Q, 16)) return fail_inval("Q must be 16-byte aligned.");
  if (N_padded < N || N_padded % 32 != 0)
    return fail_inval("N_padded must be a multiple of 32 and at least N = %d, got %d.", N, N_padded);
  ave::MxArgs p{A, A_scale, B, B_scale, nullptr, M, N, K, nullptr, 0, 1, Q, Q_scale};
  p.q_n = N_padded;
  if (ave::mx_decode_swiglu_quant_supports(p))
    return finish(ave::launch_mx_decode(p, static_cast<hipStream_t>(hip_stream)), "mxfp4 swiglu + quantise decode kernel");
  if (ave::mx_narrow_preferred(p))
    return finish(ave::launch_mx_narrow(p, static_cast<hipStream_t>(hip_stream)), "mxfp4 swiglu + quantise narrow-tile kernel");
  if (!ave::mx_tile_supports(p))
    return fail_inval("the fused SwiGLU + quantiser runs on the LDS-staged kernels only: K %% 512 == 0 with 16-byte aligned "
                      "scale tensors, or another multiple of 32 from 512 up with 16-byte aligned A and B (got M=%d N=%d K=%d).", M, N, K);
  p.touch = weights_likely_from_hbm(B, 2 * (size_t)N * (size_t)(K / 2 + K / 32)) ? 1 : 0;
  return finish(ave::launch_mx_tile(p, static_cast<hipStream_t>(hip_stream)), "mxfp4 swiglu + quantise tile kernel");
}

int ave_fp4_gemm_mxfp4_swiglu(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B, const uint8_t* B_scale,
                              uint16_t* C, int M, int N, int K, void* hip_stream) {
  return ave_fp4_gemm_mxfp4_swiglu_ex(A, A_scale, B, B_scale, C, M, N, K, hip_stream, AVE_FP4_AUTO);
}

static int scale_layout_common(const uint8_t* src, uint8_t* dst, int rows, int cols, bool to_blocked, void* hip_stream) {
  g_err[0] = 0;
  if (rows < 0) return fail_inval("rows must be non-negative, got %d.", rows);
  if (cols < 0) return fail_inval("cols must be non-negative, got %d.", cols);
  if (rows == 0 || cols == 0) return 0;
  if (!src || !dst) return fail_inval("null device pointer.");
  if (!aligned(to_blocked ? dst : src, 4)) return fail_inval("the blocked tensor must be 4-byte aligned.");
  return finish(ave::launch_scale_layout(src, dst, rows, cols, to_blocked, static_cast<hipStream_t>(hip_stream)),
                "scale layout kernel");
}

int ave_fp4_scales_to_blocked(const uint8_t* scales, int rows, int cols, uint8_t* blocked, void* hip_stream) {
  return scale_layout_common(scales, blocked, rows, cols, true, hip_stream);
}

int ave_fp4_scales_from_blocked(const uint8_t* blocked, int rows, int cols, uint8_t* scales, void* hip_stream) {
  return scale_layout_common(blocked, scales, rows, cols, false, hip_stream);
}

namespace {
int route_common(const float* logits, int tokens, int E, int32_t* token_of_row, int32_t* row_offsets, float* row_weight,
                 int32_t* rows_of_token, void* hip_stream) {
  g_err[0] = 0;
  if (tokens < 0) return fail_inval("tokens must be non-negative, got %d.", tokens);
  if (E < 2 || E > ave::route_top2_max_experts())
    return fail_inval("E must be between 2 and %d, got %d.", ave::route_top2_max_experts(), E);
  if (tokens > (1 << 29)) return fail_inval("tokens must not exceed 2^29, got %d.", tokens);
  if (!row_offsets) return fail_inval("null row_offsets pointer.");
  if (tokens > 0 && (!logits || !token_of_row)) return fail_inval("null device pointer.");
  if (!aligned(logits, 4) || !aligned(token_of_row, 4) || !aligned(row_offsets, 4) || !aligned(row_weight, 4) ||
      !aligned(rows_of_token, 4))
    return fail_inval("logits, token_of_row, row_offsets, row_weight and rows_of_token must be 4-byte aligned.");
  return finish(ave::launch_route_top2(logits, tokens, E, token_of_row, row_offsets, row_weight, rows_of_token,
                                       static_cast<hipStream_t>(hip_stream)),
                "top-2 routing kernel");
}
}  // namespace

int ave_fp4_moe_route_top2(const float* logits, int tokens, int E, int32_t* token_of_row, int32_t* row_offsets,
                           float* row_weight, void* hip_stream) {
  return route_common(logits, tokens, E, token_of_row, row_offsets, row_weight, nullptr, hip_stream);
}

int ave_fp4_moe_route_top2_ex(const float* logits, int tokens, int E, int32_t* token_of_row, int32_t* row_offsets,
                              float* row_weight, int32_t* rows_of_token, void* hip_stream) {
  return route_common(logits, tokens, E, token_of_row, row_offsets, row_weight, rows_of_token, hip_stream);
}

int ave_fp4_moe_combine_top2(const uint16_t* rows, const int32_t* rows_of_token, const float* row_weight, int tokens,
                             int H, int renormalize, uint16_t* out, void* hip_stream) {
  g_err[0] = 0;
  if (tokens < 0) return fail_inval("tokens must be non-negative, got %d.", tokens);
  if (tokens > (1 << 29)) return fail_inval("tokens must not exceed 2^29, got %d.", tokens);
  if (H <= 0 || H % 8 != 0) return fail_inval("H must be a positive multiple of 8, got %d.", H);
  if (tokens == 0) return 0;
  if (!rows || !rows_of_token || !row_weight || !out) return fail_inval("null device pointer.");
  if (!aligned(rows, 16) || !aligned(out, 16)) return fail_inval("rows and out must be 16-byte aligned.");
  if (!aligned(rows_of_token, 4) || !aligned(row_weight, 4))
    return fail_inval("rows_of_token and row_weight must be 4-byte aligned.");
  return finish(ave::launch_combine_top2(rows, rows_of_token, row_weight, tokens, H, 2 * tokens, renormalize != 0, out,
                                         static_cast<hipStream_t>(hip_stream)),
                "top-2 combine kernel");
}

int ave_fp4_gather_rows_mxfp4(const uint8_t* A, const uint8_t* A_scale, const int32_t* index, int rows, int src_rows,
                              int K, uint8_t* out, uint8_t* out_scale, void* hip_stream) {
  g_err[0] = 0;
  if (rows < 0) return fail_inval("rows must be non-negative, got %d.", rows);
  if (src_rows < 0) return fail_inval("src_rows must be non-negative, got %d.", src_rows);
  if (K <= 0 || K % 32 != 0) return fail_inval("K must be a positive multiple of 32, got %d.", K);
  if (rows == 0) return 0;
  if (!index || !out || !out_scale || (src_rows > 0 && (!A || !A_scale))) return fail_inval("null device pointer.");
  if (!aligned(A, 16) || !aligned(out, 16)) return fail_inval("A and out must be 16-byte aligned.");
  if (!aligned(index, 4)) return fail_inval("index must be 4-byte aligned.");
  return finish(ave::launch_gather_rows(A, A_scale, index, rows, src_rows, K, out, out_scale,
                                        static_cast<hipStream_t>(hip_stream)),
                "row gather kernel");
}

int ave_fp4_grouped_gemm_mxfp4_ex(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B,
                                  const uint8_t* B_scale, const int32_t* row_offsets, uint16_t* C, int total_M,
                                  int E, int N, int K, void* hip_stream, int variant) {
  g_err[0] = 0;
  if (E <= 0) return fail_inval("E must be positive, got %d.", E);
  if (int rc = check_common(A, A_scale, B, B_scale, C, total_M, N, K, 32, 16)) return rc;
  if (total_M == 0 || N == 0) return 0;
  if (!row_offsets) return fail_inval("null row_offsets pointer.");
  ave::MxArgs p{A, A_scale, B, B_scale, C, total_M, N, K, row_offsets, E};
  hipStream_t s = static_cast<hipStream_t>(hip_stream);
  switch (variant) {
    case AVE_FP4_AUTO:
      if (ave::mx_narrow_preferred(p)) return finish(ave::launch_mx_narrow(p, s), "grouped mxfp4 narrow-tile kernel");
      if (ave::mx_tile_supports(p)) return finish(ave::launch_mx_tile(p, s), "grouped mxfp4 tile kernel");
      return finish(ave::launch_mx_generic(p, s), "grouped mxfp4 generic kernel");
    case AVE_FP4_NARROW:
      if (!ave::mx_narrow_supports(p))
        return fail_inval("narrow-tile kernel does not support total_M=%d N=%d K=%d.", total_M, N, K);
      return finish(ave::launch_mx_narrow(p, s), "grouped mxfp4 narrow-tile kernel");
    case AVE_FP4_GENERIC:
      return finish(ave::launch_mx_generic(p, s), "grouped mxfp4 generic kernel");
    case AVE_FP4_TILE:
      if (!ave::mx_tile_supports(p))
        return fail_inval("tile kernel does not support total_M=%d N=%d K=%d.", total_M, N, K);
      return finish(ave::launch_mx_tile(p, s), "grouped mxfp4 tile kernel");
    default:
      return fail_inval("unknown kernel variant %d.", variant);
  }
}

int ave_fp4_grouped_gemm_mxfp4_swiglu(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B,
                                      const uint8_t* B_scale, const int32_t* row_offsets, uint16_t* C, int total_M,
                                      int E, int N, int K, void* hip_stream) {
  g_err[0] = 0;
  if (E <= 0) return fail_inval("E must be positive, got %d.", E);
  if (int rc = check_common(A, A_scale, B, B_scale, C, total_M, N, K, 32, 16)) return rc;
  if (total_M == 0 || N == 0) return 0;
  if (N > (1 << 30)) return fail_inval("N must not exceed 2^30, got %d.", N);
  if (!row_offsets) return fail_inval("null row_offsets pointer.");
  ave::MxArgs p{A, A_scale, B, B_scale, C, total_M, N, K, row_offsets, E, 1};
  hipStream_t s = static_cast<hipStream_t>(hip_stream);
  if (ave::mx_narrow_preferred(p)) return finish(ave::launch_mx_narrow(p, s), "grouped mxfp4 swiglu narrow-tile kernel");
  if (ave::mx_tile_supports(p)) return finish(ave::launch_mx_tile(p, s), "grouped mxfp4 swiglu tile kernel");
  return finish(ave::launch_mx_generic(p, s), "grouped mxfp4 swiglu generic kernel");
}

int ave_fp4_grouped_gemm_mxfp4_swiglu_quant(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B,
                                            const uint8_t* B_scale, const int32_t* row_offsets, uint8_t* Q,
                                            uint8_t* Q_scale, int total_M, int E, int N, int K, void* hip_stream) {
  return ave_fp4_grouped_gemm_mxfp4_swiglu_quant_padded(A, A_scale, B, B_scale, row_offsets, Q, Q_scale, total_M, E, N, N,
                                                        K, hip_stream);
}

int ave_fp4_grouped_gemm_mxfp4_swiglu_quant_padded(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B,
                                                   const uint8_t* B_scale, const int32_t* row_offsets, uint8_t* Q,
                                                   uint8_t* Q_scale, int total_M, int E, int N, int N_padded, int K,
                                                   void* hip_stream) {
  g_err[0] = 0;
  if (E <= 0) return fail_inval("E must be positive, got %d.", E);
  if (int rc = check_common(A, A_scale, B, B_scale, Q, total_M, N, K, 32, 16)) return rc;
  if (total_M == 0 || N == 0) return 0;
  if (N > (1 << 30)) return fail_inval("N must not exceed 2^30, got %d.", N);
  if (N % 32 != 0) return fail_inval("N must be a multiple of 32 (whole scale blocks per row), got %d.", N);
  if (!row_offsets) return fail_inval("null row_offsets pointer.");
  if (!Q_scale) return fail_inval("null device pointer.");
  if (!aligned(Q, 16)) return fail_inval("Q must be 16-byte aligned.");
  if (N_padded < N || N_padded % 32 != 0)
    return fail_inval("N_padded must be a multiple of 32 and at least N = %d, got %d.", N, N_padded);
  ave::MxArgs p{A, A_scale, B, B_scale, nullptr, total_M, N, K, row_offsets, E, 1, Q, Q_scale};
  p.q_n = N_padded;
  if (ave::mx_narrow_preferred(p))
    return finish(ave::launch_mx_narrow(p, static_cast<hipStream_t>(hip_stream)), "grouped mxfp4 swiglu + quantise narrow-tile kernel");
  if (!ave::mx_tile_supports(p))
    return fail_inval("the fused SwiGLU + quantiser runs on the LDS-staged kernels only: K %% 512 == 0 with 16-byte aligned "
                      "scale tensors, or another multiple of 32 from 512 up with 16-byte aligned A and B (got total_M=%d N=%d K=%d).", total_M, N, K);
  return finish(ave::launch_mx_tile(p, static_cast<hipStream_t>(hip_stream)), "grouped mxfp4 swiglu + quantise tile kernel");
}

int ave_fp4_grouped_gemm_mxfp4(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B, const uint8_t* B_scale,
                               const int32_t* row_offsets, uint16_t* C, int total_M, int E, int N, int K,
                               void* hip_stream) {
  return ave_fp4_grouped_gemm_mxfp4_ex(A, A_scale, B, B_scale, row_offsets, C, total_M, E, N, K, hip_stream,
                                       AVE_FP4_AUTO);
}

}  // extern "C"
