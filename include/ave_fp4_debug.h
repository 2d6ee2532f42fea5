/*
 * ave_fp4_debug.h -- diagnostics of libave_fp4.so: test hooks and measurement probes.
 *
 * These symbols live in the same library as the entry points of ave_fp4.h but are no part of the product ABI: a
 * binding for callers of the GEMM needs ave_fp4.h alone.  They exist for the library's own tests (the host-side
 * arithmetic of the tile map, the grouped tile lookup, the split planner and the launch grids, which the device code
 * shares) and for its benchmark (matrix-core and streaming-read probes that put a measured ceiling beside a kernel's
 * figure).  None has a counterpart in the reference (causalflow-ai/avelang), which reports no roofline and has neither
 * a grouped GEMM nor a K split; the one reference function a hook mirrors is named at that hook.
 */
#ifndef AVE_FP4_DEBUG_H_
#define AVE_FP4_DEBUG_H_

#include "ave_fp4.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Host-only diagnostic: how ave_fp4_gemm_mxfp4_ws would cut K for a shape on a device with compute_units compute
 * units: slices (1: no split), pairs of 256-element stages per slice, the tiles the slices run on (0: 256 x 256,
 * 1: 256 x 128, 2: 128 x 128), and the workspace bytes (slices * M * N * 4, or 0). */
int ave_fp4_debug_split_plan(int M, int N, int K, int compute_units, int* slices, int* slice_pairs, int* narrow_tiles,
                             size_t* workspace_bytes);
/* Diagnostic and test hook: split K into slices of slice_pairs x 512 elements whatever the shape (K % 512 == 0,
 * 16-byte aligned scale tensors), on 256 x 256 tiles (narrow_tiles = 0) or on the 256 x 128 (1) or 128 x 128 (2)
 * tiles of AVE_FP4_NARROW; the workspace must hold ceil(K / 512 / slice_pairs) * M * N * 4 bytes. */
int ave_fp4_debug_gemm_mxfp4_splitk(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B, const uint8_t* B_scale,
                                    uint16_t* C, int M, int N, int K, void* workspace, size_t workspace_bytes,
                                    int slice_pairs, int narrow_tiles, void* hip_stream);
/* The same plan when the partial sums may take at most max_workspace_bytes: the best split that fits, or none.  This is
 * what ave_fp4_gemm_mxfp4_noalloc runs with max_workspace_bytes = AVE_FP4_NOALLOC_SCRATCH_BYTES. */
int ave_fp4_debug_split_plan_capped(int M, int N, int K, int compute_units, size_t max_workspace_bytes, int* slices,
                                    int* slice_pairs, int* narrow_tiles, size_t* workspace_bytes);

/*
 * Diagnostic, host only (no GPU needed): the output tile (tm, tn) that workgroup `pid` of the
 * LDS-staged kernels works on when the grid has m_tiles x n_tiles tiles.  The map undoes the
 * round-robin of workgroup ids over the 8 XCDs (one band of 4 m-tiles per XCD at a time); it plays the role
 * of the reference's _wgm_mapping (python/avelang_kernels/amdgpu_gemm.py:43-90) and must be a
 * bijection.  Returns 0, or AVE_FP4_EINVAL for pid outside [0, m_tiles*n_tiles).
 */
int ave_fp4_debug_map_tile(int pid, int m_tiles, int n_tiles, int* tm, int* tn);

/*
 * Diagnostic, host only: how the grouped kernels find m-tile `tm` (tiles of tile_rows rows) in the concatenation of
 * the experts' tile lists -- the function the device code runs, on a HOST copy of row_offsets [E+1].  Table entries
 * are clamped to [0, total_M] and a range that is empty after clamping has no tiles, so that a stale or malformed
 * table can leave rows unwritten but never makes a kernel address rows outside A or C.  Returns 1 and sets expert,
 * m_begin, m_end (0 <= m_begin < m_end <= total_M), 0 when tm lies behind the last tile, AVE_FP4_EINVAL for a
 * rejected argument.  No counterpart in the reference, which has no grouped GEMM.
 */
int ave_fp4_debug_locate_group_tile(const int32_t* row_offsets, int E, int total_M, int tile_rows, int tm, int* expert,
                                    int* m_begin, int* m_end);

/*
 * Diagnostic, host only: workgroups of the shape-agnostic kernels (AVE_FP4_GENERIC) for an M x N problem with E
 * experts (0: plain GEMM) -- ceil(N / 128) * (ceil(M / 32) + E) in one grid dimension, or 0 when that exceeds the
 * 2^31 - 1 a dimension holds (the launch then fails with hipErrorInvalidConfiguration).
 */
int ave_fp4_debug_generic_grid(int M, int N, int E, unsigned* workgroups);

/*
 * Diagnostic: launches `workgroups` workgroups of eight wavefronts that each issue `iters` x 8
 * v_mfma_scale_f32_32x32x64_f8f6f4 on FP4 operand fragments read once from `codes` (device memory, `bytes`
 * >= 16, 16-byte aligned) and writes the floating-point operations of the launch to *flop (host).  The caller
 * times it: the rate is the matrix-core ceiling of this GPU for operands with that bit pattern (the clock
 * under MFMA load depends on the data: zeros run near the published peak, quantised random data well below).
 * `sink` is one device float the kernel practically never writes.  No counterpart in the reference, which
 * reports no roofline; bench.py prints the figure beside the GEMM's.
 */
int ave_fp4_debug_mfma_rate(const uint8_t* codes, size_t bytes, int workgroups, int iters, float* sink,
                            void* hip_stream, double* flop);

/* The same probe with v_mfma_f32_32x32x16_f16 on the codes dequantised to f16 (E2M1 x 1.0): the ceiling of the NVFP4
 * kernels, which multiply as f16, for operands with that bit pattern. */
int ave_fp4_debug_mfma_rate_f16(const uint8_t* codes, size_t bytes, int workgroups, int iters, float* sink,
                                void* hip_stream, double* flop);

/*
 * Diagnostic: `workgroups` workgroups of 256 lanes read `bytes` bytes of device memory (a multiple of 16, 16-byte
 * aligned) once, 16 bytes per lane and trip with four loads in flight, compute nothing and write nothing (`sink`
 * is one device int that is practically never written).  The caller times it: over a buffer larger than the
 * last-level cache this is the rate at which the GPU streams HBM into a kernel that does nothing else -- the floor
 * under the weight-streaming (small M) GEMMs, whose roofline is the published 8 TB/s.  No counterpart in the
 * reference; bench.py prints the figure beside the decode GEMM's (`--only stream_read`).
 */
int ave_fp4_debug_stream_read(const void* src, size_t bytes, int workgroups, int32_t* sink, void* hip_stream);

/* The same read followed by `dst_bytes` (a multiple of 16, 16-byte aligned) of writes, 16 bytes per lane, consecutive
 * lanes consecutive addresses: the floor for a streaming GEMM that also stores a result of that size (a kernel that
 * leaves modified lines in L2 ends later than one that leaves none).  No counterpart in the reference. */
int ave_fp4_debug_stream_read_write(const void* src, size_t bytes, void* dst, size_t dst_bytes, int workgroups,
                                    int32_t* sink, void* hip_stream);

/*
 * Diagnostic, host only: how many tiles (of 16 weight rows, or of 8 outputs with the fused SwiGLU) the weight-streaming
 * kernels give a workgroup for n_tiles tiles on compute_units compute units, at most t_max, a multiple of step -- one
 * round of workgroups when that fits, balanced rounds beyond it.  0 for arguments out of range.
 */
int ave_fp4_debug_tiles_per_workgroup(int n_tiles, int compute_units, int t_max, int step);

/*
 * Diagnostic, host only: the hint that shape-based dispatch of the MXFP4 GEMMs takes before it launches the 256 x 256
 * kernel -- 1 when a weight tensor at address B of `bytes` bytes is expected to come from HBM (the kernel then runs
 * with look-ahead touches, AVE_FP4_TILE_STREAMED), 0 when it is expected in the last-level cache.  The call RECORDS B
 * as the device's most recent weight tensor, exactly as a GEMM call does: the library keeps the last eight per device,
 * most recent first, and takes a tensor to be resident when it is found among the most recent ones whose sizes add up
 * to 192 MB at most.  Nothing is launched and B is not dereferenced.
 */
int ave_fp4_debug_weights_from_hbm(const void* B, size_t bytes);

#ifdef __cplusplus
}
#endif
#endif /* AVE_FP4_DEBUG_H_ */
