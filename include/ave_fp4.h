/*
 * ave_fp4.h -- C ABI of libave_fp4.so: block-scaled FP4 GEMM for AMD MI355X (gfx950).
 *
 * Every entry point computes  C[M,N] (bf16) = A[M,K] . B[N,K]^T  with fp32
 * accumulation and a round-to-nearest-even bf16 store.  All data pointers are
 * DEVICE pointers to row-major contiguous arrays.  Calls enqueue work on the
 * given HIP stream and return immediately; they never synchronise and never
 * allocate, so they may be recorded into a HIP graph.
 *
 * Packed E2M1: two 4-bit codes per byte, LOW nibble = even k.
 *
 * Return value: 0 on success; AVE_FP4_EINVAL (-1) for a rejected argument;
 * otherwise the hipError_t of the failing HIP call.  ave_fp4_last_error()
 * returns the message for the calling thread.
 *
 * Reference interface each entry point stands in for (causalflow-ai/avelang):
 *   host wrapper  python/avelang_kernels/amdgpu_gemm.py:458-494
 *                 (gemm_pipeline_transposed_b: validate, allocate out, launch)
 *   launch path   python/avelang/runtime/jit.py:791-831 and
 *                 python/avelang/backends/amdgpu/driver.py:325-365
 *                 (current stream, raw data pointers, asynchronous, no sync)
 *   error text    python/avelang/backends/amdgpu/driver.py:125-138
 * The reference has only a bf16 kernel; the FP4 signatures below extend its
 * (A, B, out) convention with the block-scale tensors.
 */
#ifndef AVE_FP4_H_
#define AVE_FP4_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AVE_FP4_EINVAL (-1)

/* Kernel selection for the *_ex entry points (testing and benchmarking). */
enum ave_fp4_variant {
  AVE_FP4_AUTO = 0,    /* shape-based dispatch, what the plain entry points use */
  AVE_FP4_GENERIC = 1, /* one wave per 32x32 tile, no LDS; any shape */
  AVE_FP4_TILE = 2,    /* 256x256 LDS-staged MFMA kernel; MXFP4: K % 256 == 0, or any multiple of 32 from 512 up with
                          16-byte aligned A and B (512 * n is fastest); NVFP4: K % 256 == 0 */
  AVE_FP4_DECODE = 3,  /* weight-streaming small-M kernel; MXFP4: M <= 64 and K a multiple of 32 from 512 up (16-byte
                          aligned operands), or M <= 16 and
                          K % 128 == 0 (K % 32 == 0 for up to 16 MB of weights);
                          NVFP4: M <= 64 and K % 128 == 0, or M <= 32 and K a multiple of 32 from 512 up, or
                          M <= 64 and K a multiple of 32 from 1024 up with an even number of whole 512-element units */
  AVE_FP4_NARROW = 4,  /* MXFP4 only: 256x128 tiles, three stage buffers; needs K a multiple of 32 from 512 up and 16-byte aligned scale
                          tensors; shape-based dispatch takes it for more than 64 rows when its tiles fit the compute units,
                          and for 33..64 rows against a nearly full round of 128-row tiles (N around 28672..32768 on 256
                          compute units) */
  AVE_FP4_TILE_F16 = 5, /* NVFP4 only: 256x256 tiles whose operands are dequantised to f16 once per workgroup on their way
                          into LDS, in steps of 64 elements of K; any K (a multiple of 16: a last step of 16, 32 or 48
                          elements is staged with zeros behind it).  Shape-based dispatch takes it for K % 256 != 0,
                          where AVE_FP4_TILE cannot run (for K % 256 == 0 AVE_FP4_TILE is faster), when C holds more
                          than 1536 blocks of 32 x 32 (below that AVE_FP4_GENERIC is the faster one) */
  AVE_FP4_TILE_STREAMED = 6 /* MXFP4 plain GEMM only: AVE_FP4_TILE with look-ahead touches -- eight K stages before a
                          tile's end the workgroups request the weight panels of their next tiles, so that weights
                          which come from HBM (a model's layers, each with weights of its own) are in the last-level
                          cache when their stage loads ask for them; takes effect with K % 512 == 0, 16-byte aligned
                          scale tensors and more 256 x 256 tiles than compute units, and is AVE_FP4_TILE otherwise.
                          Same bits as AVE_FP4_TILE; on 8192 x 14336 x 4096 7 % faster on weights from HBM, 1 %
                          slower on cache-resident ones.  Also for the fused SwiGLU forms.  Shape-based dispatch keeps,
                          per device, the weight tensors of its latest MXFP4 GEMMs: weights found among the most
                          recent ones that add up to 192 MB at most are taken to be in the 256 MB last-level cache
                          (one GEMM replayed on the same operands) and run as AVE_FP4_TILE, all others as this form */
};

/*
 * MXFP4: A [M, K/2] packed E2M1, A_scale [M, K/32] E8M0 bytes (2^(b-127), one per
 * 32 consecutive k); B [N, K/2], B_scale [N, K/32] likewise; C [M, N] bf16.
 * K must be a positive multiple of 32.  Replaces gemm_pipeline_transposed_b
 * (amdgpu_gemm.py:458-494) for MXFP4 operands; the reference's M % 128 / N % 128
 * restriction (amdgpu_gemm.py:471-474) is lifted.
 */
int ave_fp4_gemm_mxfp4(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B, const uint8_t* B_scale,
                       uint16_t* C, int M, int N, int K, void* hip_stream);
int ave_fp4_gemm_mxfp4_ex(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B, const uint8_t* B_scale,
                          uint16_t* C, int M, int N, int K, void* hip_stream, int variant);

/*
 * The same GEMM with a caller-provided device workspace, for shapes with far fewer 256 x 256 output tiles than
 * compute units and a long K (a few hundred rows of activations against a weight matrix with few rows, e.g.
 * 128..2048 x 4096 x 14336): K is cut into slices that run on different compute units, each slice's fp32 sums go
 * to the workspace, and a second kernel adds them in slice order and rounds to bf16 (deterministic; within the
 * same tolerance as the unsplit GEMM but not bit-identical to it, since the fp32 additions associate differently).
 * ave_fp4_gemm_mxfp4_workspace_bytes returns the bytes this takes for a shape on the current device, 0 when K
 * would not be split.  With a smaller (or null) workspace, or scale tensors that are not 16-byte aligned, the call
 * is ave_fp4_gemm_mxfp4.  The workspace must be 16-byte aligned; its contents need no initialisation and are
 * garbage afterwards; calls that may overlap on the device need workspaces of their own.  The library itself never
 * allocates.  No counterpart in the reference, whose gemm_pipeline_transposed_b (amdgpu_gemm.py:458-494) runs one
 * workgroup per output tile over the whole of K.
 */
size_t ave_fp4_gemm_mxfp4_workspace_bytes(int M, int N, int K);
int ave_fp4_gemm_mxfp4_ws(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B, const uint8_t* B_scale,
                          uint16_t* C, int M, int N, int K, void* workspace, size_t workspace_bytes, void* hip_stream);
/*
 * The same GEMM for callers that cannot allocate: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  No counterpart in the reference.  It is ave_fp4_gemm_mxfp4_ws with the partial sums of the K
 * split in a buffer that the library itself holds -- a static device array of AVE_FP4_NOALLOC_SCRATCH_BYTES, one
 * copy per GPU for the life of the process -- instead of a caller's workspace: same kernels and, wherever that split's
 * partial sums fit the scratch (e.g. 512 x 4096 x 14336, which takes exactly the 32 MiB), the same split and bit-identical
 * results.  The call allocates nothing and frees nothing.  The K split is planned under the scratch's size: where
 * ave_fp4_gemm_mxfp4_ws would want more partial sums than the scratch holds (on 256 compute units: a few hundred rows
 * against a K of about 30000 and more, e.g. 640 x 4096 x 32768 with 50 MiB) this call takes the best split that fits --
 * fewer, longer slices, or none -- so every shape the plain entry point accepts is accepted here, and the result then
 * differs from ave_fp4_gemm_mxfp4_ws's in the association of the fp32 sums only (same tolerance);
 * a shape that is not split runs as ave_fp4_gemm_mxfp4.  The scratch needs no initialisation (every partial sum
 * that is read was written by the same call) and keeps the last call's contents.  ALL calls on one GPU share the one
 * array: calls that may overlap on a GPU (different streams, or graphs replayed concurrently) race -- serialise
 * them, or give the others a workspace of their own through ave_fp4_gemm_mxfp4_ws.  The first call on a device looks
 * the array's address up; make it outside stream capture.
 */
#define AVE_FP4_NOALLOC_SCRATCH_BYTES (32u << 20)
int ave_fp4_gemm_mxfp4_noalloc(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B, const uint8_t* B_scale,
                               uint16_t* C, int M, int N, int K, void* hip_stream);
/*
 * MXFP4 gate+up GEMM with the SwiGLU activation fused into the epilogue:
 *   C[m, n] = silu(g) * u,  g = sum_k A[m,k] B[n,k],  u = sum_k A[m,k] B[N+n,k],  silu(x) = x / (1 + exp(-x)),
 * evaluated in fp32 on the fp32 accumulators, then rounded to bf16.  B [2N, K/2] and B_scale
 * [2N, K/32] hold the N gate rows followed by the N up rows; C is [M, N].  M <= 64 with N % 8 == 0
 * and K a multiple of 32 from 512 up runs on the weight-streaming kernel (AVE_FP4_DECODE); larger M with K % 512 == 0 and
 * 16-byte-aligned scale tensors -- or any K that is a multiple of 32 from 512 up with 16-byte aligned A and B --
 * on the LDS-staged kernel (AVE_FP4_TILE: a tile is 256 rows by 128 outputs,
 * its gate and up values meet in LDS as fp32); any other shape on the shape-agnostic kernel (AVE_FP4_GENERIC).  Extends gemm_pipeline_transposed_b
 * (amdgpu_gemm.py:458-494), which has no epilogue beyond the bf16 store (amdgpu_gemm.py:293-329).
 */
int ave_fp4_gemm_mxfp4_swiglu(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B, const uint8_t* B_scale,
                              uint16_t* C, int M, int N, int K, void* hip_stream);
int ave_fp4_gemm_mxfp4_swiglu_ex(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B, const uint8_t* B_scale,
                                 uint16_t* C, int M, int N, int K, void* hip_stream, int variant);

/*
 * The same gate+up GEMM and SwiGLU, with the MXFP4 quantiser of the next GEMM's activations fused behind it:
 * the fp32 result is rounded to bf16 and quantised per 32 consecutive n exactly as ave_fp4_quantize_mxfp4_bf16
 * would quantise the bf16 output of ave_fp4_gemm_mxfp4_swiglu (bit-identical codes and scales), without that
 * output ever being written.  Q [M, N/2] packed E2M1 (16-byte aligned), Q_scale [M, N/32] E8M0; N % 32 == 0.
 * Up to 32 rows run on the weight-streaming kernel (K a multiple of 32 from 512 up, 16-byte aligned operands), everything
 * else on the LDS-staged kernels: K % 512 == 0 with 16-byte-aligned scale tensors, or any other multiple of
 * 32 from 512 up with 16-byte-aligned A and B; else AVE_FP4_EINVAL (use the two calls then).  No counterpart in the reference, whose kernel ends at the bf16 store
 * (amdgpu_gemm.py:293-329).
 */
int ave_fp4_gemm_mxfp4_swiglu_quant(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B, const uint8_t* B_scale,
                                    uint8_t* Q, uint8_t* Q_scale, int M, int N, int K, void* hip_stream);

/*
 * NVFP4: A_scale [M, K/16] and B_scale [N, K/16] are E4M3 bytes (one per 16
 * consecutive k); A_global / B_global point to ONE fp32 each in device memory
 * (per-tensor scale).  C = (A_global * B_global) * sum_k (a*sa)(b*sb).
 * K must be a positive multiple of 16.  Same reference counterpart as above.
 */
int ave_fp4_gemm_nvfp4(const uint8_t* A, const uint8_t* A_scale, const float* A_global, const uint8_t* B,
                       const uint8_t* B_scale, const float* B_global, uint16_t* C, int M, int N, int K,
                       void* hip_stream);
int ave_fp4_gemm_nvfp4_ex(const uint8_t* A, const uint8_t* A_scale, const float* A_global, const uint8_t* B,
                          const uint8_t* B_scale, const float* B_global, uint16_t* C, int M, int N, int K,
                          void* hip_stream, int variant);
/*
 * The NVFP4 GEMM with a caller-provided device workspace, the counterpart of ave_fp4_gemm_mxfp4_ws: for more than 64
 * rows and at most half as many 256 x 256 tiles as compute units, K is cut into slices that run on different
 * compute units (the NVFP4 tile kernel is bound by its fp4 -> f16 conversions, several microseconds per 256
 * elements of K, so few tiles over a long K are slow: 270 us for 128 x 4096 x 14336 unsplit).  Same contract as the
 * MXFP4 form: ave_fp4_gemm_nvfp4_workspace_bytes gives the size (0: no split), a smaller or null workspace makes
 * the call ave_fp4_gemm_nvfp4, the result is deterministic and within the GEMM's tolerance.
 */
size_t ave_fp4_gemm_nvfp4_workspace_bytes(int M, int N, int K);
int ave_fp4_gemm_nvfp4_ws(const uint8_t* A, const uint8_t* A_scale, const float* A_global, const uint8_t* B,
                          const uint8_t* B_scale, const float* B_global, uint16_t* C, int M, int N, int K, void* workspace,
                          size_t workspace_bytes, void* hip_stream);

/*
 * Grouped (MoE) MXFP4: rows row_offsets[e] .. row_offsets[e+1]-1 of A belong to
 * expert e and are multiplied by B[e] ([E, N, K/2], scales [E, N, K/32]).
 * row_offsets is a DEVICE array of E+1 non-decreasing int32 with
 * row_offsets[0] == 0 and row_offsets[E] == total_M; it is read by the kernel,
 * never by the host, so the call stays asynchronous.  One launch covers all
 * experts.  The reference has no grouped GEMM; the calling convention follows
 * amdgpu_gemm.py:458-494.
 */
int ave_fp4_grouped_gemm_mxfp4(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B, const uint8_t* B_scale,
                               const int32_t* row_offsets, uint16_t* C, int total_M, int E, int N, int K,
                               void* hip_stream);
int ave_fp4_grouped_gemm_mxfp4_ex(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B,
                                  const uint8_t* B_scale, const int32_t* row_offsets, uint16_t* C, int total_M,
                                  int E, int N, int K, void* hip_stream, int variant);

/*
 * Grouped gate+up GEMM with SwiGLU (and, in the _quant form, the MXFP4 quantiser of the result) for an MoE expert
 * layer in one launch: rows row_offsets[e] .. row_offsets[e+1]-1 of A use expert e's weights B[e], which hold the N
 * gate rows followed by the N up rows (B [E, 2N, K/2], B_scale [E, 2N, K/32]); C is [total_M, N] bf16, or
 * Q [total_M, N/2] + Q_scale [total_M, N/32] with N % 32 == 0.  Every expert's rows equal what
 * ave_fp4_gemm_mxfp4_swiglu (ave_fp4_gemm_mxfp4_swiglu_quant) gives for that expert alone, bit for bit on the
 * same kernel.  K % 512 == 0 with 16-byte-aligned scale tensors, or another multiple of 32 from 512 up with
 * 16-byte-aligned A and B, takes the LDS-staged kernel; other K the shape-agnostic one (the _quant form then returns
 * AVE_FP4_EINVAL).  No counterpart in the reference.
 */
int ave_fp4_grouped_gemm_mxfp4_swiglu(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B,
                                      const uint8_t* B_scale, const int32_t* row_offsets, uint16_t* C, int total_M,
                                      int E, int N, int K, void* hip_stream);
int ave_fp4_grouped_gemm_mxfp4_swiglu_quant(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B,
                                            const uint8_t* B_scale, const int32_t* row_offsets, uint8_t* Q,
                                            uint8_t* Q_scale, int total_M, int E, int N, int K, void* hip_stream);

/*
 * MXFP4 quantiser: x [rows, K] row-major fp32 (ave_fp4_quantize_mxfp4_f32) or bf16 bit patterns
 * (..._bf16) -> packed [rows, K/2] E2M1 codes and scales [rows, K/32] E8M0 bytes, in the layout the
 * GEMM entry points take.  Per 32 consecutive k: scale 2^(floor(log2(amax)) - 2) (exponent clamped to
 * [-127, 127]; an all-zero block gets byte 127), elements divided by it and rounded to nearest-even
 * onto the E2M1 grid, saturating.  K % 32 == 0, x 16-byte aligned, packed 4-byte aligned.  Inputs
 * must be finite.  No counterpart in the reference (its benchmark feeds bf16 tensors directly,
 * benchmark/gemm/bench_amdgpu_gemm.py:27-29); this is the producer of the GEMM's operands.
 */
int ave_fp4_quantize_mxfp4_f32(const float* x, uint8_t* packed, uint8_t* scales, int rows, int K, void* hip_stream);
int ave_fp4_quantize_mxfp4_bf16(const uint16_t* x, uint8_t* packed, uint8_t* scales, int rows, int K,
                                void* hip_stream);

/*
 * Operands padded along K.  The LDS-staged kernels move whole 128-byte cache lines and whole 512-element units of K:
 * a K whose packed rows (K/2 bytes) are no multiple of 128 bytes costs their main loop about a quarter more per stage
 * (every 128-byte piece of a row then lies in two cache lines), and K % 512 != 0 adds a tail.  Operands whose rows are
 * padded with ZERO BLOCKS (zero codes, any finite scale byte) up to a multiple of 512 give the same sums -- a zero
 * code contributes exactly +0 whatever its scale -- at the speed of the padded length (measured: 8192 x 2880 x 2880
 * 66.7 us as it is, 57.5 us padded to 3072; 8192 x 14336 x 4128 305 us, 264 us padded to 4608).  Weights are padded once,
 * offline; these entry points produce padded activations without a copy:
 *   ave_fp4_quantize_mxfp4_{f32,bf16}_padded: x [rows, K] -> packed [rows, K_padded/2], scales [rows, K_padded/32];
 *     columns K .. K_padded-1 are written as zero codes under the scale byte 127.  K_padded >= K, both multiples of 32;
 *     K_padded == K is the plain quantiser.
 *   ave_fp4_gemm_mxfp4_swiglu_quant_padded / ave_fp4_grouped_gemm_mxfp4_swiglu_quant_padded (declared here, described
 *     with their unpadded forms above): Q [M, N_padded/2], Q_scale [M, N_padded/32]; columns N .. N_padded-1 of both are
 *     NOT written -- fill the two buffers with zero bytes once (code 0 under scale byte 0 = 2^-127 is a zero block).
 * The consumer is then called with K = K_padded (N_padded).  No counterpart in the reference, which takes K % 64 == 0
 * only (amdgpu_gemm.py:475-476).
 */
int ave_fp4_quantize_mxfp4_f32_padded(const float* x, uint8_t* packed, uint8_t* scales, int rows, int K, int K_padded,
                                      void* hip_stream);
int ave_fp4_quantize_mxfp4_bf16_padded(const uint16_t* x, uint8_t* packed, uint8_t* scales, int rows, int K, int K_padded,
                                       void* hip_stream);
int ave_fp4_gemm_mxfp4_swiglu_quant_padded(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B,
                                           const uint8_t* B_scale, uint8_t* Q, uint8_t* Q_scale, int M, int N,
                                           int N_padded, int K, void* hip_stream);
int ave_fp4_grouped_gemm_mxfp4_swiglu_quant_padded(const uint8_t* A, const uint8_t* A_scale, const uint8_t* B,
                                                   const uint8_t* B_scale, const int32_t* row_offsets, uint8_t* Q,
                                                   uint8_t* Q_scale, int total_M, int E, int N, int N_padded, int K,
                                                   void* hip_stream);

/*
 * NVFP4 quantiser for a per-tensor scale the caller supplies: x [rows, K] row-major fp32 or bf16 bit patterns,
 * global_scale a device pointer to one positive fp32 g (calibrated ahead of time; amax / (448 * 6) uses the whole
 * range) -> packed [rows, K/2] E2M1 codes and scales [rows, K/16] E4M3 bytes, in the layout ave_fp4_gemm_nvfp4
 * takes together with the same g.  Per 16 consecutive k, each step one IEEE fp32 operation:
 * u = min((amax / 6) / g, 448); scale byte = E4M3(u), round to nearest even; d = decode(scale byte) * g;
 * codes = E2M1(x / d), round to nearest even, saturating (d == 0: zero codes).  K % 16 == 0, x 16-byte aligned,
 * packed 4-byte aligned.  Inputs must be finite.  No counterpart in the reference (see ave_fp4_quantize_mxfp4_f32).
 */
int ave_fp4_quantize_nvfp4_f32(const float* x, const float* global_scale, uint8_t* packed, uint8_t* scales, int rows,
                               int K, void* hip_stream);
int ave_fp4_quantize_nvfp4_bf16(const uint16_t* x, const float* global_scale, uint8_t* packed, uint8_t* scales, int rows,
                                int K, void* hip_stream);

/*
 * MoE routing in front of the grouped GEMM.  logits [tokens, E] fp32 router scores (finite).  Every
 * token is routed to its two highest-scoring experts (equal scores: the lower expert index ranks
 * first).  The 2*tokens routed rows are ordered by expert, inside an expert by token and then by rank
 * (a stable sort of the row-major [tokens, 2] choice table by expert):
 *   token_of_row [2*tokens] int32   token whose activations routed row i carries,
 *   row_offsets  [E+1]      int32   first routed row of every expert (the grouped GEMM's row_offsets),
 *   row_weight   [2*tokens] fp32    softmax(logits[token])[expert] of routed row i; may be NULL.
 * 2 <= E <= 256, tokens <= 2^29.  No counterpart in the reference, which has no MoE
 * code; it exists so that routing, gather and grouped GEMM can be recorded into one graph.
 */
int ave_fp4_moe_route_top2(const float* logits, int tokens, int E, int32_t* token_of_row, int32_t* row_offsets,
                           float* row_weight, void* hip_stream);

/*
 * The same routing, with one more output: rows_of_token [tokens, 2] int32, the routed row of every token's first
 * and second choice (the inverse of token_of_row; may be null), which ave_fp4_moe_combine_top2 reads.
 */
int ave_fp4_moe_route_top2_ex(const float* logits, int tokens, int E, int32_t* token_of_row, int32_t* row_offsets,
                              float* row_weight, int32_t* rows_of_token, void* hip_stream);

/*
 * The step behind the expert GEMMs: out[t, :] = w0 * rows[r0, :] + w1 * rows[r1, :] with (r0, r1) =
 * rows_of_token[t], w = row_weight of those rows, divided by w0 + w1 when `renormalize` is non-zero.  rows
 * [2*tokens, H] bf16 (the down projection's output in routed order), out [tokens, H] bf16, both 16-byte aligned;
 * H % 8 == 0.  The two products and the sum are single IEEE fp32 operations, then one rounding to bf16; a row
 * index outside [0, 2*tokens) contributes zeros.  No counterpart in the reference.
 */
int ave_fp4_moe_combine_top2(const uint16_t* rows, const int32_t* rows_of_token, const float* row_weight, int tokens,
                             int H, int renormalize, uint16_t* out, void* hip_stream);

/*
 * Row gather of an MXFP4 operand: out[i] = A[index[i]], out_scale[i] = A_scale[index[i]] for
 * i < rows; A [src_rows, K/2], A_scale [src_rows, K/32], index [rows] int32.  An index outside
 * [0, src_rows) produces a row of zero bytes.  K % 32 == 0; A and out 16-byte aligned.  No
 * counterpart in the reference; it builds the grouped GEMM's A operand from token_of_row.
 */
int ave_fp4_gather_rows_mxfp4(const uint8_t* A, const uint8_t* A_scale, const int32_t* index, int rows, int src_rows,
                              int K, uint8_t* out, uint8_t* out_scale, void* hip_stream);

/*
 * Scale-layout adapters.  The GEMM entry points take block scales row-major, [rows, cols] bytes
 * (cols = K/32 for MXFP4, K/16 for NVFP4).  Other FP4 stacks keep them "blocked": padded to
 * multiples of 128 rows and 4 columns, cut into 128 x 4 tiles of 512 bytes stored in row-major tile
 * order, scale (r, c) of a tile at byte (r % 32) * 16 + (r / 32) * 4 + c.  The blocked tensor holds
 * ceil(rows/128)*128 * ceil(cols/4)*4 bytes and must be 4-byte aligned; to_blocked writes its
 * padding as zero, from_blocked ignores it.  No counterpart in the reference, whose kernel takes
 * no scales.
 */
int ave_fp4_scales_to_blocked(const uint8_t* scales, int rows, int cols, uint8_t* blocked, void* hip_stream);
int ave_fp4_scales_from_blocked(const uint8_t* blocked, int rows, int cols, uint8_t* scales, void* hip_stream);

/*
 * The MXFP4 GEMM on scale tensors that are ALREADY in the blocked layout above -- A_scale_blocked for [M, K/32],
 * B_scale_blocked for [N, K/32], each ceil(rows/128)*128 * K/32 bytes, 16-byte aligned -- read by the kernels as they
 * are: no conversion launch, no workspace.  K % 512 == 0 (then K/32 is a multiple of 4 and the tensors have no column
 * padding).  Up to 64 rows run on the weight-streaming kernel, which gathers a K step's four scale bytes per row as one
 * dword of a 512-byte tile; more rows on the 256 x 256 LDS-staged kernel, which copies the four column tiles of a pair of
 * K stages as whole kilobytes.  Same arithmetic in the same order as ave_fp4_gemm_mxfp4_ex with AVE_FP4_DECODE /
 * AVE_FP4_TILE on row-major scales: bit-identical results.  Other K: AVE_FP4_EINVAL (convert with
 * ave_fp4_scales_from_blocked).  The reference's entry takes its operands as its caller has them
 * (amdgpu_gemm.py:458-462); this is that for callers whose quantiser emits blocked scales.
 */
int ave_fp4_gemm_mxfp4_blocked_scales(const uint8_t* A, const uint8_t* A_scale_blocked, const uint8_t* B,
                                      const uint8_t* B_scale_blocked, uint16_t* C, int M, int N, int K, void* hip_stream);

/* Message of the last failure on the calling thread ("" if none). */
const char* ave_fp4_last_error(void);

/* Library ABI version (bumped when a signature changes). */
int ave_fp4_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* AVE_FP4_H_ */
