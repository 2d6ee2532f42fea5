// The two steps in front of the grouped (MoE) GEMM, on the device so that the whole expert layer can
// be recorded into one HIP graph:
//
//   route_top2_kernel   router logits [T, E] -> for every token its two highest-scoring experts, the
//                       2T routed rows sorted by expert (stable: by token, then by rank) as a list of
//                       token indices, the E+1 row offsets the grouped GEMM reads, and the softmax
//                       probability of every routed row;
//   gather_rows_kernel  packed MXFP4 rows and their scale rows copied into that order;
//   combine_top2_kernel the step behind the expert GEMMs: every token's two expert outputs, weighted with their
//                       routing probabilities, summed back into token order.
//
// Both are integer/byte work.  Routing is a counting sort without any exchange between workgroups:
// workgroup (e, part) scans ALL tokens once (token = iteration*1024 + thread, so loads are coalesced)
// to count the routed rows of experts below e and the rows of e in front of its own token range --
// that is the position of its first row -- and then places the rows of expert e for its range,
// iteration by iteration, with a ballot per wave and a 16-entry prefix over the waves.  Tokens rise
// with (iteration, wave, lane), so the order inside an expert is by token: the stable order.
#include "fp4_common.hpp"
#include "kernels.hpp"

namespace ave {
namespace {

constexpr int kRouteThreads = 1024;

struct Top2 {
  int e0, e1;
  float p0, p1;
};

// Highest and second-highest logit; among equal values the lower expert index ranks first.
// Probabilities are those of the full softmax over the E logits.  The row is read eight values at a
// time with all eight loads in flight together (two 16-byte loads when `vec`: E % 4 == 0 and an
// aligned base), because a one-value-per-trip loop pays the memory latency E times per token.
__device__ inline Top2 top2_of(const float* l, int E, bool vec, bool want_prob) {
  float v0 = -__builtin_inff(), v1 = -__builtin_inff();
  // the softmax denominator is added up in double: a float sum of E terms drifts by about sqrt(E) roundings, which for
  // 200 and more experts is more than the 2e-6 relative error the probabilities are stated to keep
  double sum = 0.0;
  int e0 = -1, e1 = -1;
  for (int c = 0; c < E; c += 8) {
    float x[8];
    if (vec) {
      const v4f lo = *reinterpret_cast<const v4f*>(l + c);
      const v4f hi = c + 4 < E ? *reinterpret_cast<const v4f*>(l + c + 4) : v4f{0, 0, 0, 0};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        x[j] = lo[j];
        x[4 + j] = hi[j];
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) x[j] = c + j < E ? l[c + j] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (c + j < E) {
        const float v = x[j];
        if (e0 < 0 || v > v0) {
          if (want_prob) sum = e0 < 0 ? 1.0 : sum * (double)expf(v0 - v) + 1.0;   // running sum of exp(l - max)
          v1 = v0;
          e1 = e0;
          v0 = v;
          e0 = c + j;
        } else {
          if (want_prob) sum += (double)expf(v - v0);
          if (e1 < 0 || v > v1) {
            v1 = v;
            e1 = c + j;
          }
        }
      }
    }
  }
  Top2 r{e0, e1, 0.f, 0.f};
  if (want_prob) {
    r.p0 = (float)(1.0 / sum);
    r.p1 = (float)((double)expf(v1 - v0) / sum);
  }
  return r;
}

// sum over the workgroup; `buf` holds one int per wave; every thread returns the total
__device__ inline int block_sum(int v, int* buf, int lane, int w) {
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) v += __shfl_xor(v, d, 64);
  __syncthreads();   // earlier readers of buf are done
  if (lane == 0) buf[w] = v;
  __syncthreads();
  int total = 0;
  for (int ww = 0; ww < kRouteThreads / 64; ++ww) total += buf[ww];
  return total;
}

// rows_of_token (optional, [T, 2]): the routed row of every token's first and second choice -- the inverse of
// token_of_row, which the combine step reads.
__global__ __launch_bounds__(kRouteThreads) void route_top2_kernel(const float* logits, int T, int E, int P,
                                                                    int32_t* token_of_row, int32_t* row_offsets,
                                                                    float* row_weight, int32_t* rows_of_token) {
  __shared__ int wave_buf[2][kRouteThreads / 64];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int e = blockIdx.x / P, part = blockIdx.x % P;
  const bool vec = (E & 3) == 0 && (reinterpret_cast<uintptr_t>(logits) & 15) == 0;
  const int iters = (T + kRouteThreads - 1) / kRouteThreads;
  const int per_part = (iters + P - 1) / P;
  const int it0 = part * per_part < iters ? part * per_part : iters;
  const int it1 = it0 + per_part < iters ? it0 + per_part : iters;

  // ---- pass 1: where do this workgroup's rows start? ----------------------------------------
  int below = 0, mine_before = 0, mine_all = 0;
  for (int it = 0; it < iters; ++it) {
    const int t = it * kRouteThreads + tid;
    if (t < T) {
      const Top2 r = top2_of(logits + (size_t)t * E, E, vec, false);
      below += (r.e0 < e) + (r.e1 < e);
      const int hit = (r.e0 == e) | (r.e1 == e);
      mine_all += hit;
      if (it < it0) mine_before += hit;
    }
  }
  below = block_sum(below, wave_buf[0], lane, w);
  mine_before = block_sum(mine_before, wave_buf[0], lane, w);
  mine_all = block_sum(mine_all, wave_buf[0], lane, w);
  if (part == 0 && tid == 0) {
    row_offsets[e + 1] = below + mine_all;
    if (e == 0) row_offsets[0] = 0;
  }
  __syncthreads();

  // ---- pass 2: place the rows of expert e for tokens of iterations [it0, it1) -----------------
  int run = below + mine_before;
  for (int it = it0; it < it1; ++it) {
    const int t = it * kRouteThreads + tid;
    bool hit = false;
    float prob = 0.f;
    int rank = 0;
    if (t < T) {
      const Top2 r = top2_of(logits + (size_t)t * E, E, vec, row_weight != nullptr);
      hit = r.e0 == e || r.e1 == e;
      prob = r.e0 == e ? r.p0 : r.p1;
      rank = r.e0 == e ? 0 : 1;
    }
    const unsigned long long mask = __ballot(hit);
    int* buf = wave_buf[it & 1];   // alternating buffers: one barrier per iteration is enough
    if (lane == 0) buf[w] = __popcll(mask);
    __syncthreads();
    int before = 0, total = 0;
    for (int ww = 0; ww < kRouteThreads / 64; ++ww) {
      const int c = buf[ww];
      before += ww < w ? c : 0;
      total += c;
    }
    if (hit) {
      const int pos = run + before + __popcll(mask & ((1ull << lane) - 1ull));
      token_of_row[pos] = t;
      if (row_weight) row_weight[pos] = prob;
      if (rows_of_token) rows_of_token[2 * (size_t)t + rank] = pos;
    }
    run += total;
  }
}

// dst row i = src row index[i] (data: row_bytes, a multiple of 16; scales: row_scales bytes moved SV at a
// time).  An index outside [0, src_rows) yields a row of zeros.  A thread moves kGatherUnroll pieces
// per trip and issues all their loads (index, then data) before the first store.
constexpr int kGatherUnroll = 4;

template <int SV>
__global__ __launch_bounds__(256) void gather_rows_kernel(const uint8_t* src, const uint8_t* src_s,
                                                          const int32_t* index, int rows, int src_rows,
                                                          unsigned row_bytes, unsigned row_scales, uint8_t* dst,
                                                          uint8_t* dst_s) {
  const unsigned data_units = row_bytes / 16, scale_units = row_scales / SV, units = data_units + scale_units;
  const size_t total = (size_t)rows * units, stride = (size_t)gridDim.x * 256;
  for (size_t i0 = (size_t)blockIdx.x * 256 + threadIdx.x; i0 < total; i0 += stride * kGatherUnroll) {
    unsigned row[kGatherUnroll], u[kGatherUnroll];
    int from[kGatherUnroll];
#pragma unroll
    for (int j = 0; j < kGatherUnroll; ++j) {
      const size_t i = i0 + (size_t)j * stride;
      row[j] = (unsigned)(i / units);
      u[j] = (unsigned)(i % units);
      from[j] = i < total ? index[row[j]] : -1;
    }
    v4i data[kGatherUnroll];
#pragma unroll
    for (int j = 0; j < kGatherUnroll; ++j) {
      const bool ok = from[j] >= 0 && from[j] < src_rows;
      data[j] = v4i{0, 0, 0, 0};
      if (ok) {
        if (u[j] < data_units) {
          data[j] = *reinterpret_cast<const v4i*>(src + (size_t)from[j] * row_bytes + 16 * u[j]);
        } else {
          const uint8_t* s = src_s + (size_t)from[j] * row_scales + (u[j] - data_units) * SV;
          if (SV == 16) data[j] = *reinterpret_cast<const v4i*>(s);
          else if (SV == 4) data[j][0] = *reinterpret_cast<const int*>(s);
          else data[j][0] = *s;
        }
      }
    }
#pragma unroll
    for (int j = 0; j < kGatherUnroll; ++j) {
      if (i0 + (size_t)j * stride < total) {
        if (u[j] < data_units) {
          *reinterpret_cast<v4i*>(dst + (size_t)row[j] * row_bytes + 16 * u[j]) = data[j];
        } else {
          uint8_t* d = dst_s + (size_t)row[j] * row_scales + (u[j] - data_units) * SV;
          if (SV == 16) *reinterpret_cast<v4i*>(d) = data[j];
          else if (SV == 4) *reinterpret_cast<int*>(d) = data[j][0];
          else *d = (uint8_t)data[j][0];
        }
      }
    }
  }
}

// out[t, :] = w0 * rows[r0, :] + w1 * rows[r1, :] with (r0, r1) = rows_of_token[t] and (w0, w1) their routing
// probabilities, divided by their sum when `renormalize`.  bf16 in and out; the two products and the sum are
// single IEEE fp32 operations (no contraction into an fma), so the result does not depend on the compiler and
// equals the same three numpy float32 operations bit for bit.  A thread moves 8 columns (16 bytes) of one token.
__global__ __launch_bounds__(256) void combine_top2_kernel(const uint16_t* rows, const int32_t* rows_of_token,
                                                           const float* row_weight, int T, int H8, int n_rows,
                                                           int renormalize, uint16_t* out) {
#pragma clang fp contract(off)   // hipcc contracts a * b + c into an fma by default; the operators below are written out
                                 // (not __fmul_rn / __fadd_rn, whose bodies the pragma does not reach) so that it applies
  const size_t total = (size_t)T * H8, stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
    const size_t t = i / H8;
    const unsigned c = (unsigned)(i % H8);
    const int r0 = rows_of_token[2 * t], r1 = rows_of_token[2 * t + 1];
    const bool ok0 = r0 >= 0 && r0 < n_rows, ok1 = r1 >= 0 && r1 < n_rows;   // a row out of range counts as zeros
    float w0 = ok0 ? row_weight[r0] : 0.f, w1 = ok1 ? row_weight[r1] : 0.f;
    if (renormalize) {
      const float sum = w0 + w1;
      w0 = __fdiv_rn(w0, sum);
      w1 = __fdiv_rn(w1, sum);
    }
    const v4i zero = {0, 0, 0, 0};
    const v4i x0 = ok0 ? reinterpret_cast<const v4i*>(rows + (size_t)r0 * H8 * 8)[c] : zero;
    const v4i x1 = ok1 ? reinterpret_cast<const v4i*>(rows + (size_t)r1 * H8 * 8)[c] : zero;
    v4i o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float a_lo = __builtin_bit_cast(float, (unsigned)x0[j] << 16), a_hi = __builtin_bit_cast(float, (unsigned)x0[j] & 0xFFFF0000u);
      const float b_lo = __builtin_bit_cast(float, (unsigned)x1[j] << 16), b_hi = __builtin_bit_cast(float, (unsigned)x1[j] & 0xFFFF0000u);
      const float lo = w0 * a_lo + w1 * b_lo;   // three roundings each: see the pragma above
      const float hi = w0 * a_hi + w1 * b_hi;
      o[j] = (int)pack_bf16x2(lo, hi);
    }
    reinterpret_cast<v4i*>(out + t * H8 * 8)[c] = o;
  }
}

}  // namespace

int route_top2_max_experts() { return 256; }

hipError_t launch_route_top2(const float* logits, int T, int E, int32_t* token_of_row, int32_t* row_offsets,
                             float* row_weight, int32_t* rows_of_token, hipStream_t s) {
  // token ranges per expert: enough workgroups to occupy the chip, at least one iteration each
  const int iters = (T + kRouteThreads - 1) / kRouteThreads;
  int parts = 256 / E;
  parts = parts > 8 ? 8 : parts;
  parts = parts > iters ? iters : parts;
  parts = parts < 1 ? 1 : parts;
  hipLaunchKernelGGL(route_top2_kernel, dim3((unsigned)(E * parts)), dim3(kRouteThreads), 0, s, logits, T, E, parts,
                     token_of_row, row_offsets, row_weight, rows_of_token);
  return hipGetLastError();
}

hipError_t launch_combine_top2(const uint16_t* rows, const int32_t* rows_of_token, const float* row_weight, int T, int H,
                               int n_rows, int renormalize, uint16_t* out, hipStream_t s) {
  const size_t total = (size_t)T * (H / 8);
  if (total == 0) return hipSuccess;
  size_t blocks = (total + 255) / 256;
  if (blocks > 256 * 16) blocks = 256 * 16;   // grid-stride beyond 16 workgroups per CU
  hipLaunchKernelGGL(combine_top2_kernel, dim3((unsigned)blocks), dim3(256), 0, s, rows, rows_of_token, row_weight, T,
                     H / 8, n_rows, renormalize, out);
  return hipGetLastError();
}

hipError_t launch_gather_rows(const uint8_t* src, const uint8_t* src_s, const int32_t* index, int rows, int src_rows,
                              int K, uint8_t* dst, uint8_t* dst_s, hipStream_t s) {
  const unsigned row_bytes = (unsigned)K / 2, row_scales = (unsigned)K / 32;
  const uintptr_t sbits = reinterpret_cast<uintptr_t>(src_s) | reinterpret_cast<uintptr_t>(dst_s) | row_scales;
  const int sv = (sbits & 15) == 0 ? 16 : ((sbits & 3) == 0 ? 4 : 1);
  const size_t total = (size_t)rows * (row_bytes / 16 + row_scales / sv);
  size_t blocks = (total + 255) / 256;
  if (blocks > 256 * 16) blocks = 256 * 16;   // grid-stride beyond 16 workgroups per CU
  const dim3 grid((unsigned)blocks), block(256);
  if (sv == 16)
    hipLaunchKernelGGL(gather_rows_kernel<16>, grid, block, 0, s, src, src_s, index, rows, src_rows, row_bytes,
                       row_scales, dst, dst_s);
  else if (sv == 4)
    hipLaunchKernelGGL(gather_rows_kernel<4>, grid, block, 0, s, src, src_s, index, rows, src_rows, row_bytes,
                       row_scales, dst, dst_s);
  else
    hipLaunchKernelGGL(gather_rows_kernel<1>, grid, block, 0, s, src, src_s, index, rows, src_rows, row_bytes,
                       row_scales, dst, dst_s);
  return hipGetLastError();
}

}  // namespace ave
