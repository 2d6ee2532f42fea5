// NVFP4 GEMM for decode-time shapes (at most 64 activation rows) on gfx950: the weights are streamed from HBM
// exactly once and dequantised exactly once, in the registers of the one workgroup that owns their rows.  (The
// LDS-staged NVFP4 kernel dequantises whole 256-row operand tiles per stage whatever M is: 85 us for 16 rows against
// 28672 x 4096 weights.)
//
// A workgroup owns T consecutive 16-column tiles of C and splits K over its WAVES wavefronts: wave w handles the
// K steps (128 elements each) SPW*w .. SPW*w+SPW-1 of every chunk of WAVES*SPW steps.  Per step a lane loads, for
// every tile, the 16 bytes of row l % 16 that hold k = 128 s + 32 (l / 16) .. + 31 -- two scale blocks -- and their
// two E4M3 bytes, converts them to f16 (E2M1 x E4M3 is exact in f16) and feeds dword d (8 elements) to MFMA d of the
// step: v_mfma_f32_16x16x32_f16 with srcA = weight rows, srcB = activation rows, so a lane ends with 4 consecutive
// n of one row m.  Activation and weight fragments use the same assignment of k to lanes and MFMAs, so the sum
// runs over every k exactly once.  MB blocks of 16 activation rows share every dequantised weight fragment.
// Partial tiles of the waves are summed through LDS; the two per-tensor scales are applied once, at the end.
#include "fp4_common.hpp"
#include "kernels.hpp"

namespace ave {
namespace {

constexpr int kWaves = 8, kSpw = 2;

template <int T, int MB>
__global__ __launch_bounds__(kWaves * 64) void nv_decode_kernel(NvArgs p, int n_tiles16) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int r = lane & 15, g = lane >> 4;
  const int tile0 = blockIdx.x * T;
  const unsigned row_bytes = (unsigned)p.K / 2, row_scales = (unsigned)p.K / 16;
  const int steps = p.K / 128;

  // Buffer resources give 32-bit offsets and make rows past M / N read as zeros (zero codes and a zero scale).
  // The hardware compares only the per-lane offset (plus the immediate) with the buffer size, not the scalar offset
  // operand: the row displacement of a tile or row block therefore goes into the per-lane offset, and the scalar
  // operand carries the position inside the row alone, which is in range for every row.
  const __amdgpu_buffer_rsrc_t ra = make_rsrc(p.A, (unsigned)p.M * row_bytes);
  const __amdgpu_buffer_rsrc_t ras = make_rsrc(p.As, (unsigned)p.M * row_scales);
  const __amdgpu_buffer_rsrc_t rb = make_rsrc(p.B, (unsigned)p.N * row_bytes);
  const __amdgpu_buffer_rsrc_t rbs = make_rsrc(p.Bs, (unsigned)p.N * row_scales);
  const unsigned a_off = (unsigned)r * row_bytes + 16 * g;          // + mb * 16 * row_bytes
  const unsigned as_off = (unsigned)r * row_scales + 2 * g;         // + mb * 16 * row_scales
  const unsigned b_off = (unsigned)(tile0 * 16 + r) * row_bytes + 16 * g;   // + t * 16 * row_bytes
  const unsigned bs_off = (unsigned)(tile0 * 16 + r) * row_scales + 2 * g;  // + t * 16 * row_scales

  v4f acc[T][MB];
#pragma unroll
  for (int t = 0; t < T; ++t)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[t][mb] = v4f{0, 0, 0, 0};

  for (int c0 = 0; c0 < steps; c0 += kWaves * kSpw) {
    const int s0 = c0 + w * kSpw;
    v4i af[MB][kSpw], bf[T][kSpw];
    int asc[MB][kSpw], bsc[T][kSpw];
#pragma unroll
    for (int j = 0; j < kSpw; ++j) {
      const int s = s0 + j;
      if (s < steps) {
#pragma unroll
        for (int t = 0; t < T; ++t) {
          bf[t][j] = __builtin_amdgcn_raw_buffer_load_b128(rb, b_off + t * 16 * row_bytes, s * 64, 0);
          bsc[t][j] = (int)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(rbs, bs_off + t * 16 * row_scales, s * 8, 0);
        }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          af[mb][j] = __builtin_amdgcn_raw_buffer_load_b128(ra, a_off + mb * 16 * row_bytes, s * 64, 0);
          asc[mb][j] = (int)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(ras, as_off + mb * 16 * row_scales, s * 8, 0);
        }
      }
    }
#pragma unroll
    for (int j = 0; j < kSpw; ++j) {
      const int s = s0 + j;
      if (s < steps) {
        v8h a8[MB][4];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          const v2h sa = scale_pair(asc[mb][j]);
#pragma unroll
          for (int d = 0; d < 4; ++d) a8[mb][d] = dequant8((unsigned)af[mb][j][d], sa[d >> 1]);
        }
#pragma unroll
        for (int t = 0; t < T; ++t) {
          const v2h sb = scale_pair(bsc[t][j]);
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            const v8h b8 = dequant8((unsigned)bf[t][j][d], sb[d >> 1]);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
              acc[t][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b8, a8[mb][d], acc[t][mb], 0, 0, 0);
          }
        }
      }
    }
  }

  // ---- sum the partial tiles of the waves through LDS, apply the per-tensor scales, store bf16 ----------------
  v4f* part = reinterpret_cast<v4f*>(lds);  // [kWaves][T * MB][64]
#pragma unroll
  for (int t = 0; t < T; ++t)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) part[((w * T + t) * MB + mb) * 64 + lane] = acc[t][mb];
  __syncthreads();
  const float gscale = p.Ag[0] * p.Bg[0];
  for (int u = tid; u < T * MB * 64; u += kWaves * 64) {
    v4f s = part[u];
#pragma unroll
    for (int ww = 1; ww < kWaves; ++ww) s += part[ww * T * MB * 64 + u];
    const int tb = u >> 6, l = u & 63;
    const int t = tb / MB, mb = tb % MB;
    const int m = 16 * mb + (l & 15), n = (tile0 + t) * 16 + 4 * (l >> 4);
    if (m < p.M && n < p.N) {
      uint16_t* dst = p.C + (size_t)m * p.N + n;
      if (n + 4 <= p.N && (p.N % 4 == 0) && ((reinterpret_cast<uintptr_t>(p.C) & 7) == 0)) {
        v2i o = {(int)pack_bf16x2(s[0] * gscale, s[1] * gscale), (int)pack_bf16x2(s[2] * gscale, s[3] * gscale)};
        *reinterpret_cast<v2i*>(dst) = o;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n + e < p.N) dst[e] = to_bf16(s[e] * gscale);
      }
    }
  }
}

template <int T, int MB>
hipError_t launch_t(const NvArgs& p, hipStream_t s, int n_tiles16) {
  constexpr int lds_bytes = kWaves * T * MB * 64 * 16;
  if (hipError_t e = allow_dynamic_lds<nv_decode_kernel<T, MB>>(lds_bytes); e != hipSuccess) return e;
  const unsigned grid = (unsigned)((n_tiles16 + T - 1) / T);
  hipLaunchKernelGGL((nv_decode_kernel<T, MB>), dim3(grid), dim3(kWaves * 64), lds_bytes, s, p, n_tiles16);
  return hipGetLastError();
}

}  // namespace

// At most 64 rows, whole K steps, 16-byte aligned code rows, 2-byte aligned scale rows, 32-bit buffer sizes.
bool nv_decode_supports(const NvArgs& p) {
  if (nv_ring_supports(p)) return true;   // K a multiple of 32 from 512 up (33..64 rows: an even number of 512-element units)
  if (p.M <= 0 || p.M > 64 || p.N <= 0 || p.K <= 0 || p.K % 128 != 0) return false;
  if ((uint64_t)p.M * (uint64_t)(p.K / 2) >= (1ull << 32) || (uint64_t)p.N * (uint64_t)(p.K / 2) >= (1ull << 32)) return false;
  if ((reinterpret_cast<uintptr_t>(p.A) & 15) || (reinterpret_cast<uintptr_t>(p.B) & 15)) return false;
  if ((reinterpret_cast<uintptr_t>(p.As) & 1) || (reinterpret_cast<uintptr_t>(p.Bs) & 1)) return false;
  return true;
}

hipError_t launch_nv_decode(const NvArgs& p, hipStream_t s) {
  // whole 512-element units of K (33..64 rows: an even number of them): the same weights through LDS rings (gemm_mx_decode.hip), whose
  // 1 KB loads keep the memory system busier than the 64-byte pieces per row of the loads into registers here
  if (nv_ring_supports(p)) return launch_nv_ring(p, s);
  const int n_tiles16 = (p.N + 15) / 16;
  const int mb = p.M <= 16 ? 1 : (p.M <= 32 ? 2 : 4);
  // tiles per workgroup so that one round covers the 256 compute units, as far as the registers allow:
  // a tile costs 4 * MB accumulator registers and 10 for its loads in flight
  const int t_max = mb == 1 ? 7 : (mb == 2 ? 6 : 4);
  const int t = tiles_per_workgroup(n_tiles16, compute_units(), t_max);
#define AVE_NV_CASE(TT, MM) \
  if (t == TT && mb == MM) return launch_t<TT, MM>(p, s, n_tiles16);
  AVE_NV_CASE(1, 1) AVE_NV_CASE(2, 1) AVE_NV_CASE(3, 1) AVE_NV_CASE(4, 1) AVE_NV_CASE(5, 1) AVE_NV_CASE(6, 1) AVE_NV_CASE(7, 1)
  AVE_NV_CASE(1, 2) AVE_NV_CASE(2, 2) AVE_NV_CASE(3, 2) AVE_NV_CASE(4, 2) AVE_NV_CASE(5, 2) AVE_NV_CASE(6, 2)
  AVE_NV_CASE(1, 4) AVE_NV_CASE(2, 4) AVE_NV_CASE(3, 4) AVE_NV_CASE(4, 4)
#undef AVE_NV_CASE
  return hipErrorInvalidValue;
}

}  // namespace ave
