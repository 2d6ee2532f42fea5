// MXFP4 GEMM for decode-time shapes (M <= 16) on gfx950: the weights B are streamed from
// HBM exactly once, straight into MFMA operand registers; nothing but the 16-row activation
// panel is re-read.  The kernel is bound by HBM bandwidth, so the design is about keeping
// every weight byte of a workgroup in flight at once:
//
//   * a workgroup owns T consecutive 16-column tiles of C (T*16 rows of B) and splits K over
//     its WAVES wavefronts: wave w handles K steps (128 elements each) SPW*w .. SPW*w+SPW-1
//     of every chunk of WAVES*SPW steps;
//   * per step a lane issues one 16-byte load per tile (row l%16 of the tile, 32 consecutive
//     k = one E8M0 block) and all loads of a chunk are issued before the first MFMA;
//   * v_mfma_scale_f32_16x16x128_f8f6f4 with srcA = weight rows, srcB = activation rows, so a
//     lane ends with 4 consecutive n of one row m;
//   * the WAVES partial 16x16 tiles are summed through LDS and stored as bf16 (RNE).
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
  const int steps = p.K / 128;

  // Buffer resources give 32-bit offsets and make rows past M / N read as zeros
  // (zero codes contribute nothing whatever the scale byte is).
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
#pragma unroll
        for (int t = 0; t < T; ++t) {
          bf[t][j] = __builtin_amdgcn_raw_buffer_load_b128(rb, b_off, s * 64 + t * 16 * row_bytes, 0);
          bsc[t][j] = __builtin_amdgcn_raw_buffer_load_b32(rbs, bs_off, s * 4 + t * 16 * row_scales, 0);
        }
        af[j] = __builtin_amdgcn_raw_buffer_load_b128(ra, a_off, s * 64, 0);
        asc[j] = __builtin_amdgcn_raw_buffer_load_b32(ras, as_off, s * 4, 0);
      }
    }
#pragma unroll
    for (int j = 0; j < SPW; ++j) {
      const int s = s0 + j;
      if (s < steps) {
        const int sa = rotr_bytes(asc[j], g);
#pragma unroll
        for (int t = 0; t < T; ++t) acc[t] = mfma16<0, 0>(bf[t][j], af[j], acc[t], rotr_bytes(bsc[t][j], g), sa);
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
  static hipError_t attr_state =
      hipFuncSetAttribute(reinterpret_cast<const void*>(mx_decode_kernel<WAVES, T, SPW>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
  if (attr_state != hipSuccess) return attr_state;
  const unsigned grid = (unsigned)((n_tiles16 + T - 1) / T);
  hipLaunchKernelGGL((mx_decode_kernel<WAVES, T, SPW>), dim3(grid), dim3(WAVES * 64), lds_bytes, s, p, n_tiles16);
  return hipGetLastError();
}

}  // namespace

bool mx_decode_supports(const MxArgs& p) {
  if (p.row_offsets) return false;
  if (p.M < 1 || p.M > 16 || p.N < 1) return false;
  if (p.K % 128 != 0) return false;
  if ((reinterpret_cast<uintptr_t>(p.As) & 3) || (reinterpret_cast<uintptr_t>(p.Bs) & 3)) return false;
  if ((uint64_t)p.N * (uint64_t)(p.K / 2) >= (1ull << 32)) return false;   // 32-bit buffer offsets
  return true;
}

hipError_t launch_mx_decode(const MxArgs& p, hipStream_t s) {
  const int n_tiles16 = (p.N + 15) / 16;
  int t = (n_tiles16 + 255) / 256;  // tiles per workgroup so that one round covers the 256 CUs
  t = t < 1 ? 1 : (t > kMaxT ? kMaxT : t);
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
