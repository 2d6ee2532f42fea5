// NVFP4 GEMM for gfx950 with operands staged in LDS as f16: every element is dequantised ONCE per workgroup, and K
// advances in steps of 64 elements -- the LDS-staged kernel for every K the format allows (K % 16 == 0) that
// gemm_nv_tile.hip (K % 256 == 0) cannot run.  K % 64 != 0 (TAILK): the last step holds one to three scale blocks of 16;
// the blocks behind the row's end are staged as zeros, and since rows then start at multiples of 8 bytes only and scale
// rows anywhere, codes are fetched in 8-byte pieces and scale bytes one by one.
//
// E4M3 scales per 16 elements do not fit the scaled MFMA (one E8M0 per 32), so NVFP4 operands are multiplied as f16
// (E2M1 x E4M3 has at most 6 significant bits and lies in [2^-10, 2688]: exact in f16) with
// v_mfma_f32_32x32x16_f16.  The kernel of gemm_nv_tile.hip keeps the packed codes in LDS and lets every wave convert
// the fragments it multiplies: each A row is converted twice and each B row four times per workgroup (eight waves
// of 64 x 128 on a 256 x 256 tile).  Here the conversion sits on the way INTO LDS instead:
//
//   global (packed codes + E4M3 bytes) -> VGPRs -> f16 -> LDS -> fragments -> MFMA
//
// which converts a third as much but moves four times the bytes through LDS.  Measured on 4096 x 4096 x 14336: 385 us
// against 335 us for the fp4-staged kernel on the same device -- without the conversions this kernel takes 352 us,
// without its fragment reads 364 us: it has the MXFP4 tile kernel's data flow and its time per 32 MFMAs and wave
// (1.7 us), while the fp4-staged kernel's conversions run under its MFMAs.  So this kernel serves the shapes the other
// cannot run.
//
// Per step the 512 lanes of the workgroup convert the step's 512 rows x 64
// elements exactly once -- a lane owns 32 elements of one A row and 32 of one B row: 16 bytes of codes and two scale
// bytes each -- and write them as f16 into a row-major [256 rows][128 B] image per operand, the geometry of the
// MXFP4 tile kernel's stage (16-byte chunk c of row r at position c ^ ((r >> 1) & 7), conflict-free for the
// fragment reads and for these writes).  Two such images (64 KB each) alternate; the raw codes of the next two
// steps are in flight in registers meanwhile, so a load has two steps of MFMA time to land.  One barrier per step,
// in front of the last quarter of its MFMAs as in the MXFP4 kernel: by then every wave has read the step's
// fragments and written its share of the next step's image.
//
// K order inside a step: MFMA ks (0..3) of lane half h consumes the 8 elements of chunk 4h + ks; A and B fragments
// use the same assignment, so the sum runs over every k exactly once.  MFMA operand roles and the B-row permutation
// are those of the MXFP4 tile kernel (srcA = rows of B, srcB = rows of A: a lane's 16 results are two runs of 8
// consecutive n of one row of C).  The two fp32 per-tensor scales are applied once, in the epilogue.
#include "fp4_common.hpp"
#include "kernels.hpp"
#include "tile_common.hpp"
#include "tile_map.hpp"

namespace ave {
namespace {

constexpr int BM = 256, BN = 256, BKS = 64;   // BKS: elements of K per step
constexpr int kWaves = 8;
constexpr int kRowBytes = BKS * 2;            // 128: one row of a step as f16
constexpr int kOffB = BM * kRowBytes;         // 32768
constexpr int kStepBytes = kOffB + BN * kRowBytes;   // 65536
constexpr int kLdsBytes = 2 * kStepBytes;     // 131072

__device__ inline void lds_write16(unsigned addr, v8h v) {
  *reinterpret_cast<__attribute__((address_space(3))) v8h*>((uintptr_t)addr) = v;
}
__device__ inline v8h lds_read8h(unsigned addr) {
  return *reinterpret_cast<const __attribute__((address_space(3))) v8h*>((uintptr_t)addr);
}

template <bool TAILK>
__global__ __launch_bounds__(kWaves * 64) void nv_f16_tile_kernel(NvArgs p, int m_tiles, int n_tiles) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int wm = w >> 1, wn = w & 1;

  int tm, tn;
  map_tile(blockIdx.x, m_tiles, n_tiles, tm, tn);
  const int m_begin = tm * BM, n_begin = tn * BN;
  const unsigned row_bytes = (unsigned)p.K / 2, row_scales = (unsigned)p.K / 16;
  // a wave whose 64 rows lie past the end of A multiplies nothing; it still converts its share of every step
  const bool active = m_begin + wm * 64 < p.M;

  // ---- producer side: this lane's 32 elements of tile row `prow` of A and of B per step -----------------------------
  // Rows past the end of a matrix are clamped to its last row: their products land in elements of C never stored.
  const int prow = tid >> 1, hf = tid & 1;
  int am = m_begin + prow, bn = n_begin + prow;
  am = am < p.M ? am : p.M - 1;
  bn = bn < p.N ? bn : p.N - 1;
  const uint8_t* a_codes = p.A + (size_t)am * row_bytes + hf * 16;   // + 32 bytes per step
  const uint8_t* b_codes = p.B + (size_t)bn * row_bytes + hf * 16;
  const uint8_t* a_scl = p.As + (size_t)am * row_scales;             // + 4 bytes per step; this lane's two are 2 hf, 2 hf + 1
  const uint8_t* b_scl = p.Bs + (size_t)bn * row_scales;
  const unsigned lds_base = (unsigned)(uintptr_t)lds;
  // chunk 4 hf + d of the row goes to position (4 hf + d) ^ ((row >> 1) & 7) = ((4 hf) ^ swizzle) ^ d
  const unsigned wr = (unsigned)prow * kRowBytes + (unsigned)((((4 * hf) ^ ((prow >> 1) & 7))) * 16);

  struct Raw {
    v4i a, b;      // 32 codes each
    int as, bs;    // the step's four E4M3 bytes of the row
  };
  auto load_raw = [&](int step) {
    Raw r;
    if constexpr (!TAILK) {
      r.a = *reinterpret_cast<const v4i*>(a_codes + (size_t)step * 32);
      r.b = *reinterpret_cast<const v4i*>(b_codes + (size_t)step * 32);
      r.as = *reinterpret_cast<const int*>(a_scl + (size_t)step * 4);
      r.bs = *reinterpret_cast<const int*>(b_scl + (size_t)step * 4);
    } else {
      // scale blocks from the step's start to the row's end; this lane's are 2 hf and 2 hf + 1 of the step's four.
      // What lies behind the row's end is neither read (the last row ends where the tensor ends) nor multiplied.
      const int blocks_left = p.K / 16 - step * 4;
      r.a = r.b = v4i{0, 0, 0, 0};
      r.as = r.bs = 0;
#pragma unroll
      for (int j = 0; j < 2; ++j)
        if (2 * hf + j < blocks_left) {
          v2i ca, cb;
          __builtin_memcpy(&ca, a_codes + (size_t)step * 32 + 8 * j, 8);   // rows start at multiples of 8 bytes
          __builtin_memcpy(&cb, b_codes + (size_t)step * 32 + 8 * j, 8);
          r.a[2 * j] = ca[0];
          r.a[2 * j + 1] = ca[1];
          r.b[2 * j] = cb[0];
          r.b[2 * j + 1] = cb[1];
        }
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (q < blocks_left) {
          r.as |= (int)a_scl[(size_t)step * 4 + q] << (8 * q);
          r.bs |= (int)b_scl[(size_t)step * 4 + q] << (8 * q);
        }
    }
    return r;
  };
  // dequantise this lane's 2 x 32 elements and write them into the image at `img`
  auto convert_store = [&](const Raw& r, unsigned img) {
    const v2h sa = scale_pair(r.as >> (16 * hf)), sb = scale_pair(r.bs >> (16 * hf));
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      lds_write16(img + (wr ^ (d * 16)), dequant8((unsigned)r.a[d], sa[d >> 1]));
      lds_write16(img + kOffB + (wr ^ (d * 16)), dequant8((unsigned)r.b[d], sb[d >> 1]));
    }
  };

  // ---- consumer side: fragment read addresses -----------------------------------------------------------------------
  const int rho = lane & 31, h = lane >> 5;
  const int a_row = wm * 64 + rho;              // + 32 mi
  const int b_row = wn * 128 + pi_row(rho);     // + 32 nj
  const unsigned a_frag = a_row * kRowBytes + (((4 * h) ^ ((a_row >> 1) & 7)) * 16);            // ^ ks * 16
  const unsigned b_frag = kOffB + b_row * kRowBytes + (((4 * h) ^ ((b_row >> 1) & 7)) * 16);

  v16f acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = v16f{};
  v8h af0[2], bf0[4], af1[2], bf1[4];

#define AVE_READ_FRAGS(dst_a, dst_b, img, KS)                                                                      \
  _Pragma("unroll") for (int i = 0; i < 2; ++i) dst_a[i] = lds_read8h((img) + (a_frag ^ ((KS) * 16)) + i * 4096);  \
  _Pragma("unroll") for (int i = 0; i < 4; ++i) dst_b[i] = lds_read8h((img) + (b_frag ^ ((KS) * 16)) + i * 4096);
#define AVE_MMA(fa, fb)                                                  \
  _Pragma("unroll") for (int nj = 0; nj < 4; ++nj)                       \
  _Pragma("unroll") for (int mi = 0; mi < 2; ++mi)                       \
      acc[nj][mi] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[nj], fa[mi], acc[nj][mi], 0, 0, 0);

  const int s_begin = 0, s_end = (p.K + BKS - 1) / BKS;   // TAILK: the last step is partly zeros
  // raw0 / raw1 hold the codes of the even / odd steps (counted from s_begin): the step being converted and the one
  // after it
  Raw raw0 = load_raw(s_begin), raw1 = raw0;
  if (s_begin + 1 < s_end) raw1 = load_raw(s_begin + 1);
  convert_store(raw0, lds_base);
  if (s_begin + 2 < s_end) raw0 = load_raw(s_begin + 2);
  __syncthreads();
  int s = s_begin;
  if (!active) {
    // a wave without rows: its share of every image, the barriers, its loads -- nothing else
    for (; s < s_end; ++s) {
      const int par = (s - s_begin) & 1;
      if (s + 1 < s_end) convert_store(par ? raw0 : raw1, lds_base + (par ^ 1) * kStepBytes);
      __syncthreads();
      if (s + 3 < s_end) {
        if (par) raw0 = load_raw(s + 3);
        else raw1 = load_raw(s + 3);
      }
    }
    return;
  }
  AVE_READ_FRAGS(af0, bf0, lds_base, 0)

  // One step; PAR is its parity counted from s_begin: its image is buffer PAR, the next step's codes are in RAW_NEXT.
  // MORE: step s + 1 exists; LOAD3: step s + 3 exists (both `true` at compile time in the main loop).  The step is
  // cut into eight groups of four MFMAs, fenced so that the compiler keeps them apart: the first six each carry one
  // or two of the eight conversion pieces of the next image (8 elements -> 8 VALU instructions and one LDS write
  // each would be 64; a piece is 8 elements of one operand: 8 VALU + 1 write) and the fragment reads of the
  // following quarter, earliest-needed first; the barrier sits in front of the last two.
#define AVE_MMA4(fa, fb, NJ0)                                                                        \
  _Pragma("unroll") for (int nj = (NJ0); nj < (NJ0) + 2; ++nj)                                       \
  _Pragma("unroll") for (int mi = 0; mi < 2; ++mi)                                                   \
      acc[nj][mi] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[nj], fa[mi], acc[nj][mi], 0, 0, 0);
#define AVE_PIECE_A(RAW, D) lds_write16(img_next + (wr ^ ((D) * 16)), dequant8((unsigned)RAW.a[D], sa[(D) >> 1]));
#define AVE_PIECE_B(RAW, D) lds_write16(img_next + kOffB + (wr ^ ((D) * 16)), dequant8((unsigned)RAW.b[D], sb[(D) >> 1]));
#define AVE_READ_FIRST(dst_a, dst_b, img, KS) /* what the first group of a quarter needs */                \
  _Pragma("unroll") for (int i = 0; i < 2; ++i) dst_a[i] = lds_read8h((img) + (a_frag ^ ((KS) * 16)) + i * 4096);  \
  _Pragma("unroll") for (int i = 0; i < 2; ++i) dst_b[i] = lds_read8h((img) + (b_frag ^ ((KS) * 16)) + i * 4096);
#define AVE_READ_REST(dst_b, img, KS)                                                                      \
  _Pragma("unroll") for (int i = 2; i < 4; ++i) dst_b[i] = lds_read8h((img) + (b_frag ^ ((KS) * 16)) + i * 4096);
#define AVE_FENCE __builtin_amdgcn_sched_barrier(0);
#define AVE_STEP(PAR, RAW_NEXT, MORE, LOAD3)                                                                         \
  {                                                                                                                  \
    const unsigned img = lds_base + (PAR) * kStepBytes, img_next = lds_base + ((PAR) ^ 1) * kStepBytes;              \
    const v2h sa = scale_pair(RAW_NEXT.as >> (16 * hf)), sb = scale_pair(RAW_NEXT.bs >> (16 * hf));                 \
    AVE_MMA4(af0, bf0, 0)                                                                                            \
    AVE_READ_FIRST(af1, bf1, img, 1)                                                                                 \
    if (MORE) { AVE_PIECE_A(RAW_NEXT, 0) AVE_PIECE_A(RAW_NEXT, 1) }                                                  \
    AVE_FENCE                                                                                                        \
    AVE_MMA4(af0, bf0, 2)                                                                                            \
    AVE_READ_REST(bf1, img, 1)                                                                                       \
    if (MORE) { AVE_PIECE_A(RAW_NEXT, 2) }                                                                           \
    AVE_FENCE                                                                                                        \
    AVE_MMA4(af1, bf1, 0)                                                                                            \
    AVE_READ_FIRST(af0, bf0, img, 2)                                                                                 \
    if (MORE) { AVE_PIECE_A(RAW_NEXT, 3) }                                                                           \
    AVE_FENCE                                                                                                        \
    AVE_MMA4(af1, bf1, 2)                                                                                            \
    AVE_READ_REST(bf0, img, 2)                                                                                       \
    if (MORE) { AVE_PIECE_B(RAW_NEXT, 0) AVE_PIECE_B(RAW_NEXT, 1) }                                                  \
    AVE_FENCE                                                                                                        \
    AVE_MMA4(af0, bf0, 0)                                                                                            \
    AVE_READ_FIRST(af1, bf1, img, 3)                                                                                 \
    if (MORE) { AVE_PIECE_B(RAW_NEXT, 2) }                                                                           \
    AVE_FENCE                                                                                                        \
    AVE_MMA4(af0, bf0, 2)                                                                                            \
    AVE_READ_REST(bf1, img, 3)                                                                                       \
    if (MORE) { AVE_PIECE_B(RAW_NEXT, 3) }                                                                           \
    AVE_FENCE                                                                                                        \
    __syncthreads(); /* everyone has read this step's fragments and written its share of the next image */          \
    /* the registers of the step just converted take the codes of the step after the next */                        \
    if (LOAD3) RAW_NEXT = load_raw(s + 3);                                                                           \
    AVE_MMA4(af1, bf1, 0)                                                                                            \
    if (MORE) { AVE_READ_FIRST(af0, bf0, img_next, 0) }                                                              \
    AVE_FENCE                                                                                                        \
    AVE_MMA4(af1, bf1, 2)                                                                                            \
    if (MORE) { AVE_READ_REST(bf0, img_next, 0) }                                                                    \
    AVE_FENCE                                                                                                        \
  }
  for (; s + 4 < s_end; s += 2) {
    AVE_STEP(0, raw1, true, true)
    ++s;
    AVE_STEP(1, raw0, true, true)
    --s;
  }
  // the last steps (at most four), with the conditions evaluated at run time
  for (; s < s_end; ++s) {
    AVE_STEP(0, raw1, s + 1 < s_end, s + 3 < s_end)
    if (++s >= s_end) break;
    AVE_STEP(1, raw0, s + 1 < s_end, s + 3 < s_end)
  }
#undef AVE_STEP
#undef AVE_MMA4
#undef AVE_PIECE_A
#undef AVE_PIECE_B
#undef AVE_READ_FIRST
#undef AVE_READ_REST
#undef AVE_FENCE
#undef AVE_READ_FRAGS
#undef AVE_MMA

  const float g = p.Ag[0] * p.Bg[0];
  store_wave_block<2>(acc, p.C, p.N, m_begin + wm * 64, p.M, n_begin + wn * 128, lane, g);
}

}  // namespace

// K % 64 == 0: 16-byte pieces of the code rows and dwords of the scale rows must be aligned.  Other K (a multiple of
// 16): code rows in 8-byte pieces (A and B 8-byte aligned), scale bytes one by one.
bool nv_f16_tile_supports(const NvArgs& p) {
  if (p.K % 16 != 0 || p.K <= 0 || p.M <= 0 || p.N <= 0) return false;
  if (p.K % BKS != 0) return ((reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.B)) & 7) == 0;
  if ((reinterpret_cast<uintptr_t>(p.A) & 15) || (reinterpret_cast<uintptr_t>(p.B) & 15)) return false;
  if ((reinterpret_cast<uintptr_t>(p.As) & 3) || (reinterpret_cast<uintptr_t>(p.Bs) & 3)) return false;
  return true;
}

hipError_t launch_nv_f16_tile(const NvArgs& p, hipStream_t s) {
  const int m_tiles = (p.M + BM - 1) / BM, n_tiles = (p.N + BN - 1) / BN;
  const dim3 grid((unsigned)(m_tiles * n_tiles)), block(kWaves * 64);
  if (p.K % BKS != 0) {
    if (hipError_t e = allow_dynamic_lds<nv_f16_tile_kernel<true>>(kLdsBytes); e != hipSuccess) return e;
    hipLaunchKernelGGL(nv_f16_tile_kernel<true>, grid, block, kLdsBytes, s, p, m_tiles, n_tiles);
  } else {
    if (hipError_t e = allow_dynamic_lds<nv_f16_tile_kernel<false>>(kLdsBytes); e != hipSuccess) return e;
    hipLaunchKernelGGL(nv_f16_tile_kernel<false>, grid, block, kLdsBytes, s, p, m_tiles, n_tiles);
  }
  return hipGetLastError();
}

}  // namespace ave
