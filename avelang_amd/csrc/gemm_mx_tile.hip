// MXFP4 GEMM for gfx950, compute-bound shapes: 256x256 output tile per workgroup, four
// wavefronts (2x2) of 128x128 each, v_mfma_scale_f32_32x32x64_f8f6f4 with E8M0 scales fed
// through the instruction's scale operands, fp32 accumulation in 256 registers per lane,
// bf16 round-to-nearest-even epilogue.  Also serves the grouped (MoE) GEMM: the m-tile list
// is then the concatenation of the experts' tile lists, found from row_offsets on the device.
//
// Data movement per K stage of 256 elements (128 bytes per row):
//   global -> LDS with global_load_lds_dwordx4 (no register staging).  One wave instruction
//   moves 8 rows x 128 B: 8 consecutive lanes fetch one full 128-byte line.  A lane's 16 bytes
//   land at LDS address base + 16*lane, so the LDS image is row-major [256][128 B]; the XOR
//   swizzle that makes the MFMA fragment reads conflict-free is applied on the *source* side:
//   LDS chunk c' of row r holds global chunk c' ^ (r & 7).
//   Scales: [256 rows][8 B] per operand and stage, moved with global_load_lds_dword.
//   Two stage buffers; one barrier per stage; the loads of stage s+1 are in flight while the
//   MFMAs of stage s run.
//
// MFMA operand roles: srcA carries rows of B (n), srcB carries rows of A (m), so a lane's 16
// results are 16 values of ONE row of C.  B rows are handed to the fragment in the order
// pi(8u+4q+v) = 16(u/2) + 8q + 4(u%2) + v, which makes those 16 values two runs of 8
// consecutive n: the epilogue stores two 16-byte pieces per 32x32 block.
#include "fp4_common.hpp"
#include "kernels.hpp"
#include "tile_map.hpp"
#include "tile_common.hpp"

namespace ave {
namespace {

constexpr int BM = 256, BN = 256, BK = 256;
constexpr int kRowBytes = BK / 2;                    // 128
constexpr int kOffA = 0;
constexpr int kOffB = BM * kRowBytes;                // 32768
constexpr int kOffAs = kOffB + BN * kRowBytes;       // 65536
constexpr int kOffBs = kOffAs + BM * (BK / 32);      // +2048
constexpr int kStageBytes = kOffBs + BN * (BK / 32); // 69632
constexpr int kLdsBytes = 2 * kStageBytes;           // 139264

template <int KJ>
__device__ inline void mma_step(v16f (&acc)[4][4], const v4i (&bf)[4], const v4i (&af)[4], const v2i (&bs)[4],
                                const v2i (&as)[4]) {
  constexpr int OP = 2 * (KJ & 1);
#pragma unroll
  for (int nj = 0; nj < 4; ++nj)
#pragma unroll
    for (int mi = 0; mi < 4; ++mi)
      acc[nj][mi] = mfma32<OP, OP>(bf[nj], af[mi], acc[nj][mi], bs[nj][KJ >> 1], as[mi][KJ >> 1]);
}

__global__ __launch_bounds__(256) void mx_tile_kernel(MxArgs p, int m_tiles, int n_tiles) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int wm = w >> 1, wn = w & 1;

  int tm, tn;
  map_tile(blockIdx.x, m_tiles, n_tiles, tm, tn);
  int m_begin = tm * BM, m_end = p.M, expert = 0;
  if (p.row_offsets) {
    // tm indexes the concatenation of per-expert tile lists
    int first = 0;
    bool found = false;
    for (int e = 0; e < p.E; ++e) {
      const int r0 = p.row_offsets[e], r1 = p.row_offsets[e + 1];
      const int nt = (r1 - r0 + BM - 1) / BM;
      if (!found && tm < first + nt) {
        expert = e;
        m_begin = r0 + (tm - first) * BM;
        m_end = r1;
        found = true;
      }
      first += nt;
    }
    if (!found) return;
  }
  const int n_begin = tn * BN;
  const unsigned row_bytes = (unsigned)p.K / 2, row_scales = (unsigned)p.K / 32;
  const uint8_t* Bmat = p.B + (size_t)expert * p.N * row_bytes;
  const uint8_t* Bsc = p.Bs + (size_t)expert * p.N * row_scales;

  // ---- per-lane source offsets of the direct-to-LDS loads -----------------------------
  // data: wave w, instruction i covers tile rows (8w+i)*8 .. +7; lane -> (row, swizzled chunk)
  unsigned a_off[8], b_off[8], as_off[2], bs_off[2];
  {
    const int lr = lane >> 3, cprime = lane & 7;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = (w * 8 + i) * 8 + lr;
      const int chunk = cprime ^ (row & 7);
      int am = m_begin + row;
      am = am < p.M ? am : p.M - 1;
      int bn = n_begin + row;
      bn = bn < p.N ? bn : p.N - 1;
      a_off[i] = (unsigned)am * row_bytes + chunk * 16;
      b_off[i] = (unsigned)bn * row_bytes + chunk * 16;
    }
    // scales: wave w, instruction j covers tile rows (2w+j)*32 .. +31; lane -> (row, dword)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int row = (w * 2 + j) * 32 + (lane >> 1);
      int am = m_begin + row;
      am = am < p.M ? am : p.M - 1;
      int bn = n_begin + row;
      bn = bn < p.N ? bn : p.N - 1;
      as_off[j] = (unsigned)am * row_scales + (lane & 1) * 4;
      bs_off[j] = (unsigned)bn * row_scales + (lane & 1) * 4;
    }
  }
  const unsigned lds_base = (unsigned)(uintptr_t)lds;

  auto issue_stage = [&](int s, int buf) {
    const uint8_t* ga = p.A + (size_t)s * kRowBytes;
    const uint8_t* gb = Bmat + (size_t)s * kRowBytes;
    const uint8_t* gas = p.As + (size_t)s * (BK / 32);
    const uint8_t* gbs = Bsc + (size_t)s * (BK / 32);
    const unsigned sb = lds_base + buf * kStageBytes;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      dma16(ga, a_off[i], sb + kOffA + (w * 8 + i) * 1024);
      dma16(gb, b_off[i], sb + kOffB + (w * 8 + i) * 1024);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      dma4(gas, as_off[j], sb + kOffAs + (w * 2 + j) * 256);
      dma4(gbs, bs_off[j], sb + kOffBs + (w * 2 + j) * 256);
    }
  };

  // ---- per-lane fragment read addresses ------------------------------------------------
  const int rho = lane & 31, h = lane >> 5;
  const int a_row = wm * 128 + rho;            // + 32*mi
  const int b_row = wn * 128 + pi_row(rho);    // + 32*nj
  const unsigned a_frag = kOffA + a_row * kRowBytes + ((h ^ (a_row & 7)) * 16);   // ^ (kj*32), + mi*4096
  const unsigned b_frag = kOffB + b_row * kRowBytes + ((h ^ (b_row & 7)) * 16);
  const unsigned a_sc = kOffAs + a_row * 8;    // + mi*256
  const unsigned b_sc = kOffBs + b_row * 8;

  v16f acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = v16f{};

  const int stages = p.K / BK;
  issue_stage(0, 0);
  for (int s = 0; s < stages; ++s) {
    const int buf = s & 1;
    wait_all_loads();
    __syncthreads();
    if (s + 1 < stages) issue_stage(s + 1, buf ^ 1);
    const unsigned sb = lds_base + buf * kStageBytes;

    v2i as[4], bs[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v2i x = lds_read8(sb + a_sc + i * 256);
      v2i y = lds_read8(sb + b_sc + i * 256);
      as[i] = v2i{rotr_bytes(x[0], h), rotr_bytes(x[1], h)};
      bs[i] = v2i{rotr_bytes(y[0], h), rotr_bytes(y[1], h)};
    }
    v4i af[4], bf[4];
#define AVE_LOAD_FRAGS(KJ)                                              \
  _Pragma("unroll") for (int i = 0; i < 4; ++i) {                       \
    af[i] = lds_read16(sb + (a_frag ^ ((KJ) * 32)) + i * 4096);         \
    bf[i] = lds_read16(sb + (b_frag ^ ((KJ) * 32)) + i * 4096);         \
  }
    AVE_LOAD_FRAGS(0) mma_step<0>(acc, bf, af, bs, as);
    AVE_LOAD_FRAGS(1) mma_step<1>(acc, bf, af, bs, as);
    AVE_LOAD_FRAGS(2) mma_step<2>(acc, bf, af, bs, as);
    AVE_LOAD_FRAGS(3) mma_step<3>(acc, bf, af, bs, as);
#undef AVE_LOAD_FRAGS
  }

  // ---- epilogue: fp32 -> bf16 (RNE), two 16-byte pieces per 32x32 block ----------------
  store_wave_block(acc, p.C, p.N, m_begin + wm * 128, m_end, n_begin + wn * 128, lane, 1.0f);
}

}  // namespace

bool mx_tile_supports(const MxArgs& p) {
  if (p.K % BK != 0 || p.M <= 0 || p.N <= 0) return false;
  // 32-bit byte offsets inside A and inside one expert's B
  if ((uint64_t)p.M * (uint64_t)(p.K / 2) >= (1ull << 32)) return false;
  if ((uint64_t)p.N * (uint64_t)(p.K / 2) >= (1ull << 32)) return false;
  // scale rows are fetched as aligned dwords
  if ((reinterpret_cast<uintptr_t>(p.As) & 3) || (reinterpret_cast<uintptr_t>(p.Bs) & 3)) return false;
  return true;
}

hipError_t launch_mx_tile(const MxArgs& p, hipStream_t s) {
  static hipError_t attr_state = hipFuncSetAttribute(reinterpret_cast<const void*>(mx_tile_kernel),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
  if (attr_state != hipSuccess) return attr_state;
  const int m_tiles = (p.M + BM - 1) / BM + (p.row_offsets ? p.E : 0);
  const int n_tiles = (p.N + BN - 1) / BN;
  hipLaunchKernelGGL(mx_tile_kernel, dim3((unsigned)(m_tiles * n_tiles)), dim3(256), kLdsBytes, s, p, m_tiles,
                     n_tiles);
  return hipGetLastError();
}

}  // namespace ave
