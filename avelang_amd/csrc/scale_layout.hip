// Conversion between the row-major block-scale tensor the GEMM entry points take ([rows, cols], one
// byte per scale) and the blocked layout other FP4 stacks store scales in: the tensor is padded to
// multiples of 128 rows and 4 columns and cut into 128 x 4 tiles, tiles in row-major order, 512
// bytes each; inside a tile, scale (r, c) sits at byte (r % 32) * 16 + (r / 32) * 4 + c.
// Four scales of one row are one aligned dword of the blocked image, so a thread moves one dword.
#include "fp4_common.hpp"
#include "kernels.hpp"

namespace ave {
namespace {

__device__ inline size_t blocked_dword(unsigned r, unsigned cb, unsigned col_blocks) {
  const unsigned rt = r >> 7, ri = r & 127;
  return ((size_t)rt * col_blocks + cb) * 512 + (ri & 31) * 16 + (ri >> 5) * 4;
}

// TO_BLOCKED: plain -> blocked (padding written as zero); else blocked -> plain
template <bool TO_BLOCKED, bool DWORD>
__global__ __launch_bounds__(256) void scale_layout_kernel(const uint8_t* src, uint8_t* dst, unsigned rows,
                                                           unsigned cols, unsigned col_blocks, unsigned row_pad) {
  const size_t total = (size_t)row_pad * col_blocks;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
    const unsigned r = (unsigned)(i / col_blocks), cb = (unsigned)(i % col_blocks);
    const size_t boff = blocked_dword(r, cb, col_blocks);
    const size_t poff = (size_t)r * cols + 4 * cb;
    if (TO_BLOCKED) {
      unsigned v = 0;
      if (r < rows) {
        if (DWORD) {
          v = *reinterpret_cast<const unsigned*>(src + poff);
        } else {
#pragma unroll
          for (unsigned j = 0; j < 4; ++j)
            if (4 * cb + j < cols) v |= (unsigned)src[poff + j] << (8 * j);
        }
      }
      *reinterpret_cast<unsigned*>(dst + boff) = v;
    } else if (r < rows) {
      const unsigned v = *reinterpret_cast<const unsigned*>(src + boff);
      if (DWORD) {
        *reinterpret_cast<unsigned*>(dst + poff) = v;
      } else {
#pragma unroll
        for (unsigned j = 0; j < 4; ++j)
          if (4 * cb + j < cols) dst[poff + j] = (uint8_t)(v >> (8 * j));
      }
    }
  }
}

}  // namespace

hipError_t launch_scale_layout(const uint8_t* src, uint8_t* dst, int rows, int cols, bool to_blocked, hipStream_t s) {
  const unsigned col_blocks = ((unsigned)cols + 3) / 4, row_pad = (((unsigned)rows + 127) / 128) * 128;
  const uint8_t* plain = to_blocked ? src : dst;
  const bool dword = (cols % 4 == 0) && (reinterpret_cast<uintptr_t>(plain) & 3) == 0;
  const size_t total = (size_t)row_pad * col_blocks;
  size_t blocks = (total + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  const dim3 grid((unsigned)blocks), block(256);
#define AVE_LAUNCH(TB, DW) \
  hipLaunchKernelGGL((scale_layout_kernel<TB, DW>), grid, block, 0, s, src, dst, (unsigned)rows, (unsigned)cols, col_blocks, row_pad)
  if (to_blocked) {
    if (dword) AVE_LAUNCH(true, true);
    else AVE_LAUNCH(true, false);
  } else {
    if (dword) AVE_LAUNCH(false, true);
    else AVE_LAUNCH(false, false);
  }
#undef AVE_LAUNCH
  return hipGetLastError();
}

}  // namespace ave
