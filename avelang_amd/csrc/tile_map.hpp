// Workgroup-id -> output-tile mapping for the LDS-staged kernels (host and device).
#pragma once

#ifdef __HIPCC__
#define AVE_HD __host__ __device__ inline
#else
#define AVE_HD inline
#endif

namespace ave {

constexpr int kXcds = 8;      // MI355X: 8 XCDs, each with its own L2; workgroup ids are dealt round-robin to them
// m-tiles per band; a band is walked m-fastest.  With 4, the 32 tiles an XCD runs at once form a
// 4 (m) x 8 (n) block: its 2 MB of A panels stay in the XCD's 4 MB L2 from round to round while the B
// panels stream through.  Measured on the 32 x 56 tile grid of the prefill GEMM: 1 -> 3250, 2 -> 3470,
// 4 -> 3557, 6 -> 3556, 8 -> 3355 TFLOP/s.
constexpr int kGroupM = 4;

// Undo the round-robin so that every XCD owns one contiguous range of tile numbers.
// Bijection on [0, total) for any total.
AVE_HD int xcd_contiguous_id(int pid, int total) {
  const int q = total / kXcds, rem = total % kXcds;
  const int xcd = pid % kXcds, local = pid / kXcds;
  const int first = xcd < rem ? xcd * (q + 1) : rem * (q + 1) + (xcd - rem) * q;
  return first + local;
}

// Banded order: kGroupM consecutive m-tiles x all n-tiles, m fastest inside the band.
AVE_HD void banded_tile(int id, int m_tiles, int n_tiles, int& tm, int& tn) {
  const int per_band = kGroupM * n_tiles;
  const int band = id / per_band;
  const int first_m = band * kGroupM;
  const int band_m = (m_tiles - first_m) < kGroupM ? (m_tiles - first_m) : kGroupM;
  const int in_band = id % per_band;
  tm = first_m + in_band % band_m;
  tn = in_band / band_m;
}

AVE_HD void map_tile(int pid, int m_tiles, int n_tiles, int& tm, int& tn) {
  banded_tile(xcd_contiguous_id(pid, m_tiles * n_tiles), m_tiles, n_tiles, tm, tn);
}

}  // namespace ave
