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

// Workgroup id -> tile.  Groups of 8 consecutive bands are dealt one band per XCD (workgroup pid runs on
// XCD pid % 8, so tile q of a group goes to band q % 8): every XCD walks its own band with its panels
// in its own L2, and all XCDs work on neighbouring bands at the same time, so what they stream stays
// small enough for the last-level cache (in the grouped GEMM: the weights of one or two experts
// instead of all of them).  What is left after the last complete group of 8 bands is split into one
// contiguous range per XCD.  Bijection on [0, m_tiles * n_tiles).
AVE_HD void map_tile(int pid, int m_tiles, int n_tiles, int& tm, int& tn) {
  const int per_band = kGroupM * n_tiles, per_group = kXcds * per_band;
  const int full_m = (m_tiles / (kXcds * kGroupM)) * (kXcds * kGroupM);   // m-tiles inside complete groups
  const int base = full_m * n_tiles;
  if (pid < base) {
    const int group = pid / per_group, q = pid % per_group;
    const int band = group * kXcds + q % kXcds, in_band = q / kXcds;
    tm = band * kGroupM + in_band % kGroupM;
    tn = in_band / kGroupM;
  } else {
    banded_tile(xcd_contiguous_id(pid - base, m_tiles * n_tiles - base), m_tiles - full_m, n_tiles, tm, tn);
    tm += full_m;
  }
}

// m-tile `tm` of a grouped (MoE) GEMM: the m-tile list is the concatenation of the experts' tile lists, expert e
// owning rows [row_offsets[e], row_offsets[e+1]) in tiles of `tile_rows` rows.  Every table entry is clamped to
// [0, total_m] first and a range that is empty after clamping has no tiles, so a stale or malformed table (an end
// past total_m, a negative start, a decreasing pair) can leave rows of C unwritten but never addresses a row outside
// A or C.  Returns false when tm lies behind the last tile; otherwise expert, m_begin and m_end (0 <= m_begin <
// m_end <= total_m).  The whole table is walked whatever tm is, so that the control flow is uniform.
AVE_HD bool locate_group_tile(const int* row_offsets, int experts, int total_m, int tile_rows, int tm, int& expert,
                              int& m_begin, int& m_end) {
  int first = 0;
  bool found = false;
  for (int e = 0; e < experts; ++e) {
    int r0 = row_offsets[e], r1 = row_offsets[e + 1];
    r0 = r0 < 0 ? 0 : (r0 > total_m ? total_m : r0);
    r1 = r1 < 0 ? 0 : (r1 > total_m ? total_m : r1);
    const int nt = r1 > r0 ? (r1 - r0 + tile_rows - 1) / tile_rows : 0;
    if (!found && tm >= first && tm < first + nt) {
      expert = e;
      m_begin = r0 + (tm - first) * tile_rows;
      m_end = r1;
      found = true;
    }
    first += nt;
  }
  return found;
}

}  // namespace ave
