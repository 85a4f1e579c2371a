// Device-side tile scheduler shared by the SGMV kernels.
//
// Segment bounds live in device memory (the reference passes s_start/s_end tensors and
// never syncs, punica.py:170-196), so the host cannot know how many row tiles a launch
// has.  Row tiles of `rows_per_tile` rows are numbered segment by segment; every
// workgroup maps a tile number to (segment, rows) by a wave-parallel prefix sum over
// the segment lengths.  Empty and negative segments (sgmv_cutlass.cuh:39-44) get zero
// tiles, and bounds are clamped to [0, num_tokens) so no row outside x/y is touched.
#pragma once

#include "common.h"

namespace lorax {

struct RowTile {
  int seg;      // segment (problem) index
  int row0;     // first row of the tile
  int row_end;  // one past the last row of the tile (<= end of segment)
};

// Wave-uniform.  Returns false when `tile` is past the last tile of the launch.
__device__ __forceinline__ bool find_row_tile(const int32_t* __restrict__ s_start,
                                              const int32_t* __restrict__ s_end,
                                              int num_segments, int num_tokens,
                                              int rows_per_tile, int tile, RowTile& out) {
  const int lane = lane_id();
  int base = 0;
  for (int seg0 = 0; seg0 < num_segments; seg0 += kWave) {
    const int seg = seg0 + lane;
    int s = 0, e = 0;
    if (seg < num_segments) {
      s = max(s_start[seg], 0);
      e = min(s_end[seg], num_tokens);
    }
    const int len = max(e - s, 0);
    const int nt = (len + rows_per_tile - 1) / rows_per_tile;
    int inc = nt;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const int t = __shfl_up(inc, d, kWave);
      if (lane >= d) inc += t;
    }
    const int chunk_total = __shfl(inc, kWave - 1, kWave);
    const int rel = tile - base;
    if (rel < chunk_total) {
      const bool hit = (rel >= inc - nt) && (rel < inc);
      const uint64_t mask = __ballot(hit);
      const int src = __ffsll(static_cast<unsigned long long>(mask)) - 1;
      const int ti = rel - __shfl(inc - nt, src, kWave);
      const int s_f = __shfl(s, src, kWave);
      const int e_f = __shfl(e, src, kWave);
      out.seg = seg0 + src;
      out.row0 = s_f + ti * rows_per_tile;
      out.row_end = min(e_f, out.row0 + rows_per_tile);
      return true;
    }
    base += chunk_total;
  }
  return false;
}

}  // namespace lorax
