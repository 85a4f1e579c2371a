// Host-side cutting of the segments of an SGMV launch into row tiles (no device code).
//
// The segment kernels find their row tiles on the device when all they are given is the reference's segment
// tables (s_start / s_end in device memory, punica.py:170-196): every workgroup scans the tables.  A caller that
// has the segment lengths on the host - the table builder does - can hand over the finished list instead: one
// 16-byte record per tile, read by its workgroup with one scalar load.  The host also knows the exact number of
// tiles, so the grid holds no workgroup without work, and it can cut every segment into tiles of equal height.
// (The reference's cutlass path precomputes its problem table the same way, sgmv/sgmv_cutlass.cuh:30-52.)
#pragma once

#include <stdint.h>

#include <algorithm>
#include <vector>

#include "../../include/lorax_hip.h"

namespace lorax {

constexpr int kShrinkTileRowsMax = 64;   // the LDS-staged shrink's buffers hold up to four 16-row blocks
constexpr int kExpandTileRows = 256;     // nominal height of an expand tile
constexpr int kExpandTileRowsMax = kExpandTileRows + kExpandTileRows / 8 + 16;  // with a merged remainder

struct SegmentSpan {
  int32_t seg, start, end;  // clamped to [0, num_tokens], end > start
};

inline std::vector<SegmentSpan> live_segments(const int32_t* s_start, const int32_t* s_end, int32_t num_segments,
                                              int64_t num_tokens) {
  std::vector<SegmentSpan> out;
  out.reserve(num_segments > 0 ? num_segments : 0);
  for (int32_t i = 0; i < num_segments; ++i) {
    const int64_t s = std::max<int64_t>(s_start[i], 0);
    const int64_t e = std::min<int64_t>(s_end[i], num_tokens);
    if (e > s) out.push_back({i, static_cast<int32_t>(s), static_cast<int32_t>(e)});
  }
  return out;
}

inline int64_t tiles_at_height(const std::vector<SegmentSpan>& segs, int rows) {
  int64_t n = 0;
  for (const SegmentSpan& s : segs) n += (s.end - s.start + rows - 1) / rows;
  return n;
}

// Height of the shrink's row tiles.  A launch streams at the rate of the CUs that hold a workgroup, so with
// fewer tiles than the 256 CUs the tiles are made lower until there are about as many (the same rule the
// launcher applies to its upper bound of the tile count when it has no plan; here the count is exact).  Batches
// of a thousand rows or so get 16- or 32-row tiles and are cut along the hidden dimension as well (the launcher's
// K parts).  A workgroup stages rank rows of A next to its tile's rows of x, so tiles are not lowered below a
// quarter of the rank: measured on a 4096-row run at rank 128, 32-row tiles in two K parts (256 workgroups) take
// 41 us where 16-row tiles (256 workgroups, twice the A traffic) take 53 us.  Returns a multiple of 16 in [16, 64].
inline int shrink_tile_rows(const std::vector<SegmentSpan>& segs, int64_t rows_total, int rank, int forced_rows = 0) {
  if (forced_rows > 0) return std::min(64, (forced_rows + 15) / 16 * 16);  // tuning builds only
  if (segs.empty()) return 16;
  const int64_t avg_len = rows_total / static_cast<int64_t>(segs.size());
  int mblk = 4;
  while (mblk > 1 && (tiles_at_height(segs, mblk * 16) < 128 || mblk * 8 > avg_len)) mblk /= 2;
  int rows = mblk * 16;
  const int floor_rows = std::max(16, (rank > 0 ? rank : 64) / 4);
  while (rows - 16 >= floor_rows && tiles_at_height(segs, rows - 16) <= 256) rows -= 16;
  return rows;
}

// A segment of `len` rows as `nt` tiles of equal height (to the row): tile i covers [len * i / nt, len * (i + 1) / nt).
inline void cut_evenly(const SegmentSpan& s, int nt, std::vector<lorax_sgmv_tile_t>& out) {
  const int64_t len = s.end - s.start;
  for (int i = 0; i < nt; ++i) {
    lorax_sgmv_tile_t t;
    t.seg = s.seg;
    t.row0 = s.start + static_cast<int32_t>(len * i / nt);
    t.row_end = s.start + static_cast<int32_t>(len * (i + 1) / nt);
    t.index = i;
    out.push_back(t);
  }
}

inline int plan_shrink_tiles(const std::vector<SegmentSpan>& segs, std::vector<lorax_sgmv_tile_t>& out, int rank,
                             int forced_rows = 0) {
  int64_t rows_total = 0;
  for (const SegmentSpan& s : segs) rows_total += s.end - s.start;
  const int rows = shrink_tile_rows(segs, rows_total, rank, forced_rows);
  for (const SegmentSpan& s : segs) cut_evenly(s, (s.end - s.start + rows - 1) / rows, out);
  return rows;
}

// Expand tiles: nominally 256 rows; a remainder of at most an eighth of the segment's full tiles is shared out
// among them instead of becoming a tile of its own (a tile's prologue costs as much as a hundred rows), and the
// segment's tiles get equal heights in 16-row blocks - the rule of the device-side search (merged_tile_count).
inline int plan_expand_tiles(const std::vector<SegmentSpan>& segs, std::vector<lorax_sgmv_tile_t>& out) {
  for (const SegmentSpan& s : segs) {
    const int len = s.end - s.start;
    const int full = len / kExpandTileRows;
    const int rem = len - full * kExpandTileRows;
    const int nt = (full >= 1 && rem * 8 <= full * kExpandTileRows) ? full : full + (rem > 0 ? 1 : 0);
    const int blocks = (len + 15) / 16;
    for (int i = 0; i < nt; ++i) {
      lorax_sgmv_tile_t t;
      t.seg = s.seg;
      t.row0 = s.start + 16 * static_cast<int32_t>(static_cast<int64_t>(i) * blocks / nt);
      t.row_end = std::min<int32_t>(s.end, s.start + 16 * static_cast<int32_t>(static_cast<int64_t>(i + 1) * blocks / nt));
      t.index = i;
      out.push_back(t);
    }
  }
  return kExpandTileRowsMax;
}

}  // namespace lorax
