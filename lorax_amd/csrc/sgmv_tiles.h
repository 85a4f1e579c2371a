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
  int index;    // number of the tile inside its segment
};

// One chunk of 64 segments: lane `lane` holds the clamped bounds (s, e) of segment seg0 + lane.  If `tile`
// (counted from the first tile of the chunk, `rel`) falls into the chunk, fills `out` and returns true;
// otherwise adds the chunk's tiles to `base`.
// MERGE: a remainder that would make the segment's full tiles at most an eighth taller is shared out among them
// instead of becoming a tile of its own, and the segment's tiles get equal heights (in 16-row blocks).  For
// kernels whose tile prologue is expensive (a batch of 269-row segments cost the expand 38 % more than one of
// 256-row segments) and whose tile height is free; taller tiles than that unbalance the end of the launch.
__device__ __forceinline__ int merged_tile_count(int len, int rows_per_tile) {
  const int full = len / rows_per_tile;
  const int rem = len - full * rows_per_tile;
  return (full >= 1 && rem * 8 <= full * rows_per_tile) ? full : full + (rem > 0 ? 1 : 0);
}

template <bool MERGE = false>
__device__ __forceinline__ bool tile_in_chunk(int s, int e, int seg0, int rows_per_tile, int tile, int& base,
                                              RowTile& out) {
  const int len = max(e - s, 0);
  const int nt = MERGE ? merged_tile_count(len, rows_per_tile) : (len + rows_per_tile - 1) / rows_per_tile;
  const int inc = wave_inclusive_scan(nt);
  const int chunk_total = __builtin_amdgcn_readlane(inc, kWave - 1);
  const int rel = tile - base;
  if (rel < chunk_total) {
    const bool hit = (rel >= inc - nt) && (rel < inc);
    const uint64_t mask = __ballot(hit);
    const int src = __ffsll(static_cast<unsigned long long>(mask)) - 1;
    const int ti = rel - read_lane(inc - nt, src);
    const int s_f = read_lane(s, src);
    const int e_f = read_lane(e, src);
    out.seg = seg0 + src;
    out.index = ti;
    if (MERGE) {
      const int nt_f = read_lane(nt, src);
      const int blocks = (e_f - s_f + 15) / 16;
      out.row0 = s_f + 16 * static_cast<int>(static_cast<int64_t>(ti) * blocks / nt_f);
      out.row_end = min(e_f, s_f + 16 * static_cast<int>(static_cast<int64_t>(ti + 1) * blocks / nt_f));
    } else {
      out.row0 = s_f + ti * rows_per_tile;
      out.row_end = min(e_f, out.row0 + rows_per_tile);
    }
    return true;
  }
  base += chunk_total;
  return false;
}

// Wave-uniform.  Returns false when `tile` is past the last tile of the launch.
// The bounds of the first kTilePreload * 64 segments are all requested before the first one is looked at,
// so that a batch of a few hundred segments (decode tokens inside a prefill batch) costs one memory round
// trip instead of one per 64 segments.
constexpr int kTilePreload = 4;

template <bool MERGE = false>
__device__ __forceinline__ bool find_row_tile(const int32_t* __restrict__ s_start,
                                              const int32_t* __restrict__ s_end,
                                              int num_segments, int num_tokens,
                                              int rows_per_tile, int tile, RowTile& out) {
  if (num_segments <= 0) return false;
  const int lane = lane_id();
  int s_pre[kTilePreload], e_pre[kTilePreload];
#pragma unroll
  for (int c = 0; c < kTilePreload; ++c) {
    // unconditional loads of clamped indices: every load is in flight before the first wait
    const int seg = min(c * kWave + lane, num_segments - 1);
    s_pre[c] = s_start[seg];
    e_pre[c] = s_end[seg];
  }
  int base = 0;
#pragma unroll
  for (int c = 0; c < kTilePreload; ++c) {
    if (c * kWave >= num_segments) return false;
    const bool live = c * kWave + lane < num_segments;
    const int s = live ? max(s_pre[c], 0) : 0;
    const int e = live ? min(e_pre[c], num_tokens) : 0;
    if (tile_in_chunk<MERGE>(s, e, c * kWave, rows_per_tile, tile, base, out)) return true;
  }
  for (int seg0 = kTilePreload * kWave; seg0 < num_segments; seg0 += kWave) {
    const int seg = seg0 + lane;
    int s = 0, e = 0;
    if (seg < num_segments) {
      s = max(s_start[seg], 0);
      e = min(s_end[seg], num_tokens);
    }
    if (tile_in_chunk<MERGE>(s, e, seg0, rows_per_tile, tile, base, out)) return true;
  }
  return false;
}

// A launch's row tiles: from the caller's plan when it brought one (one 16-byte record per tile, wave-uniform
// address: a scalar load), else by the search above.  Records are clamped to the call's sizes - a wrong plan gives
// wrong results, but no access outside the call's tensors - and a record without rows ends the workgroup's walk.
struct TileList {
  const int32_t* records;  // lorax_sgmv_tile_t[num_tiles] in device memory, or null
  int num_tiles;
  int max_rows;            // no tile is higher
};

template <bool MERGE = false>
__device__ __forceinline__ bool get_row_tile(const TileList& plan, const int32_t* __restrict__ s_start,
                                             const int32_t* __restrict__ s_end, int num_segments, int num_tokens,
                                             int rows_per_tile, int tile, RowTile& out) {
  if (plan.records == nullptr) return find_row_tile<MERGE>(s_start, s_end, num_segments, num_tokens, rows_per_tile, tile, out);
  if (tile >= plan.num_tiles || num_segments <= 0) return false;
  typedef int int32x4 __attribute__((ext_vector_type(4)));
  const int32x4 rec = *reinterpret_cast<const int32x4*>(plan.records + 4 * static_cast<int64_t>(tile));
  out.seg = min(max(rec[0], 0), num_segments - 1);
  out.row0 = min(max(rec[1], 0), num_tokens);
  out.row_end = min(min(rec[2], num_tokens), out.row0 + plan.max_rows);
  out.index = rec[3];
  return out.row_end > out.row0;
}

// The stack address of a tile's segment without a memory round trip after the tile search: every lane asks for
// the table entry of "its" segment BEFORE the search (the loads travel together with the search's own), and the
// entry of the segment the search lands on is read from that lane afterwards.  Segments past the first 64 fall
// back to a load.  Table entries are only read, never dereferenced, here.
__device__ __forceinline__ int64_t preload_segment_entry(const int64_t* __restrict__ table, int num_segments) {
  return table[min(lane_id(), max(num_segments, 1) - 1)];
}
__device__ __forceinline__ int64_t segment_entry(int64_t preloaded, const int64_t* __restrict__ table, int seg) {
  if (seg >= kWave) return table[seg];
  const int src = __builtin_amdgcn_readfirstlane(seg);
  const uint32_t lo = __builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(preloaded)), src);
  const uint32_t hi = __builtin_amdgcn_readlane(static_cast<int>(static_cast<uint64_t>(preloaded) >> 32), src);
  return static_cast<int64_t>((static_cast<uint64_t>(hi) << 32) | lo);
}

}  // namespace lorax
