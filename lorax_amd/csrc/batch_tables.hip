// Host-side builder of the per-batch routing tables - no device code in this file.
//
// Restates, for all layer types of a batch at once, what the reference computes per layer type and per
// step in Python: find_segments (lorax_server/utils/segments.py:6-34), the grouping of segments by LoRA
// rank and the per-group pointer tables, segment bounds and per-token indices of BatchLoraWeights.load
// (lorax_server/adapters/lora.py:253-396), plus the routing plan of the batched BGMV launches.  Everything
// goes into ONE packed buffer that the caller uploads with a single host-to-device copy; the reference
// issues several small copies per layer type and rank.
#include <algorithm>
#include <cstring>
#include <vector>

#include "kernels.h"
#include "sgmv_tile_plan.h"

namespace {

constexpr int kPlanGroup = 4;   // tokens per routing-plan record
constexpr int kBgmvMaxRank = 128;  // BGMV_MAX_RANK, lorax_server/utils/punica.py:39
// Decode tokens inside a prefill batch are segments of one row (a speculating request: a few).  The segment
// kernels give every such segment a row tile of its own; the per-token kernels stream an adapter's weights at a
// higher rate and once for up to kPlanGroup rows.  A rank group with at least kMinShortSegments segments of at
// most kShortSegmentRows rows therefore gets them listed last in its tables and, besides, as a routing plan.
constexpr int kShortSegmentRows = 4;
constexpr int kMinShortSegments = 32;

struct Packer {
  char* base;
  int64_t capacity;
  int64_t used = 0;
  // Reserves `bytes` (16-byte aligned, the padding zeroed); returns the offset.  Keeps counting past the
  // capacity so that the caller learns the size it needs.
  int64_t reserve(int64_t bytes) {
    const int64_t off = used;
    used += (bytes + 15) / 16 * 16;
    if (used <= capacity && used > off + bytes) std::memset(base + off + bytes, 0, used - off - bytes);
    return off;
  }
  template <typename T>
  T* at(int64_t off) { return used <= capacity ? reinterpret_cast<T*>(base + off) : nullptr; }
};

const lorax_adapter_entry_t* find_entry(const lorax_adapter_entry_t* first, int32_t count, int64_t adapter) {
  const lorax_adapter_entry_t* last = first + count;
  const lorax_adapter_entry_t* it =
      std::lower_bound(first, last, adapter, [](const lorax_adapter_entry_t& e, int64_t a) { return e.adapter < a; });
  return (it != last && it->adapter == adapter) ? it : nullptr;
}

}  // namespace

extern "C" int lorax_build_batch_tables(const int64_t* adapter_indices, int64_t num_tokens,
                                        const lorax_adapter_entry_t* entries, const int32_t* entry_counts,
                                        int32_t num_layer_types, int32_t prefill, int32_t* segment_bounds,
                                        int64_t* segment_owners, int32_t* num_segments_out, void* packed,
                                        int64_t packed_capacity, int64_t* packed_bytes, lorax_table_group_t* groups,
                                        int32_t group_capacity, int32_t* num_groups_out) {
  if (num_tokens < 0 || num_layer_types < 0 || (num_tokens > 0 && adapter_indices == nullptr) ||
      segment_bounds == nullptr || segment_owners == nullptr || num_segments_out == nullptr ||
      packed_bytes == nullptr || num_groups_out == nullptr || (num_layer_types > 0 && entry_counts == nullptr))
    return LORAX_EINVAL;

  // Runs of equal adapter index (segments.py:6-34): bounds[0] = 0, a bound at every change, bounds[S] = T.
  int32_t num_segments = 0;
  segment_bounds[0] = 0;
  for (int64_t t = 0; t < num_tokens; ++t) {
    if (t == 0 || adapter_indices[t] != adapter_indices[t - 1]) {
      segment_bounds[num_segments] = static_cast<int32_t>(t);
      segment_owners[num_segments] = adapter_indices[t];
      ++num_segments;
    }
  }
  segment_bounds[num_segments] = static_cast<int32_t>(num_tokens);
  *num_segments_out = num_segments;

  Packer pack{static_cast<char*>(packed), packed != nullptr ? packed_capacity : 0};
  int32_t num_groups = 0;
  std::vector<const lorax_adapter_entry_t*> seg_entry(num_segments);
  std::vector<int32_t> group_of_rank;          // ranks in order of first appearance
  std::vector<std::vector<int32_t>> group_segs;  // segments of each rank group
  std::vector<int32_t> slot_of_seg(num_segments);
  std::vector<int32_t> token_seg(num_tokens);
  std::vector<int32_t> slot_count, slot_begin, slot_fill, slot_order, toks_by_slot(num_tokens), entry_first;
  std::vector<int64_t> entry_rows;
  std::vector<int32_t> tile_starts, tile_ends;
  std::vector<lorax_sgmv_tile_t> tile_buf;
  for (int32_t s = 0; s < num_segments; ++s)
    for (int32_t t = segment_bounds[s]; t < segment_bounds[s + 1]; ++t) token_seg[t] = s;

  const lorax_adapter_entry_t* type_entries = entries;
  for (int32_t lt = 0; lt < num_layer_types; ++lt) {
    const int32_t count = entry_counts[lt];
    // segments covered by an adapter that has weights for this layer type
    int max_rank = 0;
    bool any = false;
    for (int32_t s = 0; s < num_segments; ++s) {
      seg_entry[s] = count > 0 ? find_entry(type_entries, count, segment_owners[s]) : nullptr;
      if (seg_entry[s] != nullptr) {
        any = true;
        max_rank = std::max(max_rank, static_cast<int>(seg_entry[s]->rank));
      }
    }
    const lorax_adapter_entry_t* type_first = type_entries;
    type_entries += count;
    if (!any) continue;
    const bool use_sgmv = prefill != 0 || max_rank > kBgmvMaxRank;  // lora.py:311

    group_of_rank.clear();
    group_segs.clear();
    for (int32_t s = 0; s < num_segments; ++s) {
      if (seg_entry[s] == nullptr) continue;
      const int32_t rank = seg_entry[s]->rank;
      size_t g = 0;
      while (g < group_of_rank.size() && group_of_rank[g] != rank) ++g;
      if (g == group_of_rank.size()) {
        group_of_rank.push_back(rank);
        group_segs.emplace_back();
      }
      group_segs[g].push_back(s);
    }

    for (size_t g = 0; g < group_of_rank.size(); ++g) {
      std::vector<int32_t>& segs = group_segs[g];
      const int32_t n = static_cast<int32_t>(segs.size());
      // Segment tables: the order of a group's segments is free.  The segments of one adapter are put next to
      // each other: their tiles then run back to back on one XCD and the second one finds the adapter's
      // weights in L2 - decode tokens inside a prefill batch are one-row segments, and an adapter that serves
      // several of them would otherwise be streamed once per token.  Adapters with the most rows come first,
      // so that the long tiles of a launch start early.  Stable: (rows of the adapter, descending; adapter).
      int32_t n_short = 0;
      bool split = false;
      if (use_sgmv) {
        // rows per adapter, indexed by the adapter's position in this layer type's entry list
        entry_rows.assign(count, 0);
        for (int32_t x : segs) entry_rows[seg_entry[x] - type_first] += segment_bounds[x + 1] - segment_bounds[x];
        std::vector<int64_t> rows_of(num_segments, 0);
        for (int32_t x : segs) rows_of[x] = entry_rows[seg_entry[x] - type_first];
        for (int32_t x : segs) n_short += segment_bounds[x + 1] - segment_bounds[x] <= kShortSegmentRows;
        split = n_short >= kMinShortSegments;
        std::stable_sort(segs.begin(), segs.end(), [&](int32_t x, int32_t y) {
          if (split) {  // long segments first, short ones after them
            const bool sx = segment_bounds[x + 1] - segment_bounds[x] <= kShortSegmentRows;
            const bool sy = segment_bounds[y + 1] - segment_bounds[y] <= kShortSegmentRows;
            if (sx != sy) return sy;
          }
          if (rows_of[x] != rows_of[y]) return rows_of[x] > rows_of[y];
          return segment_owners[x] < segment_owners[y];
        });
      }
      lorax_table_group_t desc{};
      desc.layer_type = lt;
      desc.rank = group_of_rank[g];
      desc.use_sgmv = use_sgmv ? 1 : 0;
      desc.num_segments = n;
      desc.a_ptr_off = pack.reserve(static_cast<int64_t>(n) * 8);
      desc.b_ptr_off = pack.reserve(static_cast<int64_t>(n) * 8);
      if (int64_t* a = pack.at<int64_t>(desc.a_ptr_off)) {
        int64_t* b = pack.at<int64_t>(desc.b_ptr_off);
        for (int32_t i = 0; i < n; ++i) {
          a[i] = seg_entry[segs[i]]->a_addr;
          b[i] = seg_entry[segs[i]]->b_addr;
        }
      }
      desc.starts_off = desc.ends_off = desc.indices_off = desc.plan_off = -1;
      desc.shrink_tiles_off = desc.expand_tiles_off = -1;
      desc.num_long_segments = n;
      if (use_sgmv) {
        desc.starts_off = pack.reserve(static_cast<int64_t>(n) * 4);
        desc.ends_off = pack.reserve(static_cast<int64_t>(n) * 4);
        if (int32_t* st = pack.at<int32_t>(desc.starts_off)) {
          int32_t* en = pack.at<int32_t>(desc.ends_off);
          for (int32_t i = 0; i < n; ++i) {
            st[i] = segment_bounds[segs[i]];
            en[i] = segment_bounds[segs[i] + 1];
          }
        }
        if (split) {
          // Routing plan of the short segments' rows: the segments of one adapter are neighbours in the table
          // (the sort above), in token order; their rows are cut into records of up to kPlanGroup.
          const int32_t n_long = n - n_short;
          desc.num_long_segments = n_long;
          int32_t chunks = 0;
          for (int32_t i = n_long; i < n;) {
            int32_t rows = 0, j = i;
            for (; j < n && seg_entry[segs[j]] == seg_entry[segs[i]]; ++j)
              rows += segment_bounds[segs[j] + 1] - segment_bounds[segs[j]];
            chunks += (rows + kPlanGroup - 1) / kPlanGroup;
            i = j;
          }
          desc.num_chunks = chunks;
          desc.plan_off = pack.reserve(static_cast<int64_t>(chunks) * lorax::kPlanRecordWords * 8);
          if (int64_t* rec = pack.at<int64_t>(desc.plan_off)) {
            for (int32_t i = n_long; i < n;) {
              const lorax_adapter_entry_t* e = seg_entry[segs[i]];
              int cnt = 0;
              auto flush = [&]() {
                rec[0] = cnt;
                for (int q = cnt; q < kPlanGroup; ++q) rec[1 + q] = rec[1];
                rec[5] = e->a_addr;
                rec[6] = e->b_addr;
                rec[7] = 0;
                rec += lorax::kPlanRecordWords;
                cnt = 0;
              };
              int32_t j = i;
              for (; j < n && seg_entry[segs[j]] == e; ++j)
                for (int32_t t = segment_bounds[segs[j]]; t < segment_bounds[segs[j] + 1]; ++t) {
                  rec[1 + cnt++] = t;
                  if (cnt == kPlanGroup) flush();
                }
              if (cnt > 0) flush();
              i = j;
            }
          }
        }
        // Row-tile plans of the segments the segment kernels take (the long ones, when the short ones have a
        // routing plan): the lengths are at hand, so no workgroup has to search the tables.
        {
          tile_starts.resize(desc.num_long_segments);
          tile_ends.resize(desc.num_long_segments);
          for (int32_t i = 0; i < desc.num_long_segments; ++i) {
            tile_starts[i] = segment_bounds[segs[i]];
            tile_ends[i] = segment_bounds[segs[i] + 1];
          }
          const std::vector<lorax::SegmentSpan> live =
              lorax::live_segments(tile_starts.data(), tile_ends.data(), desc.num_long_segments, num_tokens);
          tile_buf.clear();
          desc.shrink_tile_rows = lorax::plan_shrink_tiles(live, tile_buf, desc.rank, lorax::tuning().shrink_rows);
          desc.num_shrink_tiles = static_cast<int32_t>(tile_buf.size());
          desc.shrink_tiles_off = pack.reserve(static_cast<int64_t>(tile_buf.size()) * sizeof(lorax_sgmv_tile_t));
          if (lorax_sgmv_tile_t* out = pack.at<lorax_sgmv_tile_t>(desc.shrink_tiles_off))
            std::copy(tile_buf.begin(), tile_buf.end(), out);
          tile_buf.clear();
          desc.expand_tile_rows = lorax::plan_expand_tiles(live, tile_buf);
          desc.num_expand_tiles = static_cast<int32_t>(tile_buf.size());
          desc.expand_tiles_off = pack.reserve(static_cast<int64_t>(tile_buf.size()) * sizeof(lorax_sgmv_tile_t));
          if (lorax_sgmv_tile_t* out = pack.at<lorax_sgmv_tile_t>(desc.expand_tiles_off))
            std::copy(tile_buf.begin(), tile_buf.end(), out);
        }
      } else {
        // slot of a token = position of the FIRST segment of its adapter inside this group's pointer slice
        // (lora.py:354-366); tokens of other ranks, of adapters without weights here and of no adapter: -1.
        std::fill(slot_of_seg.begin(), slot_of_seg.end(), -1);
        entry_first.assign(count, -1);  // first position of an adapter in the group, by entry position
        for (int32_t i = 0; i < n; ++i) {
          int32_t& first = entry_first[seg_entry[segs[i]] - type_first];
          if (first < 0) first = i;
          slot_of_seg[segs[i]] = first;
        }
        desc.indices_off = pack.reserve(num_tokens * 8);
        int64_t* idx = pack.at<int64_t>(desc.indices_off);
        // chunks: tokens of one slot, in token order, cut into groups of kPlanGroup; slots in order of their
        // first token.  Counting sort of the tokens by slot (flat arrays, no allocation per slot).
        slot_count.assign(n, 0);
        slot_order.clear();
        for (int64_t t = 0; t < num_tokens; ++t) {
          const int32_t slot = slot_of_seg[token_seg[t]];
          if (idx != nullptr) idx[t] = slot;
          if (slot >= 0 && slot_count[slot]++ == 0) slot_order.push_back(slot);
        }
        slot_begin.assign(n, 0);
        int32_t chunks = 0, placed = 0;
        for (int32_t slot : slot_order) {
          slot_begin[slot] = placed;
          placed += slot_count[slot];
          chunks += (slot_count[slot] + kPlanGroup - 1) / kPlanGroup;
        }
        desc.num_chunks = chunks;
        desc.plan_off = pack.reserve(static_cast<int64_t>(chunks) * lorax::kPlanRecordWords * 8);
        if (int64_t* rec = pack.at<int64_t>(desc.plan_off)) {
          slot_fill = slot_begin;
          for (int64_t t = 0; t < num_tokens; ++t) {
            const int32_t slot = slot_of_seg[token_seg[t]];
            if (slot >= 0) toks_by_slot[slot_fill[slot]++] = static_cast<int32_t>(t);
          }
          for (int32_t slot : slot_order) {
            const int32_t* toks = toks_by_slot.data() + slot_begin[slot];
            const int32_t total = slot_count[slot];
            for (int32_t i = 0; i < total; i += kPlanGroup) {
              const int cnt = std::min<int32_t>(kPlanGroup, total - i);
              rec[0] = cnt;
              for (int q = 0; q < kPlanGroup; ++q) rec[1 + q] = toks[q < cnt ? i + q : i];
              rec[5] = seg_entry[segs[slot]]->a_addr;
              rec[6] = seg_entry[segs[slot]]->b_addr;
              rec[7] = 0;
              rec += lorax::kPlanRecordWords;
            }
          }
        }
      }
      if (groups != nullptr && num_groups < group_capacity) groups[num_groups] = desc;
      ++num_groups;
    }
  }
  *packed_bytes = pack.used;
  *num_groups_out = num_groups;
  if (pack.used > pack.capacity || num_groups > group_capacity || (groups == nullptr && num_groups > 0))
    return LORAX_ESPACE;
  return LORAX_OK;
}

extern "C" int lorax_sgmv_plan_tiles(const int32_t* s_start, const int32_t* s_end, int32_t num_segments,
                                     int64_t num_tokens, int32_t kind, int32_t rank, lorax_sgmv_tile_t* tiles,
                                     int32_t capacity, int32_t* num_tiles, int32_t* tile_rows) {
  if (num_segments < 0 || num_tokens < 0 || num_tiles == nullptr || tile_rows == nullptr ||
      (num_segments > 0 && (s_start == nullptr || s_end == nullptr)) ||
      (kind != LORAX_TILES_SHRINK && kind != LORAX_TILES_EXPAND))
    return LORAX_EINVAL;
  const std::vector<lorax::SegmentSpan> live = lorax::live_segments(s_start, s_end, num_segments, num_tokens);
  std::vector<lorax_sgmv_tile_t> out;
  *tile_rows = kind == LORAX_TILES_SHRINK ? lorax::plan_shrink_tiles(live, out, rank, lorax::tuning().shrink_rows)
                                          : lorax::plan_expand_tiles(live, out);
  *num_tiles = static_cast<int32_t>(out.size());
  if (tiles == nullptr || static_cast<size_t>(capacity < 0 ? 0 : capacity) < out.size()) return out.empty() ? LORAX_OK : LORAX_ESPACE;
  std::copy(out.begin(), out.end(), tiles);
  return LORAX_OK;
}
