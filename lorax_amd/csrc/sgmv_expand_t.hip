// SGMV expand over the transposed B stack: y[s:e, off:off+h_out] += T(v[s:e, :r] @ B_i), with B_i
// stored as B_i^T = [h_out, r] (the layout the decode path keeps resident anyway).
//
// Same arithmetic and rounding as sgmv_expand.hip.  The MFMA product is v (16 rows of a block, first
// operand) times B (second operand), and with B^T in memory the second operand needs no transposition:
// the 16 bytes B^T[column(j, c)][32 s + 8 g ...] that lane (c, g) of accumulator j needs come straight from
// global memory into registers (fetched by the lane that makes the access contiguous and handed over with
// a cross-lane move, see the kernel).  There is no LDS staging, no barrier and no LDS gather in a tile's
// prologue - which, for the short segments a prefill batch is full of, took longer than the rows
// themselves.
//
// The columns of a wave's panel are dealt to the accumulators so that a lane ends up with NJ ADJACENT
// columns of four rows (see the kernel).  A y access of the wave is then four whole runs of 32 * NJ
// bytes, one per row, and the texture path handles it as a few cache lines.  (With the product the other
// way round - B^T first, v second - a lane holds 8 adjacent columns of ONE row and neighbouring lanes
// hold different rows: every 16-byte piece is then a separate cache-line lookup, 64 per instruction, and
// the kernel is bound by the address path of the CU at 60 % of what it reaches now; counters:
// TA_ADDR_STALLED_BY_TC_CYCLES at 60 % and TA_BUSY at 80 % of the kernel's duration.)
//
// Work split: a workgroup owns one row tile and 4 * panels_per_wave column panels of 16 * NJ; wave w takes
// panels w, w + 4, ... and walks ALL 16-row blocks of the tile for each.  The tile search runs once per
// workgroup.  There is no separate path for segments of a few rows: rows past the tile's end are clamped
// for loads and predicated for stores, and MFMA work on padding is free in a kernel that waits on memory.
#include "kernels.h"
#include "sgmv_tiles.h"

namespace lorax {

constexpr int kExpTWaves = 4;
constexpr int kExpTThreads = kExpTWaves * kWave;
constexpr int kExpTStages = 2;  // register stages of the row-block pipeline (a third one costs occupancy)
constexpr int kExpTLaneCols = 4;  // adjacent output columns per lane

// NJ accumulators per wave, a panel of 16 * NJ output columns.  Accumulator j stands for the columns
// n0 + NJ * c + j (c = lane & 15), so a lane ends up with NJ ADJACENT columns of the rows 4g .. 4g + 3
// (g = lane >> 4) of a 16-row block, and the 16 lanes of one g cover 32 * NJ contiguous bytes of a row.
template <typename D, int KS, int NJ>
__global__ __launch_bounds__(kExpTThreads) void sgmv_expand_t_kernel(
    typename D::E* __restrict__ Y, const typename D::E* __restrict__ V,
    const int64_t* __restrict__ W, const int32_t* __restrict__ s_start,
    const int32_t* __restrict__ s_end, int num_segments, int num_tokens, int r, int h_out,
    int64_t y_offset, int64_t y_stride, int64_t layer_idx, int rows_per_tile, int panels_per_wave,
    int tile_slots, int accumulate_into_y, const TileList plan) {
  using E = typename D::E;
  using vec8 = typename D::vec8;
  typedef E yvec __attribute__((ext_vector_type(NJ)));
  constexpr int kCols = 16 * NJ;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);  // wave-uniform, in a scalar register
  const int c = lane & 15;
  const int g = lane >> 4;
  const int num_panels = (h_out + kCols - 1) / kCols;
  // Workgroup numbering: row tiles fastest, then panel groups, and consecutive numbers on one XCD.  The
  // row tiles of a long segment read the same panels of B^T; as neighbours on one XCD they find them in
  // its L2 instead of fetching them once per tile.
  const int vid = static_cast<int>(xcd_virtual_id());
  const int panel0 = (vid / tile_slots) * kExpTWaves * panels_per_wave;
  const bool acc_y = accumulate_into_y != 0;

  // MFMA operand layout: lane g * 16 + c holds the eight k values 32 s + 8 g ... of operand row / column c.
  // Fetched that way, neighbouring lanes read different rows, r * 2 bytes apart, and every 16-byte piece
  // is a cache-line lookup of its own.  So the operands are FETCHED with lane l taking piece l & 3 of row
  // l >> 2 - a quad of lanes reads 64 contiguous bytes - and then change lanes through the LDS crossbar
  // (ds_bpermute, no LDS memory): the lane g * 16 + c takes the registers of lane 4 c + g.
  const int lc = lane >> 2;
  const int from_lane = (c * 4 + g) * 4;  // ds_bpermute addresses lanes in bytes
  auto to_operand_lanes = [&](vec8 fetched) {
    const u32x4 raw = __builtin_bit_cast(u32x4, fetched);
    u32x4 mine;
#pragma unroll
    for (int d = 0; d < 4; ++d)
      mine[d] = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(from_lane, static_cast<int>(raw[d])));
    return __builtin_bit_cast(vec8, mine);
  };
  bool k_ok[KS];  // of the operand lane: chunks beyond the rank are zeroed after the exchange
  int l_off[KS];  // of the fetching lane: chunks beyond the rank are fetched from chunk 0
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    k_ok[s] = s * 32 + g * 8 < r;
    l_off[s] = s * 32 + (lane & 3) * 8 < r ? s * 32 + (lane & 3) * 8 : 0;
  }

  const int64_t pre_w = preload_segment_entry(W, num_segments);
  for (int tile = vid % tile_slots;; tile += tile_slots) {
    RowTile rt;
    // small remainders are merged into the segment's other tiles: a tile's prologue (the search and the panel
    // operands) costs as much as a hundred rows
    if (!get_row_tile<true>(plan, s_start, s_end, num_segments, num_tokens, rows_per_tile, tile, rt)) break;
    const int64_t stack = segment_entry(pre_w, W, rt.seg);
    if (plan.records != nullptr && stack == 0) break;  // a caller's plan that names a segment without a stack
    const E* BT = reinterpret_cast<const E*>(stack) + layer_idx * h_out * static_cast<int64_t>(r);
    const int nmb = (rt.row_end - rt.row0 + 15) / 16;

    for (int pp = 0; pp < panels_per_wave; ++pp) {
      const int panel = panel0 + pp * kExpTWaves + wave;
      if (panel >= num_panels) break;
      const int n0 = panel * kCols;
      // h_out is a multiple of 8 and so is NJ * c: a lane's NJ columns are inside the matrix or outside it
      // as a whole.  Loads are unconditional: rows past the tile are clamped to its last row and a lane
      // past h_out reads the panel's first columns (both valid memory); only the stores are predicated.
      const bool col_ok = n0 + NJ * c < h_out;
      const int col = col_ok ? n0 + NJ * c : n0;
      // Addresses inside a tile: a wave-uniform 64-bit base and a 32-bit offset per lane (a tile spans at
      // most rows_per_tile * y_stride elements).
      const E* vtile = V + static_cast<int64_t>(rt.row0) * r;
      E* ytile = Y + static_cast<int64_t>(rt.row0) * y_stride + y_offset + n0;
      const uint32_t ycol = static_cast<uint32_t>(col - n0);
      const uint32_t ystride = static_cast<uint32_t>(y_stride);
      const int last = rt.row_end - rt.row0 - 1;
      auto load_block = [&](int mb, vec8(&vf)[KS], yvec(&yv)[4]) {
        // v rows are fetched like the B^T rows below: lane l takes piece l & 3 of row l >> 2 of the block, and
        // finish_block moves the pieces to the lanes the MFMA wants them in
        const uint32_t voff = static_cast<uint32_t>(min(mb * 16 + lc, last)) * static_cast<uint32_t>(r);
#pragma unroll
        for (int s = 0; s < KS; ++s) vf[s] = load8<D>(vtile + (voff + l_off[s]));
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t row = static_cast<uint32_t>(min(mb * 16 + g * 4 + i, last));
          yv[i] = *(const LORAX_GLOBAL yvec*)(ytile + (row * ystride + ycol));
        }
      };
      auto block_of = [&](int i) { return min(i, nmb - 1); };

      // first row blocks and the panel's operands go out together: one memory round trip
      vec8 vr[kExpTStages][KS];
      yvec yr[kExpTStages][4];
#pragma unroll
      for (int s = 0; s < kExpTStages - 1; ++s) load_block(block_of(s), vr[s], yr[s]);
      // B^T operands: lane l fetches piece l & 3 of the row of operand column l >> 2
      vec8 bf[NJ][KS];
      const int lcol = (n0 + NJ * lc < h_out) ? n0 + NJ * lc : n0;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
#pragma unroll
        for (int s = 0; s < KS; ++s)
          bf[j][s] = keep_if<D>(k_ok[s], to_operand_lanes(load8<D>(BT + static_cast<int64_t>(lcol + j) * r + l_off[s])));
      }

      auto finish_block = [&](bool live, int mb, vec8(&vf)[KS], yvec(&yv)[4]) {
        f32x4 acc[NJ];
#pragma unroll
        for (int s = 0; s < KS; ++s) vf[s] = to_operand_lanes(vf[s]);
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
          acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s = 0; s < KS; ++s) acc[j] = D::mfma16(vf[s], bf[j][s], acc[j]);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int row = mb * 16 + g * 4 + i;
          yvec out;
#pragma unroll
          for (int j = 0; j < NJ; ++j)  // overwrite mode: the old y counts as zero
            out[j] = accumulate<D>(acc_y ? yv[i][j] : static_cast<E>(0.0f), acc[j][i]);
          if (live && col_ok && row <= last)
            *(LORAX_GLOBAL yvec*)(ytile + (static_cast<uint32_t>(row) * ystride + ycol)) = out;
        }
      };

      // Ring of kExpTStages register stages with static indices: the y and v loads of the next
      // kExpTStages - 1 blocks are in flight while one block is multiplied and stored.  Surplus
      // trips of the last round re-load the last block and store nothing.
      for (int i = 0; i < nmb; i += kExpTStages) {
#pragma unroll
        for (int s = 0; s < kExpTStages; ++s) {
          constexpr int kAhead = kExpTStages - 1;
          load_block(block_of(i + s + kAhead), vr[(s + kAhead) % kExpTStages], yr[(s + kAhead) % kExpTStages]);
          __builtin_amdgcn_sched_barrier(0);
          finish_block(i + s < nmb, block_of(i + s), vr[s], yr[s]);
        }
      }
    }
  }
}

template <typename D, int KS, int NJ>
static hipError_t launch_expand_t_ks(const SgmvArgs& a, hipStream_t stream) {
  // 256-row tiles: the prologue is one memory round trip, so taller tiles buy nothing and even out worse
  int rows_per_tile = 256;
  if (tuning().expand_rows > 0) rows_per_tile = (tuning().expand_rows + 15) / 16 * 16;
  // The kernel addresses a tile with 32-bit element offsets, and a tile is up to 9/8 * rows_per_tile + 15 rows
  // high (merged remainders): rows of more than 2^23 elements get lower tiles.
  while (rows_per_tile > 16 && a.y_stride * (rows_per_tile + rows_per_tile / 8 + 16) >= (1ll << 32)) rows_per_tile /= 2;
  if (a.y_stride * (rows_per_tile + rows_per_tile / 8 + 16) >= (1ll << 32)) return hipErrorInvalidValue;
  // With the caller's tile plan the tile count is exact (no workgroup without work) and a tile is at most
  // tile_rows high; the plan is ignored when its tiles would overflow the 32-bit offsets.
  const bool planned = a.tiles != nullptr && a.num_tiles > 0 && a.tile_rows >= 1 && tuning().expand_rows == 0 &&
                       a.y_stride * static_cast<int64_t>(a.tile_rows) < (1ll << 32);
  const int64_t tiles = planned ? a.num_tiles : (a.num_tokens + rows_per_tile - 1) / rows_per_tile + a.num_segments;
  const TileList plan{planned ? a.tiles : nullptr, planned ? a.num_tiles : 0, planned ? a.tile_rows : 0};
  constexpr int kCols = 16 * NJ;
  const int num_panels = (a.d_out + kCols - 1) / kCols;
  // Panels per wave: more of them amortise the tile search, fewer give more workgroups; keep a few
  // thousand workgroups in the launch.
  int ppw = 4;
  while (ppw > 1 && tiles * ((num_panels + kExpTWaves * ppw - 1) / (kExpTWaves * ppw)) < 4096) ppw /= 2;
  if (tuning().expand_panels > 0) ppw = tuning().expand_panels;
  const int64_t panel_groups = (num_panels + kExpTWaves * ppw - 1) / (kExpTWaves * ppw);
  const int tile_slots = static_cast<int>(tiles < 65535 ? tiles : 65535);
  dim3 grid(static_cast<unsigned>(panel_groups * tile_slots));
  hipLaunchKernelGGL((sgmv_expand_t_kernel<D, KS, NJ>), grid, dim3(kExpTThreads), 0, stream,
                     static_cast<typename D::E*>(a.y), static_cast<const typename D::E*>(a.x), a.w_ptrs, a.s_start,
                     a.s_end, a.num_segments, static_cast<int>(a.num_tokens), a.d_in, a.d_out, a.y_offset,
                     a.y_stride, a.layer_idx, rows_per_tile, ppw, tile_slots, a.accumulate, plan);
  return hipGetLastError();
}

template <typename D>
static hipError_t launch_expand_t_dtype(const SgmvArgs& a, hipStream_t stream) {
  switch ((a.d_in + 31) / 32) {
    case 1:
      return launch_expand_t_ks<D, 1, kExpTLaneCols>(a, stream);
    case 2:
      return launch_expand_t_ks<D, 2, kExpTLaneCols>(a, stream);
    case 3:
      return launch_expand_t_ks<D, 3, kExpTLaneCols>(a, stream);
    case 4:
      return launch_expand_t_ks<D, 4, kExpTLaneCols>(a, stream);
    default:
      return hipErrorInvalidValue;
  }
}

hipError_t launch_sgmv_expand_t(const SgmvArgs& a, hipStream_t stream) {
  return a.dtype == LORAX_F16 ? launch_expand_t_dtype<F16>(a, stream) : launch_expand_t_dtype<BF16>(a, stream);
}

}  // namespace lorax
