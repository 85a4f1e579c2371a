// SGMV expand over the transposed B stack: y[s:e, off:off+h_out] += T(v[s:e, :r] @ B_i), with B_i
// stored as B_i^T = [h_out, r] (the layout the decode path keeps resident anyway).
//
// Same arithmetic and rounding as sgmv_expand.hip (the transposed MFMA product: B^T as the first
// operand, v as the second, so that a lane ends up with 8 adjacent columns of one y row and y moves
// in 16-byte pieces), but with B^T in memory the first operand needs no transposition: lane (c, g)
// of accumulator j reads the 16 bytes B^T[column(j, c)][32 s + 8 g ...] straight from global memory,
// and the 64-column panel of a wave is one contiguous run of 64 * r * 2 bytes.  That removes the LDS
// staging, its two barriers and the 2-byte LDS gathers from every tile's prologue - which, for the
// short segments a prefill batch is full of, took longer than the rows themselves - and it makes
// the weight reads of single-row segments (decode tokens inside a prefill batch) sequential.
//
// Work split: a workgroup owns one row tile and 4 * panels_per_wave column panels of 64; wave w takes
// panels w, w + 4, ... and walks ALL 16-row blocks of the tile for each (the four waves touch 512
// adjacent bytes of every row).  The tile search runs once per workgroup.  There is no separate path
// for segments of a few rows: rows past the tile's end are clamped for loads and predicated for
// stores, and MFMA work on padding is free in a kernel that waits on memory.
#include "kernels.h"
#include "sgmv_tiles.h"

namespace lorax {

constexpr int kExpTWaves = 4;
constexpr int kExpTThreads = kExpTWaves * kWave;
constexpr int kExpTCols = 64;   // output columns per wave and panel
constexpr int kExpTStages = 3;  // register stages of the row-block pipeline

// Output column (0..63) that row `a` of the first MFMA operand of accumulator j stands for: lane
// group g = a / 4 ends up with columns [8g, 8g+8) in accumulators 0,1 and [32+8g, 32+8g+8) in 2,3.
__device__ __forceinline__ int panel_col_t(int j, int a) {
  return (j >> 1) * 32 + (a >> 2) * 8 + (j & 1) * 4 + (a & 3);
}

template <typename D, int KS>
__global__ __launch_bounds__(kExpTThreads) void sgmv_expand_t_kernel(
    typename D::E* __restrict__ Y, const typename D::E* __restrict__ V,
    const int64_t* __restrict__ W, const int32_t* __restrict__ s_start,
    const int32_t* __restrict__ s_end, int num_segments, int num_tokens, int r, int h_out,
    int64_t y_offset, int64_t y_stride, int64_t layer_idx, int rows_per_tile, int panels_per_wave,
    int tile_slots, int accumulate_into_y) {
  using E = typename D::E;
  using vec8 = typename D::vec8;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int c = lane & 15;
  const int g = lane >> 4;
  const int num_panels = (h_out + kExpTCols - 1) / kExpTCols;
  // Workgroup numbering: row tiles fastest, then panel groups, and consecutive numbers on one XCD.  The
  // row tiles of a long segment read the same panels of B^T; as neighbours on one XCD they find them in
  // its L2 instead of fetching them once per tile.
  const int vid = static_cast<int>(xcd_virtual_id());
  const int panel0 = (vid / tile_slots) * kExpTWaves * panels_per_wave;

  bool k_ok[KS];
  int k_off[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    k_ok[s] = s * 32 + g * 8 < r;  // chunks beyond the rank are loaded from chunk 0 and zeroed
    k_off[s] = k_ok[s] ? s * 32 + g * 8 : 0;
  }

  for (int tile = vid % tile_slots;; tile += tile_slots) {
    RowTile rt;
    if (!find_row_tile(s_start, s_end, num_segments, num_tokens, rows_per_tile, tile, rt)) break;
    const E* BT = reinterpret_cast<const E*>(W[rt.seg]) + layer_idx * h_out * static_cast<int64_t>(r);
    const int nmb = (rt.row_end - rt.row0 + 15) / 16;

    for (int pp = 0; pp < panels_per_wave; ++pp) {
      const int panel = panel0 + pp * kExpTWaves + wave;
      if (panel >= num_panels) break;
      const int n0 = panel * kExpTCols;
      const bool col_ok0 = n0 + g * 8 < h_out;
      const bool col_ok1 = n0 + 32 + g * 8 < h_out;
      // Loads are unconditional: rows past the tile are clamped to its last row and columns past
      // h_out to the panel's first vector (both valid memory); only the stores are predicated.
      const int coff0 = col_ok0 ? g * 8 : 0;
      const int coff1 = col_ok1 ? 32 + g * 8 : 0;
      auto load_block = [&](int mb, vec8(&vf)[KS], vec8& y0, vec8& y1) {
        const int row = min(rt.row0 + mb * 16 + c, rt.row_end - 1);
        const E* vp = V + static_cast<int64_t>(row) * r;
#pragma unroll
        for (int s = 0; s < KS; ++s) vf[s] = load8<D>(vp + k_off[s]);
        const E* yp = Y + static_cast<int64_t>(row) * y_stride + y_offset + n0;
        y0 = load8<D>(yp + coff0);
        y1 = load8<D>(yp + coff1);
      };
      auto block_of = [&](int i) { return min(i, nmb - 1); };

      // first row blocks and the panel's operands go out together: one memory round trip
      vec8 vr[kExpTStages][KS], y0r[kExpTStages], y1r[kExpTStages];
#pragma unroll
      for (int s = 0; s < kExpTStages - 1; ++s) load_block(block_of(s), vr[s], y0r[s], y1r[s]);
      vec8 bf[4][KS];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int col = min(n0 + panel_col_t(j, c), h_out - 1);
#pragma unroll
        for (int s = 0; s < KS; ++s)
          bf[j][s] = keep_if<D>(k_ok[s], load8<D>(BT + static_cast<int64_t>(col) * r + k_off[s]));
      }

      auto finish_block = [&](bool live, int mb, vec8(&vf)[KS], vec8 y0, vec8 y1) {
        f32x4 acc[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s = 0; s < KS; ++s) acc[j] = D::mfma16(bf[j][s], vf[s], acc[j]);
        }
        const int row = rt.row0 + mb * 16 + c;
        const bool ok = live && row < rt.row_end;
        E* yp = Y + static_cast<int64_t>(row) * y_stride + y_offset + n0;
        y0 = keep_if<D>(accumulate_into_y != 0, y0);  // overwrite mode: the old y counts as zero
        y1 = keep_if<D>(accumulate_into_y != 0, y1);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          y0[i] = accumulate<D>(y0[i], acc[0][i]);
          y0[4 + i] = accumulate<D>(y0[4 + i], acc[1][i]);
          y1[i] = accumulate<D>(y1[i], acc[2][i]);
          y1[4 + i] = accumulate<D>(y1[4 + i], acc[3][i]);
        }
        if (ok && col_ok0) store8<D>(yp + g * 8, y0);
        if (ok && col_ok1) store8<D>(yp + 32 + g * 8, y1);
      };

      // Ring of kExpTStages register stages with static indices: the y and v loads of the next
      // kExpTStages - 1 blocks are in flight while one block is multiplied and stored.  Surplus
      // trips of the last round re-load the last block and store nothing.
      for (int i = 0; i < nmb; i += kExpTStages) {
#pragma unroll
        for (int s = 0; s < kExpTStages; ++s) {
          constexpr int kAhead = kExpTStages - 1;
          load_block(block_of(i + s + kAhead), vr[(s + kAhead) % kExpTStages], y0r[(s + kAhead) % kExpTStages],
                     y1r[(s + kAhead) % kExpTStages]);
          __builtin_amdgcn_sched_barrier(0);
          finish_block(i + s < nmb, block_of(i + s), vr[s], y0r[s], y1r[s]);
        }
      }
    }
  }
}

template <typename D, int KS>
static hipError_t launch_expand_t_ks(const SgmvArgs& a, hipStream_t stream) {
  // 256-row tiles: the prologue is one memory round trip, so taller tiles buy nothing and even out worse
  int rows_per_tile = 256;
  if (tuning().expand_rows > 0) rows_per_tile = (tuning().expand_rows + 15) / 16 * 16;
  const int64_t tiles = (a.num_tokens + rows_per_tile - 1) / rows_per_tile + a.num_segments;
  const int num_panels = (a.d_out + kExpTCols - 1) / kExpTCols;
  // Panels per wave: more of them amortise the tile search, fewer give more workgroups; keep a few
  // thousand workgroups in the launch.
  int ppw = 4;
  while (ppw > 1 && tiles * ((num_panels + kExpTWaves * ppw - 1) / (kExpTWaves * ppw)) < 4096) ppw /= 2;
  if (tuning().expand_panels > 0) ppw = tuning().expand_panels;
  const int64_t panel_groups = (num_panels + kExpTWaves * ppw - 1) / (kExpTWaves * ppw);
  const int tile_slots = static_cast<int>(tiles < 65535 ? tiles : 65535);
  dim3 grid(static_cast<unsigned>(panel_groups * tile_slots));
  hipLaunchKernelGGL((sgmv_expand_t_kernel<D, KS>), grid, dim3(kExpTThreads), 0, stream,
                     static_cast<typename D::E*>(a.y), static_cast<const typename D::E*>(a.x), a.w_ptrs, a.s_start,
                     a.s_end, a.num_segments, static_cast<int>(a.num_tokens), a.d_in, a.d_out, a.y_offset,
                     a.y_stride, a.layer_idx, rows_per_tile, ppw, tile_slots, a.accumulate);
  return hipGetLastError();
}

template <typename D>
static hipError_t launch_expand_t_dtype(const SgmvArgs& a, hipStream_t stream) {
  switch ((a.d_in + 31) / 32) {
    case 1:
      return launch_expand_t_ks<D, 1>(a, stream);
    case 2:
      return launch_expand_t_ks<D, 2>(a, stream);
    case 3:
      return launch_expand_t_ks<D, 3>(a, stream);
    case 4:
      return launch_expand_t_ks<D, 4>(a, stream);
    default:
      return hipErrorInvalidValue;
  }
}

hipError_t launch_sgmv_expand_t(const SgmvArgs& a, hipStream_t stream) {
  return a.dtype == LORAX_F16 ? launch_expand_t_dtype<F16>(a, stream) : launch_expand_t_dtype<BF16>(a, stream);
}

}  // namespace lorax
