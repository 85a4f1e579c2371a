// SGMV expand for gfx950: y[s:e, off:off+h_out] += T(v[s:e, :r] @ B_i), B_i = [r, h_out].
//
// Replaces the expand configuration of the reference's cutlass grouped GEMM
// (sgmv/sgmv_cutlass.cuh:86-131; problem set-up :30-52).
//
// The contraction is only r (<= 128) long and the output is huge, so the kernel is a
// read-modify-write stream over y.  A workgroup owns a group of up to 512 output columns of one
// row tile of one segment:
//   * long tiles: the 64-column panels of the group are taken one after the other.  The r x 64
//     panel of B goes through LDS once, TRANSPOSED on the way in (pairs of k rows are written as
//     32-bit words into a [column][k] layout), so that every wave reads its MFMA operands - eight
//     consecutive k of one column - as 16-byte LDS loads and keeps them in registers; then the waves
//     walk 16-row blocks of the tile computing v (first MFMA operand) times B (second).  Accumulator j
//     stands for the columns 4c + j (c = lane & 15), which leaves each lane with 4 adjacent columns
//     of the rows 4g .. 4g + 3 (g = lane >> 4): a y access of the wave is four whole 128-byte runs,
//     one per row, and y is never staged;
//   * tiles of a few rows (decode tokens inside a prefill batch): MFMA operand set-up would
//     dominate, and what the tile costs is reading r rows of B.  A lane owns 8 adjacent columns of
//     the workgroup's columns, so a wave instruction reads whole 128-byte runs (1 KB with 512
//     columns) of rows of B; the k rows are dealt to groups of lanes, every B element is fetched
//     once for all rows of the tile, and the groups' sums meet in LDS.
// The host picks 1, 2, 4 or 8 panels per workgroup so that a small batch still fills the chip.
#include <type_traits>

#include "kernels.h"
#include "sgmv_tiles.h"

#ifndef LORAX_EXPAND_STAGES
#define LORAX_EXPAND_STAGES 2
#endif

namespace lorax {

constexpr int kExpandWaves = 4;
constexpr int kExpandThreads = kExpandWaves * kWave;
constexpr int kExpandCols = 64;          // output columns per panel
constexpr int kExpandPanels = 8;         // panels per workgroup: a group of 512 columns
constexpr int kExpandGroupCols = kExpandCols * kExpandPanels;
constexpr int kExpandShortRows = 4;      // row tiles up to this height use the vector path
constexpr int kExpandStages = LORAX_EXPAND_STAGES;  // register stages of the row-block pipeline

// Output column (0..63) that column `c` of the second MFMA operand of accumulator j stands for.
__device__ __forceinline__ int panel_col(int j, int c) { return 4 * c + j; }

template <typename D, int KS>
__global__ __launch_bounds__(kExpandThreads) void sgmv_expand_kernel(
    typename D::E* __restrict__ Y, const typename D::E* __restrict__ V,
    const int64_t* __restrict__ W, const int32_t* __restrict__ s_start,
    const int32_t* __restrict__ s_end, int num_segments, int num_tokens, int r, int h_out,
    int64_t y_offset, int64_t y_stride, int64_t layer_idx, int rows_per_tile, int panels_per_wg,
    int accumulate_into_y) {
  using E = typename D::E;
  using vec8 = typename D::vec8;
  constexpr int kPitch = KS * 32 + 8;  // elements per column of the transposed panel: 16-byte aligned rows
  __shared__ __attribute__((aligned(16))) E panel_t[kExpandCols * kPitch];
  __shared__ float redf[kExpandWaves][kExpandGroupCols];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int c = lane & 15;
  const int g = lane >> 4;
  // Plain numbering on purpose: neighbouring column groups on one XCD (xcd_virtual_block) measured
  // slower here - they read adjacent pieces of the same rows through the same L2 channels.
  const int group0 = blockIdx.x * panels_per_wg * kExpandCols;  // first column of this workgroup
  const bool acc_y = accumulate_into_y != 0;
  const int64_t pre_w = preload_segment_entry(W, num_segments);

  for (int tile = blockIdx.y;; tile += gridDim.y) {
    RowTile rt;
    // small remainders are merged into the segment's other tiles: a tile's prologue (search, staging the panels)
    // costs as much as a hundred rows
    if (!find_row_tile<true>(s_start, s_end, num_segments, num_tokens, rows_per_tile, tile, rt)) break;
    const E* B = reinterpret_cast<const E*>(segment_entry(pre_w, W, rt.seg)) + layer_idx * r * static_cast<int64_t>(h_out);
    const int nrows = rt.row_end - rt.row0;
    if (nrows <= kExpandShortRows) {
      // ---- vector path: the lanes of the workgroup are dealt over its columns (8 adjacent ones per lane)
      // and, with what is left, over groups of k rows; a wave instruction reads whole 128-byte runs of B.
      auto short_tile = [&](auto rows_c) {
        constexpr int MR = decltype(rows_c)::value;
        constexpr int U = 8;                       // k rows of B requested together by a lane
        const int cl = panels_per_wg * 8;          // lanes across the columns: 8, 16, 32 or 64
        const int kgroups = kExpandThreads / cl;   // k groups of the workgroup; group q owns k = q, q + kgroups, ...
        const int lc = lane & (cl - 1);
        const int kg = tid / cl;
        const int col = group0 + lc * 8;
        const bool col_ok = col < h_out;  // h_out is a multiple of 8: all 8 columns or none
        const E* bp = B + (col_ok ? col : 0);
        // lane l holds v[row][l] and v[row][l + 64]; the value of a k row is fetched from its lane
        float vlo[MR], vhi[MR];
#pragma unroll
        for (int m = 0; m < MR; ++m) {
          const E* vp = V + static_cast<int64_t>(min(rt.row0 + m, rt.row_end - 1)) * r;
          vlo[m] = to_f32<D>(vp[min(lane, r - 1)]);
          vhi[m] = KS > 2 ? to_f32<D>(vp[min(lane + kWave, r - 1)]) : 0.f;
        }
        float part[MR][8];
#pragma unroll
        for (int m = 0; m < MR; ++m)
#pragma unroll
          for (int e = 0; e < 8; ++e) part[m][e] = 0.f;
        for (int base = 0; base < r; base += U * kgroups) {  // uniform trip count
          vec8 bv[U];
#pragma unroll
          for (int u = 0; u < U; ++u)
            bv[u] = load8<D>(bp + static_cast<int64_t>(min(base + kg + u * kgroups, r - 1)) * h_out);
#pragma unroll
          for (int u = 0; u < U; ++u) {
            const int k = base + kg + u * kgroups;
            if (base + u * kgroups < r) {  // uniform: some lane of the workgroup still has a k row here
              float vk[MR];
#pragma unroll
              for (int m = 0; m < MR; ++m) {
                if (cl == kWave) {  // one k row per wave: a scalar lane read
                  const int ku = __builtin_amdgcn_readfirstlane(k);
                  const float src = (KS > 2 && ku >= kWave) ? vhi[m] : vlo[m];
                  vk[m] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, src), ku & (kWave - 1)));
                } else {
                  vk[m] = __shfl(vlo[m], k & (kWave - 1));
                  if (KS > 2) {
                    const float hi = __shfl(vhi[m], k & (kWave - 1));
                    vk[m] = k < kWave ? vk[m] : hi;
                  }
                }
                vk[m] = k < r ? vk[m] : 0.f;
              }
#pragma unroll
              for (int e = 0; e < 8; ++e) {
                const float w = to_f32<D>(bv[u][e]);
#pragma unroll
                for (int m = 0; m < MR; ++m) part[m][e] = fmaf(vk[m], w, part[m][e]);
              }
            }
          }
        }
        // the k groups' sums meet in LDS, one row at a time; thread t then finishes the columns 2t, 2t + 1
        float* red = &redf[0][0];
        const int ncols = cl * 8;
#pragma unroll
        for (int m = 0; m < MR; ++m) {
          if (m < nrows) {  // uniform over the workgroup
#pragma unroll
            for (int e = 0; e < 8; ++e) red[kg * ncols + lc * 8 + e] = part[m][e];
            __syncthreads();
            const int cc = group0 + 2 * tid;
            if (2 * tid < ncols && cc < h_out) {  // h_out is even: both columns or none
              float s0 = 0.f, s1 = 0.f;
              for (int q = 0; q < kgroups; ++q) {
                s0 += red[q * ncols + 2 * tid];
                s1 += red[q * ncols + 2 * tid + 1];
              }
              typedef E pair __attribute__((ext_vector_type(2)));
              E* yp = Y + static_cast<int64_t>(rt.row0 + m) * y_stride + y_offset + cc;
              pair out;
              if (acc_y) {
                const pair old = *reinterpret_cast<const pair*>(yp);
                out[0] = accumulate<D>(old[0], s0);
                out[1] = accumulate<D>(old[1], s1);
              } else {
                out[0] = accumulate<D>(static_cast<E>(0.f), s0);
                out[1] = accumulate<D>(static_cast<E>(0.f), s1);
              }
              *reinterpret_cast<pair*>(yp) = out;
            }
            __syncthreads();
          }
        }
      };
      if (nrows == 1)
        short_tile(std::integral_constant<int, 1>{});
      else if (nrows == 2)
        short_tile(std::integral_constant<int, 2>{});
      else
        short_tile(std::integral_constant<int, kExpandShortRows>{});
      continue;
    }

    // ---- MFMA path: the panels of the group one after the other ----
    typedef E yvec __attribute__((ext_vector_type(4)));
    const int nmb = (nrows + 15) / 16;
    bool k_ok[KS];
    int k_off[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      k_ok[s] = s * 32 + g * 8 < r;
      k_off[s] = k_ok[s] ? s * 32 + g * 8 : 0;
    }
    // This wave's 16-row blocks are wave, wave + 4, ... below nmb.
    const int n = wave < nmb ? (nmb - wave + kExpandWaves - 1) / kExpandWaves : 0;
    auto block_of = [&](int i) { return wave + min(i, max(n, 1) - 1) * kExpandWaves; };
    for (int pp = 0; pp < panels_per_wg; ++pp) {
      const int n0 = group0 + pp * kExpandCols;
      if (n0 >= h_out) break;  // uniform over the workgroup
      // h_out is a multiple of 8: a lane's four columns are inside the matrix or outside it as a whole.
      // Loads are unconditional: rows past the tile are clamped to its last row and a lane past h_out
      // reads the panel's first columns (both valid memory); only the stores are predicated.
      // v chunks beyond the rank are zeroed after the load.
      const bool col_ok = n0 + 4 * c < h_out;
      const int col = n0 + (col_ok ? 4 * c : 0);
      auto load_block = [&](int mb, vec8(&vf)[KS], yvec(&yv)[4]) {
        const int vrow = min(rt.row0 + mb * 16 + c, rt.row_end - 1);
        const E* vp = V + static_cast<int64_t>(vrow) * r;
#pragma unroll
        for (int s = 0; s < KS; ++s) vf[s] = load8<D>(vp + k_off[s]);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int row = min(rt.row0 + mb * 16 + g * 4 + i, rt.row_end - 1);
          yv[i] = *(const LORAX_GLOBAL yvec*)(Y + static_cast<int64_t>(row) * y_stride + y_offset + col);
        }
      };
      // The first y / v loads of the wave's row blocks go out BEFORE the panel of B is staged: they do
      // not depend on it, so the panel's first memory round trip overlaps the operand set-up.
      vec8 vr[kExpandStages][KS];
      yvec yr[kExpandStages][4];
#pragma unroll
      for (int s = 0; s < kExpandStages - 1; ++s) load_block(block_of(s), vr[s], yr[s]);

      // Stage the r x 64 panel of B transposed: an item is a pair of k rows times 8 columns; the pair's
      // values of one column form one 32-bit word of panel_t[column][k].  Rows k >= r and columns >= h_out
      // are staged as zeros.
      for (int p = tid; p < KS * 16 * (kExpandCols / 8); p += kExpandThreads) {
        const int k = (p / (kExpandCols / 8)) * 2;
        const int cc = (p % (kExpandCols / 8)) * 8;
        vec8 b0 = zero8<D>(), b1 = zero8<D>();
        if (n0 + cc < h_out) {
          if (k < r) b0 = load8<D>(B + static_cast<int64_t>(k) * h_out + n0 + cc);
          if (k + 1 < r) b1 = load8<D>(B + static_cast<int64_t>(k + 1) * h_out + n0 + cc);
        }
        typedef E pair __attribute__((ext_vector_type(2)));
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          pair w;
          w[0] = b0[e];
          w[1] = b1[e];
          *reinterpret_cast<pair*>(panel_t + (cc + e) * kPitch + k) = w;
        }
      }
      __syncthreads();
      vec8 bf[4][KS];
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int s = 0; s < KS; ++s)
          bf[j][s] = *reinterpret_cast<const vec8*>(panel_t + panel_col(j, c) * kPitch + s * 32 + g * 8);
      __syncthreads();  // the panel may be overwritten by the next one from here on

      auto finish_block = [&](bool live, int mb, vec8(&vf)[KS], yvec(&yv)[4]) {
        f32x4 acc[4];
#pragma unroll
        for (int s = 0; s < KS; ++s) vf[s] = keep_if<D>(k_ok[s], vf[s]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s = 0; s < KS; ++s) acc[j] = D::mfma16(vf[s], bf[j][s], acc[j]);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int row = rt.row0 + mb * 16 + g * 4 + i;
          yvec out;
#pragma unroll
          for (int j = 0; j < 4; ++j)  // overwrite mode: the old y counts as zero
            out[j] = accumulate<D>(acc_y ? yv[i][j] : static_cast<E>(0.0f), acc[j][i]);
          if (live && col_ok && row < rt.row_end)
            *(LORAX_GLOBAL yvec*)(Y + static_cast<int64_t>(row) * y_stride + y_offset + col) = out;
        }
      };
      // Ring of kExpandStages register stages (static indices, unrolled): the y and v loads of the next
      // kExpandStages-1 blocks are in flight while one block is multiplied and stored.  Surplus trips of the
      // last round re-load the last block and store nothing.
      if (n > 0) {
        for (int i = 0; i < n; i += kExpandStages) {
#pragma unroll
          for (int s = 0; s < kExpandStages; ++s) {
            constexpr int kAhead = kExpandStages - 1;
            load_block(block_of(i + s + kAhead), vr[(s + kAhead) % kExpandStages], yr[(s + kAhead) % kExpandStages]);
            __builtin_amdgcn_sched_barrier(0);
            finish_block(i + s < n, block_of(i + s), vr[s], yr[s]);
          }
        }
      }
    }
  }
}

template <typename D, int KS>
static hipError_t launch_expand_ks(const SgmvArgs& a, hipStream_t stream) {
  // As many 64-column panels per workgroup (a power of two up to 8) as still leave a thousand
  // workgroups: more panels amortise the tile search, fewer fill the chip on small batches.
  int rows_per_tile = a.num_tokens >= 8192 ? 512 : 256;
  if (tuning().expand_rows > 0) rows_per_tile = (tuning().expand_rows + 63) / 64 * 64;
  const int64_t tiles = (a.num_tokens + rows_per_tile - 1) / rows_per_tile + a.num_segments;
  const int num_panels = (a.d_out + kExpandCols - 1) / kExpandCols;
  int ppw = kExpandPanels;
  while (ppw > 1 && tiles * ((num_panels + ppw - 1) / ppw) < 1024) ppw /= 2;
  if (tuning().expand_panels > 0 && tuning().expand_panels <= kExpandPanels &&
      (tuning().expand_panels & (tuning().expand_panels - 1)) == 0)
    ppw = tuning().expand_panels;
  dim3 grid((num_panels + ppw - 1) / ppw, static_cast<unsigned>(tiles < 65535 ? tiles : 65535));
  hipLaunchKernelGGL((sgmv_expand_kernel<D, KS>), grid, dim3(kExpandThreads), 0, stream,
                     static_cast<typename D::E*>(a.y), static_cast<const typename D::E*>(a.x),
                     a.w_ptrs, a.s_start, a.s_end, a.num_segments, static_cast<int>(a.num_tokens),
                     a.d_in, a.d_out, a.y_offset, a.y_stride, a.layer_idx, rows_per_tile, ppw, a.accumulate);
  return hipGetLastError();
}

template <typename D>
static hipError_t launch_expand_dtype(const SgmvArgs& a, hipStream_t stream) {
  switch ((a.d_in + 31) / 32) {
    case 1:
      return launch_expand_ks<D, 1>(a, stream);
    case 2:
      return launch_expand_ks<D, 2>(a, stream);
    case 3:
      return launch_expand_ks<D, 3>(a, stream);
    case 4:
      return launch_expand_ks<D, 4>(a, stream);
    default:
      return hipErrorInvalidValue;
  }
}

hipError_t launch_sgmv_expand(const SgmvArgs& a, hipStream_t stream) {
  return a.dtype == LORAX_F16 ? launch_expand_dtype<F16>(a, stream)
                              : launch_expand_dtype<BF16>(a, stream);
}

}  // namespace lorax
