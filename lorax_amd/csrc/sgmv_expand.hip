// SGMV expand for gfx950: y[s:e, off:off+h_out] += T(v[s:e, :r] @ B_i), B_i = [r, h_out].
//
// Replaces the expand configuration of the reference's cutlass grouped GEMM
// (sgmv/sgmv_cutlass.cuh:86-131; problem set-up :30-52).
//
// The contraction is only r (<= 128) long and the output is huge, so the kernel is a
// read-modify-write stream over y.  A workgroup owns 64 output columns of one row
// chunk of one segment:
//   * long segments: the r x 64 panel of B goes through LDS once, every wave turns it
//     into MFMA operands that stay in registers, and then walks 16-row blocks of the
//     chunk computing v (first MFMA operand) times B (second).  Accumulator j stands for
//     the columns 4c + j (c = lane & 15), which leaves each lane with 4 adjacent columns
//     of the rows 4g .. 4g + 3 (g = lane >> 4): a y access of the wave is four whole
//     128-byte runs, one per row, and y is never staged;
//   * segments of a few rows (decode tokens inside a prefill batch): MFMA operand
//     set-up would dominate, so the panel is streamed row by row on the vector ALU
//     with 16-byte loads, each lane owning 8 adjacent columns.
#include "kernels.h"
#include "sgmv_tiles.h"

#ifndef LORAX_EXPAND_STAGES
#define LORAX_EXPAND_STAGES 2
#endif

namespace lorax {

constexpr int kExpandWaves = 4;
constexpr int kExpandThreads = kExpandWaves * kWave;
constexpr int kExpandCols = 64;          // output columns per workgroup
constexpr int kExpandShortRows = 4;      // row tiles up to this height use the vector path
constexpr int kPanelPitch = kExpandCols + 4;  // LDS row pitch in elements
constexpr int kExpandStages = LORAX_EXPAND_STAGES;  // register stages of the row-block pipeline

// Output column (0..63) that column `c` of the second MFMA operand of accumulator j stands for.
__device__ __forceinline__ int panel_col(int j, int c) { return 4 * c + j; }

template <typename D, int KS>
__global__ __launch_bounds__(kExpandThreads) void sgmv_expand_kernel(
    typename D::E* __restrict__ Y, const typename D::E* __restrict__ V,
    const int64_t* __restrict__ W, const int32_t* __restrict__ s_start,
    const int32_t* __restrict__ s_end, int num_segments, int num_tokens, int r, int h_out,
    int64_t y_offset, int64_t y_stride, int64_t layer_idx, int rows_per_tile, int accumulate_into_y) {
  using E = typename D::E;
  using vec8 = typename D::vec8;
  __shared__ __attribute__((aligned(16))) E panel[KS * 32 * kPanelPitch];
  __shared__ float redf[kExpandWaves][kExpandCols];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int c = lane & 15;
  const int g = lane >> 4;
  // Plain numbering on purpose: neighbouring column panels on one XCD (xcd_virtual_block) measured
  // 30 % slower here - they read adjacent 128-byte pieces of the same rows through the same L2 channels.
  const int n0 = blockIdx.x * kExpandCols;

  for (int tile = blockIdx.y;; tile += gridDim.y) {
    RowTile rt;
    if (!find_row_tile(s_start, s_end, num_segments, num_tokens, rows_per_tile, tile, rt)) break;
    const E* B = reinterpret_cast<const E*>(W[rt.seg]) + layer_idx * r * static_cast<int64_t>(h_out);
    const int nrows = rt.row_end - rt.row0;
    if (nrows <= kExpandShortRows) {
      // ---- vector path: thread (kq, c8) owns k = kq, kq+32, ... and 8 columns ----
      const int c8 = tid & 7;
      const int kq = tid >> 3;
      const int col = n0 + c8 * 8;
      float bw[KS][8];
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const int k = kq + 32 * s;
        vec8 bv = zero8<D>();
        if (k < r && col < h_out) bv = load8<D>(B + static_cast<int64_t>(k) * h_out + col);
#pragma unroll
        for (int e = 0; e < 8; ++e) bw[s][e] = to_f32<D>(bv[e]);
      }
      for (int row = rt.row0; row < rt.row_end; ++row) {
        float part[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) part[e] = 0.f;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
          const int k = kq + 32 * s;
          const float vk = k < r ? to_f32<D>(V[static_cast<int64_t>(row) * r + k]) : 0.f;
#pragma unroll
          for (int e = 0; e < 8; ++e) part[e] = fmaf(vk, bw[s][e], part[e]);
        }
        // lanes of a wave are (kq % 8, c8): fold the eight kq of the wave together
#pragma unroll
        for (int m = 8; m < kWave; m <<= 1)
#pragma unroll
          for (int e = 0; e < 8; ++e) part[e] += __shfl_xor(part[e], m, kWave);
        if (lane < 8) {
#pragma unroll
          for (int e = 0; e < 8; ++e) redf[wave][c8 * 8 + e] = part[e];
        }
        __syncthreads();
        if (tid < kExpandCols && n0 + tid < h_out) {
          float s = 0.f;
#pragma unroll
          for (int w = 0; w < kExpandWaves; ++w) s += redf[w][tid];
          E* yp = Y + static_cast<int64_t>(row) * y_stride + y_offset + n0 + tid;
          *yp = accumulate<D>(accumulate_into_y != 0 ? *yp : static_cast<E>(0.f), s);
        }
        __syncthreads();
      }
      continue;
    }

    vec8 bf[4][KS];
    typedef E yvec __attribute__((ext_vector_type(4)));
    const int nmb = (nrows + 15) / 16;
    // h_out is a multiple of 8: a lane's four columns are inside the matrix or outside it as a whole.
    // Loads are unconditional: rows past the tile are clamped to its last row and a lane past h_out
    // reads the panel's first columns (both valid memory); only the stores are predicated.
    // v chunks beyond the rank are zeroed after the load.
    const bool col_ok = n0 + 4 * c < h_out;
    const int col = n0 + (col_ok ? 4 * c : 0);
    bool k_ok[KS];
    int k_off[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      k_ok[s] = s * 32 + g * 8 < r;
      k_off[s] = k_ok[s] ? s * 32 + g * 8 : 0;
    }
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
          out[j] = accumulate<D>(accumulate_into_y != 0 ? yv[i][j] : static_cast<E>(0.0f), acc[j][i]);
        if (live && col_ok && row < rt.row_end)
          *(LORAX_GLOBAL yvec*)(Y + static_cast<int64_t>(row) * y_stride + y_offset + col) = out;
      }
    };

    // This wave's 16-row blocks are wave, wave + 4, ... below nmb.  They run through a ring of
    // kExpandStages register stages (static indices, unrolled): the y and v loads of the next
    // kExpandStages-1 blocks are in flight while one block is multiplied and stored.  Surplus
    // trips of the last round re-load the last block and store nothing.
    // The first y / v loads of the wave's row blocks go out BEFORE the panel of B is staged: they do
    // not depend on it, so the tile's first memory round trip overlaps the operand set-up.
    const int n = wave < nmb ? (nmb - wave + kExpandWaves - 1) / kExpandWaves : 0;
    auto block_of = [&](int i) { return wave + min(i, max(n, 1) - 1) * kExpandWaves; };
    vec8 vr[kExpandStages][KS];
    yvec yr[kExpandStages][4];
#pragma unroll
    for (int s = 0; s < kExpandStages - 1; ++s) load_block(block_of(s), vr[s], yr[s]);

    // ---- MFMA path ----
    // Stage the r x 64 panel of B in LDS (rows k >= r and columns >= h_out as zeros).
    for (int p = tid; p < KS * 32 * (kExpandCols / 8); p += kExpandThreads) {
      const int k = p / (kExpandCols / 8);
      const int cc = (p % (kExpandCols / 8)) * 8;
      vec8 bv = zero8<D>();
      if (k < r && n0 + cc < h_out) bv = load8<D>(B + static_cast<int64_t>(k) * h_out + n0 + cc);
      // rows are 8-byte aligned (pitch 68 elements), so two 8-byte LDS stores
      const u32x4 bits = __builtin_bit_cast(u32x4, bv);
      u32x2* dst = reinterpret_cast<u32x2*>(panel + k * kPanelPitch + cc);
      dst[0] = u32x2{bits[0], bits[1]};
      dst[1] = u32x2{bits[2], bits[3]};
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int colj = panel_col(j, c);
#pragma unroll
      for (int s = 0; s < KS; ++s)
#pragma unroll
        for (int e = 0; e < 8; ++e) bf[j][s][e] = panel[(s * 32 + g * 8 + e) * kPanelPitch + colj];
    }
    __syncthreads();  // the panel may be overwritten by the next tile from here on

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

template <typename D, int KS>
static hipError_t launch_expand_ks(const SgmvArgs& a, hipStream_t stream) {
  // Rows per tile: the tile prologue (tile search, staging and transposing the panel of B) is
  // amortised over the tile's rows, so tiles are tall when there are many rows to go round.
  int rows_per_tile = a.num_tokens >= 8192 ? 512 : 256;
  if (tuning().expand_rows > 0) rows_per_tile = (tuning().expand_rows + 63) / 64 * 64;
  const int64_t tiles = (a.num_tokens + rows_per_tile - 1) / rows_per_tile + a.num_segments;
  dim3 grid((a.d_out + kExpandCols - 1) / kExpandCols,
            static_cast<unsigned>(tiles < 65535 ? tiles : 65535));
  hipLaunchKernelGGL((sgmv_expand_kernel<D, KS>), grid, dim3(kExpandThreads), 0, stream,
                     static_cast<typename D::E*>(a.y), static_cast<const typename D::E*>(a.x),
                     a.w_ptrs, a.s_start, a.s_end, a.num_segments, static_cast<int>(a.num_tokens),
                     a.d_in, a.d_out, a.y_offset, a.y_stride, a.layer_idx, rows_per_tile, a.accumulate);
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
