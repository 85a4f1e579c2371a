// SGMV shrink for gfx950: v[s:e, :r] += T(x[s:e, :] @ A_i) for every segment i.
//
// Replaces flashinfer::sgmv::sgmv_shrink (sgmv_flashinfer/sgmv_flashinfer.cuh:13-353,
// launched from sgmv_flashinfer/sgmv_all.cu:10-65) for the [L, r, h_in] layout and the
// shrink configuration of the cutlass grouped GEMM (sgmv/sgmv_cutlass.cuh:132-178) for
// the [L, h_in, r] layout.
//
// [L, r, h_in] kernel: both operands are K-contiguous, which is the register layout
// v_mfma_f32_16x16x32_{bf16,f16} wants (lane l supplies 8 consecutive k of row l%16
// starting at k = 8*(l/16)), so x and A go from global memory straight into MFMA
// operands with 16-byte loads.  A workgroup owns a row tile and a K range; its waves
// interleave over the K steps of that range and meet in LDS.  When a launch has too
// few row tiles to fill the chip, K is also split across workgroups: every workgroup
// stores its fp32 partial tile, and the last one to arrive (one atomic counter per
// row tile) adds the partials in a fixed order and rounds once.  There is no grid-wide
// barrier (the reference needs a cooperative launch for this, sgmv_all.cu:44-55).
#include "kernels.h"
#include "sgmv_tiles.h"

namespace lorax {

template <typename D, int NB, int MB, int WAVES>
__global__ __launch_bounds__(WAVES * kWave) void sgmv_shrink_rh_kernel(
    typename D::E* __restrict__ V, const typename D::E* __restrict__ X,
    const int64_t* __restrict__ W, const int32_t* __restrict__ s_start,
    const int32_t* __restrict__ s_end, int num_segments, int num_tokens, int h_in,
    int64_t layer_idx, int ksplit, float* __restrict__ partials,
    uint32_t* __restrict__ counters, int num_counters, int rotate_k, float scale, int accumulate_into_v) {
  using E = typename D::E;
  using vec8 = typename D::vec8;
  constexpr int R = NB * 16;
  constexpr int ROWS = MB * 16;
  constexpr int THREADS = WAVES * kWave;
  // register stages of the K pipeline: as many as fit next to the accumulators
  constexpr int kBudget = WAVES >= 16 ? 96 : (WAVES >= 8 ? 200 : 232);  // registers for stages + accumulators
  constexpr int STAGES = (MB + NB) * 4 * 4 + MB * NB * 4 <= kBudget - 32
                             ? 4
                             : ((MB + NB) * 4 * 3 + MB * NB * 4 <= kBudget ? 3 : 2);
  __shared__ f32x4 red[WAVES][NB][kWave];
  __shared__ uint32_t arrival;

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int c = lane & 15;   // operand row inside a 16-row block
  const int g = lane >> 4;   // which 8 of the 32 k of a step
  // XCD-aware numbering: consecutive row tiles (the tiles of one segment) run on one XCD, so the
  // segment's A is fetched into one L2 instead of into every L2 that happens to get a tile.
  const VirtualBlock vb = xcd_virtual_block();
  const int kc = vb.x;

  const int ksteps = (h_in + 31) / 32;
  const int per = (ksteps + ksplit - 1) / ksplit;
  const int ks0 = kc * per;
  const int ks1 = min(ks0 + per, ksteps);

  for (int tile = vb.y;; tile += gridDim.y) {
    RowTile rt;
    if (!find_row_tile(s_start, s_end, num_segments, num_tokens, ROWS, tile, rt)) break;
    // Disjoint segments never produce this many tiles (the host sizes ksplit for that);
    // overlapping ones are outside the contract and must only not fault.
    if (ksplit > 1 && tile >= num_counters) break;
    const int nmb = (rt.row_end - rt.row0 + 15) / 16;
    const E* A = reinterpret_cast<const E*>(W[rt.seg]) + layer_idx * R * static_cast<int64_t>(h_in);

    // Operand addresses.  Rows past the end of the tile are clamped to its last row: they load
    // valid memory, produce output rows nobody stores, and keep the loop free of conditional
    // loads (a load into a register that was just zeroed makes the compiler wait for it).
    const E* xp[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int row = min(rt.row0 + mb * 16 + c, rt.row_end - 1);
      xp[mb] = X + static_cast<int64_t>(row) * h_in + g * 8;
    }
    const E* ap = A + static_cast<int64_t>(c) * h_in + g * 8;

    f32x4 acc[MB][NB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = f32x4{0.f, 0.f, 0.f, 0.f};

    auto load_step = [&](int ks, vec8(&xf)[MB], vec8(&wf)[NB]) {
      const int k = ks * 32;
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) xf[mb] = load8<D>(xp[mb] + k);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) wf[nb] = load8<D>(ap + static_cast<int64_t>(nb) * 16 * h_in + k);
    };
    auto mma_step = [&](bool live, vec8(&xf)[MB], const vec8(&wf)[NB]) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const vec8 xm = keep_if<D>(live, xf[mb]);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = D::mfma16(wf[nb], xm, acc[mb][nb]);
      }
    };

    // This wave's K steps are ks0 + wave, + WAVES, ... below `last` (whole steps only).  They run
    // through a ring of STAGES register stages with STAGES-1 steps of loads in flight while one
    // step multiplies.  The ring is unrolled, so stage indices are static; the trip count is
    // rounded up to a multiple of STAGES, the surplus steps re-load the last step (clamped
    // address) and multiply zeros.
    const int last = min(ks1, h_in / 32);
    const int first = ks0 + wave;
    if (first < last) {
      const int n = (last - first + WAVES - 1) / WAVES;
      // Rows of x are a power-of-two number of bytes apart, so workgroups that all start at k = 0
      // and advance in step keep hitting the same few HBM channels.  Every tile therefore starts
      // its walk over K at a different step and wraps around (the sum does not care about order).
      const int rot = static_cast<int>((static_cast<unsigned>(tile) * 2654435761u) >> 8) % n;
      auto step_ks = [&](int i) {
        const int j = min(i, n - 1) + (rotate_k ? rot : 0);
        return first + (j >= n ? j - n : j) * WAVES;
      };
      vec8 xr[STAGES][MB], wr[STAGES][NB];
#pragma unroll
      for (int s = 0; s < STAGES - 1; ++s) load_step(step_ks(s), xr[s], wr[s]);
      for (int i = 0; i < n; i += STAGES) {
#pragma unroll
        for (int s = 0; s < STAGES; ++s) {
          load_step(step_ks(i + s + STAGES - 1), xr[(s + STAGES - 1) % STAGES], wr[(s + STAGES - 1) % STAGES]);
          __builtin_amdgcn_sched_barrier(0);
          mma_step(i + s < n, xr[s], wr[s]);
        }
      }
    }
    // A hidden size that is not a multiple of 32 leaves one partial step: the lanes whose 8 k
    // lie beyond h_in contribute zeros.
    if ((h_in & 31) != 0) {
      const int kt = h_in / 32;
      if (kt >= ks0 && kt < ks1 && (kt - ks0) % WAVES == wave) {
        const bool kok = kt * 32 + g * 8 < h_in;
        const int k = kok ? kt * 32 : 0;
        vec8 xt[MB], wt[NB];
        load_step(k / 32, xt, wt);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) wt[nb] = keep_if<D>(kok, wt[nb]);
        mma_step(kok, xt, wt);
      }
    }

    // acc[mb][nb][i] of lane (g, c) is D[n = nb*16 + 4g + i][row = mb*16 + c].
    // Sum the waves' tiles one 16-row block at a time through LDS.
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      if (mb < nmb) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) red[wave][nb][lane] = acc[mb][nb];
        __syncthreads();
        for (int p = tid; p < NB * kWave; p += THREADS) {
          const int nb = p / kWave;
          const int ln = p % kWave;
          f32x4 s = red[0][nb][ln];
#pragma unroll
          for (int w = 1; w < WAVES; ++w) s += red[w][nb][ln];
          const int row = rt.row0 + mb * 16 + (ln & 15);
          const int n = nb * 16 + 4 * (ln >> 4);
          if (row < rt.row_end) {
            if (ksplit == 1) {
              update4<D>(accumulate_into_v != 0, V + static_cast<int64_t>(row) * R + n, s * scale);
            } else {
              float* pp = partials + (static_cast<int64_t>(kc) * num_tokens + row) * R + n;
              *reinterpret_cast<f32x4*>(pp) = s;
            }
          }
        }
        __syncthreads();
      }
    }

    if (ksplit > 1) {
      // Publish this workgroup's partial tile, then let the last arrival finish the tile.
      __threadfence();
      __syncthreads();
      if (tid == 0) arrival = atomicAdd(&counters[tile], 1u);
      __syncthreads();
      const bool last = arrival == static_cast<uint32_t>(ksplit - 1);
      if (last) {
        __threadfence();
        const int nrows = rt.row_end - rt.row0;
        for (int p = tid; p < nrows * (R / 4); p += THREADS) {
          const int row = rt.row0 + p / (R / 4);
          const int n = (p % (R / 4)) * 4;
          f32x4 s = f32x4{0.f, 0.f, 0.f, 0.f};
          for (int q = 0; q < ksplit; ++q) {
            const float* pp = partials + (static_cast<int64_t>(q) * num_tokens + row) * R + n;
            s += *reinterpret_cast<const f32x4*>(pp);
          }
          update4<D>(accumulate_into_v != 0, V + static_cast<int64_t>(row) * R + n, s * scale);
        }
        if (tid == 0) atomicExch(&counters[tile], 0u);
      }
      __syncthreads();
    }
  }
}

// [L, h_in, r] layout (rank 8 in the reference: use_cutlass_shrink, punica.py:79-80).
// A's rows are only r long, so this is a streaming kernel on the vector ALU: a thread
// owns 8 consecutive k, reads 16 bytes of each of the tile's x rows and the matching
// 8 x 8 block of A, and the per-thread sums meet in a wave reduction.
template <typename D, int RT>
__global__ __launch_bounds__(256) void sgmv_shrink_hr_kernel(
    typename D::E* __restrict__ V, const typename D::E* __restrict__ X,
    const int64_t* __restrict__ W, const int32_t* __restrict__ s_start,
    const int32_t* __restrict__ s_end, int num_segments, int num_tokens, int h_in, int r,
    int64_t layer_idx, float scale, int accumulate_into_v) {
  using E = typename D::E;
  using vec8 = typename D::vec8;
  constexpr int THREADS = 256;
  constexpr int NV = RT * 8;
  __shared__ float red[THREADS / kWave][NV];
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;

  for (int tile = blockIdx.x;; tile += gridDim.x) {
    RowTile rt;
    if (!find_row_tile(s_start, s_end, num_segments, num_tokens, RT, tile, rt)) break;
    const E* A = reinterpret_cast<const E*>(W[rt.seg]) + layer_idx * r * static_cast<int64_t>(h_in);
    for (int n0 = 0; n0 < r; n0 += 8) {
      float acc[NV];
#pragma unroll
      for (int i = 0; i < NV; ++i) acc[i] = 0.f;
      for (int k = tid * 8; k < h_in; k += THREADS * 8) {
        float xf[RT][8];
#pragma unroll
        for (int m = 0; m < RT; ++m) {
          const int row = min(rt.row0 + m, rt.row_end - 1);
          const vec8 xv = load8<D>(X + static_cast<int64_t>(row) * h_in + k);
#pragma unroll
          for (int e = 0; e < 8; ++e) xf[m][e] = to_f32<D>(xv[e]);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const vec8 wv = load8<D>(A + static_cast<int64_t>(k + e) * r + n0);
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float w = to_f32<D>(wv[j]);
#pragma unroll
            for (int m = 0; m < RT; ++m) acc[m * 8 + j] = fmaf(xf[m][e], w, acc[m * 8 + j]);
          }
        }
      }
      transpose_reduce<NV>(acc);
      if ((lane & (kWave / NV - 1)) == 0) red[wave][transpose_reduce_index<NV>(lane)] = acc[0];
      __syncthreads();
      if (tid < NV) {
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < THREADS / kWave; ++w) s += red[w][tid];
        const int row = rt.row0 + tid / 8;
        if (row < rt.row_end) {
          E* vp = V + static_cast<int64_t>(row) * r + n0 + (tid % 8);
          *vp = accumulate<D>(accumulate_into_v != 0 ? *vp : static_cast<E>(0.f), s * scale);
        }
      }
      __syncthreads();
    }
  }
}

// Arrival counters must read zero when a split-K launch starts.  The last arrival of every tile resets its
// counter, but the scratch may be a buffer nobody ever initialised (the caller's tmp) or may have been left
// dirty by a launch that was torn down, so every split-K launch is preceded by this fill.  A kernel, not a
// memset, so that the pair can be captured into a graph.
__global__ void zero_counters_kernel(uint32_t* __restrict__ counters, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) counters[i] = 0u;
}

// ---------------------------------------------------------------------------------
// Host-side launchers
// ---------------------------------------------------------------------------------
// Row-tile height (in 16-row blocks) of the register-operand kernel: 64 rows when there are many rows, 16 for
// short batches so the few tiles there are do not carry padding; above rank 64 at most 32 rows (registers).
static int rh_row_blocks(const SgmvArgs& a) {
  const int nb = a.d_out / 16;
  int mb = a.num_tokens >= 2048 ? 4 : (a.num_tokens >= 256 ? 2 : 1);
  if (tuning().shrink_mb > 0) mb = tuning().shrink_mb;
  if (mb != 1 && mb != 2 && mb != 4) mb = 1;
  if (nb > 4 && mb > 2) mb = 2;
  return mb;
}

// Splitting K across workgroups costs a device-scope fence per workgroup, which is only worth paying when the
// row tiles alone cannot occupy the 256 CUs; the split is cut to what the scratch holds.
int sgmv_shrink_ksplit(const SgmvArgs& a) {
  const int mb = rh_row_blocks(a);
  const int64_t tiles = (a.num_tokens + mb * 16 - 1) / (mb * 16) + a.num_segments;
  const int ksteps = (a.d_in + 31) / 32;
  int ksplit = 1;
  if (fixed_order_shrink()) return 1;
  if (tuning().shrink_ksplit > 0) {
    ksplit = tuning().shrink_ksplit;
  } else if (tiles < 192) {
    const int64_t want = (384 + tiles - 1) / tiles;
    const int kmax = ksteps / 16 > 0 ? ksteps / 16 : 1;
    ksplit = static_cast<int>(want < kmax ? want : kmax);
    if (ksplit > 8) ksplit = 8;
  }
  if (ksplit > ksteps) ksplit = ksteps;
  if (ksplit < 1) ksplit = 1;
  if (ksplit > 1) {
    const size_t per_chunk = static_cast<size_t>(a.num_tokens) * a.d_out * sizeof(float);
    const size_t fit = per_chunk ? a.partial_bytes / per_chunk : 1;
    if (static_cast<size_t>(ksplit) > fit) ksplit = static_cast<int>(fit);
    if (ksplit < 1) ksplit = 1;
    if (static_cast<size_t>(tiles) > a.num_counters || a.partials == nullptr || a.counters == nullptr) ksplit = 1;
  }
  return ksplit;
}

template <typename D, int NB, int MB, int WAVES>
static hipError_t launch_rh_w(const SgmvArgs& a, int ksplit, hipStream_t stream) {
  const int64_t tiles = (a.num_tokens + MB * 16 - 1) / (MB * 16) + a.num_segments;
  dim3 grid(ksplit, static_cast<unsigned>(tiles < 65535 ? tiles : 65535));
  if (ksplit > 1) {
    const int n = static_cast<int>(tiles);  // sgmv_shrink_ksplit: tiles <= num_counters whenever K is split
    hipLaunchKernelGGL(zero_counters_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, a.counters, n);
  }
  hipLaunchKernelGGL((sgmv_shrink_rh_kernel<D, NB, MB, WAVES>), grid, dim3(WAVES * kWave), 0,
                     stream, static_cast<typename D::E*>(a.y),
                     static_cast<const typename D::E*>(a.x), a.w_ptrs, a.s_start, a.s_end,
                     a.num_segments, static_cast<int>(a.num_tokens), a.d_in, a.layer_idx, ksplit,
                     a.partials, a.counters, static_cast<int>(a.num_counters),
                     (tuning().shrink_no_rotate || fixed_order_shrink()) ? 0 : 1, a.scale,
                     a.accumulate);
  return hipGetLastError();
}

// Waves per workgroup = how many ways K is split inside the workgroup (through LDS, no fences).
template <typename D, int NB, int MB>
static hipError_t launch_rh(const SgmvArgs& a, int ksplit, hipStream_t stream) {
  int waves = 4;
  if (tuning().shrink_waves > 0) waves = tuning().shrink_waves;
  if (waves >= 16) return launch_rh_w<D, NB, MB, 16>(a, ksplit, stream);
  if (waves >= 8) return launch_rh_w<D, NB, MB, 8>(a, ksplit, stream);
  return launch_rh_w<D, NB, MB, 4>(a, ksplit, stream);
}

template <typename D, int NB>
static hipError_t launch_rh_nb(const SgmvArgs& a, hipStream_t stream) {
  const int mb = rh_row_blocks(a);
  const int ksplit = sgmv_shrink_ksplit(a);
  if constexpr (NB <= 4) {
    if (mb == 4) return launch_rh<D, NB, 4>(a, ksplit, stream);
  }
  if (mb >= 2) return launch_rh<D, NB, 2>(a, ksplit, stream);
  return launch_rh<D, NB, 1>(a, ksplit, stream);
}

template <typename D>
static hipError_t launch_shrink_dtype(const SgmvArgs& a, hipStream_t stream) {
  if (a.a_layout == LORAX_A_HR) {
    constexpr int RT = 4;
    const int64_t tiles = (a.num_tokens + RT - 1) / RT + a.num_segments;
    dim3 grid(static_cast<unsigned>(tiles < (1 << 20) ? tiles : (1 << 20)));
    hipLaunchKernelGGL((sgmv_shrink_hr_kernel<D, RT>), grid, dim3(256), 0, stream,
                       static_cast<typename D::E*>(a.y), static_cast<const typename D::E*>(a.x),
                       a.w_ptrs, a.s_start, a.s_end, a.num_segments,
                       static_cast<int>(a.num_tokens), a.d_in, a.d_out, a.layer_idx, a.scale, a.accumulate);
    return hipGetLastError();
  }
  if (a.d_out % 16 != 0) return hipErrorInvalidValue;  // the register-operand kernel works in 16-column blocks
  switch (a.d_out / 16) {
    case 1:
      return launch_rh_nb<D, 1>(a, stream);
    case 2:
      return launch_rh_nb<D, 2>(a, stream);
    case 3:
      return launch_rh_nb<D, 3>(a, stream);
    case 4:
      return launch_rh_nb<D, 4>(a, stream);
    case 5:
      return launch_rh_nb<D, 5>(a, stream);
    case 6:
      return launch_rh_nb<D, 6>(a, stream);
    case 7:
      return launch_rh_nb<D, 7>(a, stream);
    case 8:
      return launch_rh_nb<D, 8>(a, stream);
    default:
      return hipErrorInvalidValue;
  }
}

ShrinkRoute sgmv_shrink_route(const SgmvArgs& a) {
  if (a.d_out < 8 || a.d_out > 128 || a.d_out % 8 != 0 || a.d_in <= 0 || a.d_in % 8 != 0) return ShrinkRoute::kNone;
  if (a.a_layout == LORAX_A_HR) return ShrinkRoute::kNarrowRows;
  if (a.a_layout != LORAX_A_RH) return ShrinkRoute::kNone;
  // Up to a few hundred rows there are too few MFMA tiles to occupy the chip; the streaming kernel splits K
  // inside every workgroup instead of across workgroups (64 rows: 4.2 us against 10.4 us).
  const int rows_max = tuning().shrink_rows_max != 0 ? tuning().shrink_rows_max : 512;
  if (a.num_tokens <= rows_max) return ShrinkRoute::kRows;
  // The LDS-staged kernel is the faster one wherever it applies (h_in a multiple of 128).
  if (tuning().shrink_lds >= 0 && sgmv_shrink_lds_applies(a)) return ShrinkRoute::kLds;
  return a.d_out % 16 == 0 ? ShrinkRoute::kRegisters : ShrinkRoute::kNone;
}

hipError_t launch_sgmv_shrink(const SgmvArgs& a, hipStream_t stream) {
  switch (sgmv_shrink_route(a)) {
    case ShrinkRoute::kRows:
      return launch_sgmv_shrink_rows(a, stream);
    case ShrinkRoute::kLds:
      return launch_sgmv_shrink_lds(a, stream);
    case ShrinkRoute::kRegisters:
    case ShrinkRoute::kNarrowRows:
      return a.dtype == LORAX_F16 ? launch_shrink_dtype<F16>(a, stream) : launch_shrink_dtype<BF16>(a, stream);
    default:
      return hipErrorInvalidValue;
  }
}

}  // namespace lorax
