// SGMV shrink, LDS-staged variant for the [L, r, h_in] layout and hidden sizes that are a
// multiple of 128: v[s:e, :r] += T(x[s:e, :] @ A_i^T).
//
// Why it exists: in the register-only kernel (sgmv_shrink.hip) every wave instruction reads
// 16 rows x 64 bytes, rows a power-of-two number of bytes apart, and every wave fetches its own
// copy of the A fragments through L1.  Measured with the arithmetic removed, x alone streams at
// 3.3-3.7 TB/s in that pattern against 5.4-5.7 TB/s for contiguous 1 KB reads, and adding the
// (fully L2-resident) A fragments costs another 60 %: the L2 -> L1 path, not HBM and not the
// MFMAs, bounds that kernel.  Here a workgroup stages x and A tiles in LDS with direct-to-LDS
// loads (global_load_lds_dwordx4: 64 lanes x 16 B per instruction, four 256-byte row pieces), A
// is fetched once per workgroup instead of once per wave, and the MFMA operands come from LDS.
//
// Layout of one stage in LDS: x tile [ROWS][128 k] then A tile [R][128 k], rows of 256 bytes = 16
// chunks of 16 bytes; chunk q of row i is stored at position q ^ (i & 15), so the 16 lanes of one
// ds_read_b128 group (same chunk, 16 consecutive rows) hit 16 different bank groups - no padding,
// which direct-to-LDS loads could not produce anyway (a wave instruction writes 1 KB contiguously).
//
// Pipeline: STAGES buffers; the loads of the next STAGES-1 stages are in flight while one stage is
// multiplied.  Per K step one s_waitcnt vmcnt(N) (the wave's own loads of that stage have landed)
// and one s_barrier (everybody's have; everybody is done with the buffer about to be refilled).
// The barrier is a bare s_barrier: __syncthreads() would wait for ALL outstanding loads and
// serialise the pipeline.
#include <atomic>

#include "kernels.h"
#include "sgmv_tiles.h"

namespace lorax {

constexpr int kLdsKc = 128;             // k elements per stage
constexpr int kLdsRowBytes = kLdsKc * 2;
constexpr int kLdsThreads = 256;
constexpr int kLdsMaxStages = 8;
constexpr int kLdsMaxBytes = 156 * 1024;  // of the CU's 160 KB

#define LORAX_LDS __attribute__((address_space(3)))

// s_waitcnt vmcnt(N), N a compile-time constant (gfx9 encoding: vmcnt = simm16[3:0] | simm16[15:14] << 4)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  constexpr int n = N < 63 ? N : 63;  // 6-bit counter; waiting for fewer outstanding loads is always safe
  __builtin_amdgcn_s_waitcnt((n & 15) | ((n >> 4) << 14) | (7 << 4) | (15 << 8));
}

// Waits until at most `pending` groups of LOADS loads (the younger stages) are outstanding.
template <int LOADS>
__device__ __forceinline__ void wait_pending(int pending) {
  switch (pending) {
    case 0: wait_vmcnt<0>(); break;
    case 1: wait_vmcnt<LOADS>(); break;
    case 2: wait_vmcnt<2 * LOADS>(); break;
    case 3: wait_vmcnt<3 * LOADS>(); break;
    case 4: wait_vmcnt<4 * LOADS>(); break;
    case 5: wait_vmcnt<5 * LOADS>(); break;
    default: wait_vmcnt<6 * LOADS>(); break;
  }
}

template <typename D, int NB, int MBLK, bool KSPLIT>
__global__ __launch_bounds__(kLdsThreads) void sgmv_shrink_lds_kernel(
    const ShrinkGroup grp, const typename D::E* __restrict__ X, const int32_t* __restrict__ s_start,
    const int32_t* __restrict__ s_end, int num_segments, int num_tokens, int h_in, int64_t layer_idx,
    int stages, float scale, int accumulate_into_v, int rows_per_tile, int kparts, int tile_slots,
    float* __restrict__ partials, int rotate, const TileList plan) {
  using E = typename D::E;
  using vec8 = typename D::vec8;
  // The A tile stacks the A matrices of grp.count projections of rank r: row p * r + i is row i of
  // projection p, and column p * r + i of the result goes to projection p's v.  (One projection: the
  // plain shrink.)  NB = ceil(count * r / 16) rank blocks; r only needs to be a multiple of 8: rows of the
  // A tile past count * r re-read the last row and their columns of the result are not stored.
  const int r = grp.rank;
  constexpr int R = NB * 16;
  constexpr int ROWS = MBLK * 16;
  constexpr int kXBytes = ROWS * kLdsRowBytes;
  constexpr int kABytes = R * kLdsRowBytes;
  constexpr int kStageBytes = kXBytes + kABytes;
  constexpr int kXLoads = MBLK;  // 16-byte loads per thread and stage for x: ROWS * 16 chunks / 256 threads
  constexpr int kALoads = NB;
  constexpr int kLoads = kXLoads + kALoads;
  // Work split among the four waves.  KSPLIT: each wave multiplies one 32-wide k slice of every
  // stage for all blocks of the tile and the partial sums are added through LDS at the end (every
  // staged byte is read from LDS once).  Otherwise: waves as WM x WN over the (row block, rank
  // block) grid, each with its own output blocks and all k.
  // (three row blocks - 48-row tiles - only divide as 1 x 4, which needs the rank blocks to be a multiple of 4)
  constexpr int WN = KSPLIT ? 1 : (MBLK % 2 != 0 ? 4 : ((NB % 2 == 0) ? 2 : 1));
  constexpr int WM = KSPLIT ? 1 : 4 / WN;
  static_assert(KSPLIT || NB % WN == 0, "rank blocks must divide among the waves");
  static_assert(MBLK % WM == 0, "row blocks must divide among the waves");
  // KSPLIT: the partial sums (4 * MBLK * NB KB) go where the stage buffers are; the launcher sizes the LDS for it
  constexpr int MPW = MBLK / WM;  // row blocks per wave
  constexpr int NPW = NB / WN;    // rank blocks per wave
  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int c = lane & 15;
  const int g = lane >> 4;
  const int wm = KSPLIT ? 0 : wave % WM;
  const int wn = KSPLIT ? 0 : wave / WM;
  const VirtualBlock vb = xcd_virtual_block();
  // K split across workgroups (kparts > 1, launches with few row tiles): workgroup p * tile_slots + t multiplies
  // part p of the hidden dimension for tile t and leaves its fp32 sums in partials[p][row][R]; a second kernel
  // adds the parts in a fixed order.  Tiles are numbered fastest: neighbours (one XCD) read the same part of A.
  const int kpart = kparts > 1 ? vb.x / tile_slots : 0;
  const int first_tile = kparts > 1 ? vb.x - kpart * tile_slots : vb.x;
  const int st_begin = static_cast<int>(static_cast<int64_t>(kpart) * (h_in / kLdsKc) / kparts);
  const int nst = static_cast<int>(static_cast<int64_t>(kpart + 1) * (h_in / kLdsKc) / kparts) - st_begin;
  const int k_begin = st_begin * kLdsKc;

  // the projections' table entries of the first 64 segments travel with the tile's own loads (sgmv_tiles.h)
  int64_t pre_w[kMaxShrinkGroup];
#pragma unroll
  for (int p = 0; p < kMaxShrinkGroup; ++p) pre_w[p] = preload_segment_entry(grp.w[p < grp.count ? p : 0], num_segments);

  for (int tile = first_tile;; tile += gridDim.x) {
    if (kparts > 1 && tile != first_tile) break;  // one tile per workgroup when K is split
    RowTile rt;
    // tiles may be lower than the ROWS the buffers hold: rows past a tile's end re-read its last row
    if (!get_row_tile(plan, s_start, s_end, num_segments, num_tokens, rows_per_tile, tile, rt)) break;
    const E* A[kMaxShrinkGroup];
    int64_t stack0 = 0;
    bool missing = false;
#pragma unroll
    for (int p = 0; p < kMaxShrinkGroup; ++p) {
      const int64_t stack = segment_entry(pre_w[p], grp.w[p < grp.count ? p : 0], rt.seg);
      if (p == 0) stack0 = stack;
      missing = missing || stack == 0;
      A[p] = reinterpret_cast<const E*>(stack) + layer_idx * r * static_cast<int64_t>(h_in);
    }
    // (a caller's plan that names a segment without a stack: nothing to multiply; the search never yields one)
    if (plan.records != nullptr && missing) break;

    // Source addresses of this thread's chunks.  Load j of a thread covers chunk id j * 256 + tid of
    // the tile: row = id / 16, position = id % 16, and it fetches the row's chunk position ^ (row & 15).
    const E* xsrc[kXLoads];
    const E* asrc[kALoads];
#pragma unroll
    for (int j = 0; j < kXLoads; ++j) {
      const int id = j * kLdsThreads + tid;
      const int row = id >> 4;
      const int grow = min(rt.row0 + row, rt.row_end - 1);  // rows past the tile re-read its last row
      xsrc[j] = X + static_cast<int64_t>(grow) * h_in + k_begin + (((id & 15) ^ (row & 15)) << 3);
    }
#pragma unroll
    for (int j = 0; j < kALoads; ++j) {
      const int id = j * kLdsThreads + tid;
      const int row = id >> 4;
      int proj = row / r, arow = row - proj * r;
      if (proj >= grp.count) proj = grp.count - 1, arow = r - 1;
      const E* Ap = proj == 0 ? A[0] : (proj == 1 ? A[1] : (proj == 2 ? A[2] : A[3]));
      asrc[j] = Ap + static_cast<int64_t>(arow) * h_in + k_begin + (((id & 15) ^ (row & 15)) << 3);
    }
    // Where this tile starts its walk over the hidden dimension (it wraps round).  Workgroups that all walk from
    // k = 0 ask for the same 256-byte column of rows a power-of-two-ish number of bytes apart at the same time,
    // i.e. for the same few memory channels: x alone then streams at 4.0-5.3 TB/s for row lengths of 16, 28, 32
    // or 56 KB where staggered walks reach 6.0-6.5 TB/s.  The tiles of one segment that run on one XCD stay
    // within a few stages of each other, so that they still find the segment's A tiles in that XCD's L2.
    // Tiles that read the same stack of A (one adapter, whatever the segment) keep the same start.
    const unsigned who = static_cast<unsigned>(static_cast<uint64_t>(stack0) >> 12) * 2654435761u >> 20;
    const int rot = rotate ? static_cast<int>((37u * (who * kXcds + blockIdx.x % kXcds) +
                                               static_cast<unsigned>(rt.index) % 8u) % static_cast<unsigned>(nst))
                           : 0;
    auto issue = [&](int st, int slot) {
      char* buf = lds + slot * kStageBytes;
      const int sr = st + rot;
      const int k = (sr >= nst ? sr - nst : sr) * kLdsKc;
#pragma unroll
      for (int j = 0; j < kXLoads; ++j)
        __builtin_amdgcn_global_load_lds((const LORAX_GLOBAL void*)(xsrc[j] + k),
                                         (LORAX_LDS void*)(buf + (j * kLdsThreads + wave * kWave) * 16), 16, 0, 0);
#pragma unroll
      for (int j = 0; j < kALoads; ++j)
        __builtin_amdgcn_global_load_lds((const LORAX_GLOBAL void*)(asrc[j] + k),
                                         (LORAX_LDS void*)(buf + kXBytes + (j * kLdsThreads + wave * kWave) * 16), 16,
                                         0, 0);
    };

    f32x4 acc[MPW][NPW];
#pragma unroll
    for (int mb = 0; mb < MPW; ++mb)
#pragma unroll
      for (int nb = 0; nb < NPW; ++nb) acc[mb][nb] = f32x4{0.f, 0.f, 0.f, 0.f};

    // all waves must be done reading the previous tile's buffers before they are refilled
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    for (int s = 0; s < stages - 1; ++s)
      if (s < nst) issue(s, s);

    int slot = 0;            // buffer holding stage st
    int fill = stages - 1;   // buffer the next issued stage goes to
    for (int st = 0; st < nst; ++st) {
      // the loads of stage st were issued stages-1 steps ago; up to stages-2 later stages are pending
      wait_pending<kLoads>(min(stages - 2, nst - 1 - st));
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      if (st + stages - 1 < nst) issue(st + stages - 1, fill);
      const char* xb = lds + slot * kStageBytes;
      const char* ab = xb + kXBytes;
      slot = slot + 1 == stages ? 0 : slot + 1;
      fill = fill + 1 == stages ? 0 : fill + 1;
#pragma unroll
      for (int jj = 0; jj < (KSPLIT ? 1 : kLdsKc / 32); ++jj) {
        const int j = KSPLIT ? wave : jj;
        const int q = ((j * 4 + g) ^ c) * 16;  // swizzled chunk position of this lane's 8 k
        vec8 xf[MPW], af[NPW];
#pragma unroll
        for (int mb = 0; mb < MPW; ++mb)
          xf[mb] = *reinterpret_cast<const vec8*>(xb + ((wm * MPW + mb) * 16 + c) * kLdsRowBytes + q);
#pragma unroll
        for (int nb = 0; nb < NPW; ++nb)
          af[nb] = *reinterpret_cast<const vec8*>(ab + ((wn * NPW + nb) * 16 + c) * kLdsRowBytes + q);
#pragma unroll
        for (int mb = 0; mb < MPW; ++mb)
#pragma unroll
          for (int nb = 0; nb < NPW; ++nb) acc[mb][nb] = D::mfma16(af[nb], xf[mb], acc[mb][nb]);
      }
    }

    // acc[mb][nb][i] of lane (g, c) is D[n = nblock*16 + 4g + i][row = mblock*16 + c].
    // Four adjacent columns of one row (r is a multiple of 8: they belong to one projection).
    auto store4 = [&](int row, int col, f32x4 sum) {
      const int proj = col / r;
      if (kparts > 1) {
        if (row < rt.row_end && proj < grp.count)
          *reinterpret_cast<f32x4*>(partials + (static_cast<int64_t>(kpart) * num_tokens + row) * R + col) = sum;
      } else if (row < rt.row_end && proj < grp.count) {
        E* Vp = static_cast<E*>(proj == 0 ? grp.v[0] : (proj == 1 ? grp.v[1] : (proj == 2 ? grp.v[2] : grp.v[3])));
        update4<D>(accumulate_into_v != 0, Vp + static_cast<int64_t>(row) * r + (col - proj * r), sum * scale);
      }
    };
    if constexpr (KSPLIT) {
      // Partial sums of the four waves meet in LDS (the stage buffers are free: the last stage was
      // waited for with no load outstanding), then the 256 threads share the blocks' elements.
      f32x4* red = reinterpret_cast<f32x4*>(lds);
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
      for (int mb = 0; mb < MBLK; ++mb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) red[(wave * MBLK * NB + mb * NB + nb) * kWave + lane] = acc[mb][nb];
      __syncthreads();
      for (int i = tid; i < MBLK * NB * kWave; i += kLdsThreads) {
        const int blk = i / kWave, l = i % kWave;
        f32x4 sum = red[i];
#pragma unroll
        for (int w = 1; w < 4; ++w) {
          const f32x4 part = red[w * MBLK * NB * kWave + i];
          sum[0] += part[0]; sum[1] += part[1]; sum[2] += part[2]; sum[3] += part[3];
        }
        const int row = rt.row0 + (blk / NB) * 16 + (l & 15);
        const int col = (blk % NB) * 16 + 4 * (l >> 4);
        store4(row, col, sum);
      }
    } else {
      // every wave owns its output blocks: no cross-wave reduction
#pragma unroll
      for (int mb = 0; mb < MPW; ++mb) {
        const int row = rt.row0 + (wm * MPW + mb) * 16 + c;
        if (row < rt.row_end) {
#pragma unroll
          for (int nb = 0; nb < NPW; ++nb) {
            const int col = (wn * NPW + nb) * 16 + 4 * g;
            store4(row, col, acc[mb][nb]);
          }
        }
      }
    }
  }
}

// Second pass of a launch that split K across workgroups: adds the parts of every row of every tile in a fixed
// order and finishes the row exactly as the one-pass kernel does (scale, round, add or overwrite).
template <typename D>
__global__ __launch_bounds__(kLdsThreads) void sgmv_shrink_parts_kernel(
    const ShrinkGroup grp, const float* __restrict__ partials, const int32_t* __restrict__ s_start,
    const int32_t* __restrict__ s_end, int num_segments, int num_tokens, int R, int kparts, float scale,
    int accumulate_into_v, int rows_per_tile, const TileList plan) {
  using E = typename D::E;
  const int r = grp.rank;
  const int n4 = grp.count * r / 4;  // groups of 4 adjacent columns per row (r is a multiple of 8)
  for (int tile = blockIdx.x;; tile += gridDim.x) {
    RowTile rt;
    if (!get_row_tile(plan, s_start, s_end, num_segments, num_tokens, rows_per_tile, tile, rt)) break;
    const int n = (rt.row_end - rt.row0) * n4;
    for (int i = threadIdx.x; i < n; i += kLdsThreads) {
      const int row = rt.row0 + i / n4;
      const int col = (i % n4) * 4;
      f32x4 sum = *reinterpret_cast<const f32x4*>(partials + static_cast<int64_t>(row) * R + col);
      for (int p = 1; p < kparts; ++p) {
        const f32x4 part =
            *reinterpret_cast<const f32x4*>(partials + (static_cast<int64_t>(p) * num_tokens + row) * R + col);
        sum[0] += part[0]; sum[1] += part[1]; sum[2] += part[2]; sum[3] += part[3];
      }
      const int proj = col / r;
      E* Vp = static_cast<E*>(proj == 0 ? grp.v[0] : (proj == 1 ? grp.v[1] : (proj == 2 ? grp.v[2] : grp.v[3])));
      update4<D>(accumulate_into_v != 0, Vp + static_cast<int64_t>(row) * r + (col - proj * r), sum * scale);
    }
  }
}

// ---------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------
// Raising the dynamic LDS limit is needed once per kernel instantiation and device (the current one).
template <typename D, int NB, int MBLK, bool KSPLIT>
static hipError_t raise_lds_limit() {
  static std::atomic<bool> configured[64] = {};  // callers may come from several host threads
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return e;
  if (device >= 0 && device < 64 && configured[device].load(std::memory_order_acquire)) return hipSuccess;
  e = hipFuncSetAttribute(reinterpret_cast<const void*>(sgmv_shrink_lds_kernel<D, NB, MBLK, KSPLIT>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, kLdsMaxBytes);
  if (e != hipSuccess) return e;
  if (device >= 0 && device < 64) configured[device].store(true, std::memory_order_release);
  return hipSuccess;
}

// What a launch looks like: decided from host-known sizes only (and from the caller's tile plan, which knows the
// tiles exactly), so that the same call always runs the same way.
struct LdsLaunch {
  int mblk;           // 16-row blocks of the stage buffers (1, 2, 3, 4)
  bool kslices;       // the four waves split the k slices of a stage (else the output blocks)
  int rows_per_tile;  // tile height, at most 16 * mblk
  int64_t tiles;      // row tiles: exact with a plan, else an upper bound
  bool planned;
  int kparts;         // parts the hidden dimension is cut into across workgroups (1 = none)
};

// `room`: bytes of scratch for the K parts' fp32 sums.
static LdsLaunch lds_launch_shape(const SgmvArgs& a, size_t room) {
  const int NB = (a.d_out + 15) / 16;
  LdsLaunch l{};
  const bool kslices_pref = tuning().shrink_lds != 2;
  l.planned = a.tiles != nullptr && a.num_tiles > 0 && a.tile_rows >= 1 && a.tile_rows <= 64 && tuning().shrink_mb == 0;
  if (l.planned) {
    // the plan's tiles in buffers just high enough; the waves take k slices wherever that variant exists
    l.mblk = (a.tile_rows + 15) / 16;
    l.rows_per_tile = l.mblk * 16;
    l.kslices = l.mblk != 4 || NB <= 4;
    l.tiles = a.num_tiles;
  } else {
    // Row-tile height: the tallest of 64 / 32 / 16 rows that still yields 128 tiles (a workgroup streams about
    // 50 GB/s, so fewer, larger tiles leave HBM idle) and is not much taller than the average segment (rows past a
    // segment's end are padding).  Short tiles re-read A more often, but from L2.
    const int64_t avg_len = a.num_tokens / (a.num_segments > 0 ? a.num_segments : 1);
    int mblk = 4;
    while (mblk > 1 && ((a.num_tokens + mblk * 16 - 1) / (mblk * 16) + a.num_segments < 128 || mblk * 8 > avg_len))
      mblk /= 2;
    if (tuning().shrink_mb > 0) mblk = tuning().shrink_mb;
    if (mblk != 1 && mblk != 2 && mblk != 4) mblk = 1;
    // every staged byte read from LDS once (k slices per wave) up to rank 64 in 64-row buffers; above, the waves
    // split the output blocks instead (k slices at rank 128 need 128 accumulator registers per lane and measured
    // no faster)
    l.mblk = mblk;
    l.kslices = mblk == 4 ? (NB <= 4 && kslices_pref) : (mblk == 2 ? !(NB % 2 == 0 && !kslices_pref) : true);
    // A launch streams at the rate of the CUs that have a workgroup, so when the full-height tiles are fewer than
    // the 256 CUs the tiles are lowered (in steps of 16 rows) until they are about as many.  The host knows the
    // rows and the number of segments, not their lengths: ceil(T / M) + segments bounds the count.
    int rows = mblk * 16;
    if (tuning().shrink_rows <= 0) {
      while (rows > 16 && (a.num_tokens + rows - 17) / (rows - 16) + a.num_segments <= 256) rows -= 16;
    } else if (tuning().shrink_rows < rows) {
      rows = (tuning().shrink_rows + 15) / 16 * 16;
    }
    // Tiles of 48 rows in buffers of 48: the fourth row block of 64-row buffers would be staged (re-reading the
    // tile's last row) and multiplied for nothing.  With three row blocks the waves take k slices at every rank
    // (96 accumulator registers per lane at rank 128; a stacked gate/up launch of rank 128 37.0 -> 34.8 us
    // against the waves splitting the output blocks).
    if (mblk == 4 && rows == 48 && tuning().shrink_mb == 0 && (l.kslices || NB > 4 || NB % 4 == 0)) {
      l.mblk = 3;
      l.kslices = l.kslices || NB > 4;
    }
    l.rows_per_tile = rows;
    l.tiles = (a.num_tokens + rows - 1) / rows + a.num_segments;
  }
  // K parts: a workgroup streams its tile's x and A at about 50 GB/s whatever the launch, so a launch of a
  // hundred tiles (a prefill batch of one or two thousand rows) leaves most of the chip idle.  Its hidden
  // dimension is cut into parts of at least 8 stages and a second small launch adds the parts.  Up to 128 tiles:
  // about one workgroup per CU (two measured no faster).  Up to 192 tiles (a single long run of a few thousand
  // rows cut into 32-row tiles): two or three parts, about two workgroups per CU - measured on a 4096-row run at
  // rank 128, 140 tiles: 51 -> 40 us over h_in = 8192 and 145 -> 86 us over h_in = 28672 with three parts (two: 45
  // and 116 us; four and more, which no longer fit the CUs at once: 46 and 104 us).  Launches with more tiles
  // than that are slower with parts than without (254 tiles in two parts: 27 against 23 us).  Needs the scratch
  // (fp32 sums, kparts x rows x R).
  const int R = NB * 16;
  const int nst_all = a.d_in / kLdsKc;
  l.kparts = 1;
  if (a.partials != nullptr && !fixed_order_shrink() && (l.tiles < 192 || tuning().shrink_ksplit > 0)) {
    // (a 4096-row run at rank 128 planned as exactly 128 tiles: 41 us in two parts, one workgroup per CU, against
    // 48 us in three)
    const int64_t nt = l.tiles > 0 ? l.tiles : 1;
    int kparts = static_cast<int>(nt <= 128 ? 256 / nt : 512 / nt);
    if (kparts > 8) kparts = 8;
    if (kparts > nst_all / 8) kparts = nst_all / 8;
    if (tuning().shrink_ksplit > 0) kparts = tuning().shrink_ksplit < nst_all ? tuning().shrink_ksplit : nst_all;
    while (kparts > 1 && static_cast<size_t>(kparts) * a.num_tokens * R * sizeof(float) > room) --kparts;
    l.kparts = kparts < 1 ? 1 : kparts;
  }
  return l;
}

template <typename D, int NB, int MBLK, bool KSPLIT>
static hipError_t launch_lds_m(const SgmvArgs& a, const LdsLaunch& l, hipStream_t stream) {
  constexpr int kStageBytes = (MBLK + NB) * 16 * kLdsRowBytes;
  constexpr int kRedBytes = KSPLIT ? 4 * MBLK * NB * 1024 : 0;  // partial sums of the four waves at the end of a tile
  static_assert(kRedBytes <= kLdsMaxBytes, "partial sums must fit in LDS");
  constexpr int R = NB * 16;
  const int64_t tiles = l.tiles;
  const int kparts = l.kparts;
  const int64_t wgs = tiles * kparts;
  // Stage buffers: all of a CU's LDS when there is at most one workgroup per CU; a third of it when the
  // workgroups make one to three rounds over the CUs (more resident workgroups even out the last round);
  // half of it for long launches.  2 to 8 stages.
  int budget = wgs <= 256 ? 150 * 1024 : (wgs <= 768 ? 50 * 1024 : 76 * 1024);
  if (tuning().shrink_lds_kb > 0) budget = tuning().shrink_lds_kb * 1024;
  int stages = budget / kStageBytes;
  stages = stages < 2 ? 2 : (stages > kLdsMaxStages ? kLdsMaxStages : stages);
  static_assert(2 * kStageBytes <= kLdsMaxBytes, "two stages must fit in LDS");
  while (stages * kStageBytes > kLdsMaxBytes) --stages;
  int lds_bytes = stages * kStageBytes;
  if (lds_bytes < kRedBytes) lds_bytes = kRedBytes;
  auto kernel = sgmv_shrink_lds_kernel<D, NB, MBLK, KSPLIT>;
  // lorax_init has raised the dynamic LDS limit of every instantiation; a caller that skipped it gets it here.
  if (hipError_t e = raise_lds_limit<D, NB, MBLK, KSPLIT>(); e != hipSuccess) return e;
  dim3 grid(static_cast<unsigned>(kparts > 1 ? wgs : (tiles < (1 << 20) ? tiles : (1 << 20))));
  ShrinkGroup grp = a.group;
  if (grp.count <= 1) {
    grp = ShrinkGroup{};
    grp.v[0] = a.y;
    grp.w[0] = a.w_ptrs;
    grp.count = 1;
    grp.rank = a.d_out;
  }
  const TileList plan{l.planned ? a.tiles : nullptr, l.planned ? a.num_tiles : 0, l.rows_per_tile};
  const int rotate = (tuning().shrink_no_rotate || fixed_order_shrink()) ? 0 : 1;
  hipLaunchKernelGGL(kernel, grid, dim3(kLdsThreads), lds_bytes, stream, grp, static_cast<const typename D::E*>(a.x),
                     a.s_start, a.s_end, a.num_segments, static_cast<int>(a.num_tokens), a.d_in, a.layer_idx, stages,
                     a.scale, a.accumulate, l.rows_per_tile, kparts, static_cast<int>(tiles), a.partials, rotate, plan);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess || kparts == 1) return e;
  hipLaunchKernelGGL(sgmv_shrink_parts_kernel<D>, dim3(static_cast<unsigned>(tiles)), dim3(kLdsThreads), 0, stream, grp,
                     a.partials, a.s_start, a.s_end, a.num_segments, static_cast<int>(a.num_tokens), R, kparts, a.scale,
                     a.accumulate, l.rows_per_tile, plan);
  return hipGetLastError();
}

template <typename D, int NB>
static hipError_t launch_lds_nb(const SgmvArgs& a, hipStream_t stream) {
  // (the first 8 MiB of the scratch whatever the buffer's size, so that the result does not depend on it)
  const LdsLaunch l = lds_launch_shape(a, a.partial_bytes < kPartialBytes ? a.partial_bytes : kPartialBytes);
  switch (l.mblk) {
    case 4:
      if constexpr (NB <= 4) {
        if (l.kslices) return launch_lds_m<D, NB, 4, true>(a, l, stream);
      }
      return launch_lds_m<D, NB, 4, false>(a, l, stream);
    case 3:
      if constexpr (NB <= 4 && NB % 4 == 0) {
        if (!l.kslices) return launch_lds_m<D, NB, 3, false>(a, l, stream);
      }
      return launch_lds_m<D, NB, 3, true>(a, l, stream);
    case 2:
      if constexpr (NB % 2 == 0) {
        if (!l.kslices) return launch_lds_m<D, NB, 2, false>(a, l, stream);
      }
      return launch_lds_m<D, NB, 2, true>(a, l, stream);
    default:
      return launch_lds_m<D, NB, 1, true>(a, l, stream);
  }
}

template <typename D>
static hipError_t launch_lds_dtype(const SgmvArgs& a, hipStream_t stream) {
  switch ((a.d_out + 15) / 16) {
    case 1:
      return launch_lds_nb<D, 1>(a, stream);
    case 2:
      return launch_lds_nb<D, 2>(a, stream);
    case 3:
      return launch_lds_nb<D, 3>(a, stream);
    case 4:
      return launch_lds_nb<D, 4>(a, stream);
    case 5:
      return launch_lds_nb<D, 5>(a, stream);
    case 6:
      return launch_lds_nb<D, 6>(a, stream);
    case 7:
      return launch_lds_nb<D, 7>(a, stream);
    case 8:
      return launch_lds_nb<D, 8>(a, stream);
    default:
      return hipErrorInvalidValue;
  }
}

// Every instantiation launch_lds_nb can reach, for the per-device set-up: the same case analysis as the launchers.
template <typename D, int NB>
static hipError_t raise_lds_limits_nb() {
  hipError_t e = hipSuccess;
  auto also = [&](hipError_t r) { if (e == hipSuccess) e = r; };
  if constexpr (NB <= 4) {
    also(raise_lds_limit<D, NB, 4, true>());
    also(raise_lds_limit<D, NB, 3, true>());
  }
  also(raise_lds_limit<D, NB, 4, false>());
  if constexpr (NB > 4) also(raise_lds_limit<D, NB, 3, true>());
  else if constexpr (NB % 4 == 0) also(raise_lds_limit<D, NB, 3, false>());
  if constexpr (NB % 2 == 0) also(raise_lds_limit<D, NB, 2, false>());
  also(raise_lds_limit<D, NB, 2, true>());
  also(raise_lds_limit<D, NB, 1, true>());
  return e;
}
template <typename D>
static hipError_t raise_lds_limits_dtype() {
  hipError_t e = hipSuccess;
  auto also = [&](hipError_t r) { if (e == hipSuccess) e = r; };
  also(raise_lds_limits_nb<D, 1>());
  also(raise_lds_limits_nb<D, 2>());
  also(raise_lds_limits_nb<D, 3>());
  also(raise_lds_limits_nb<D, 4>());
  also(raise_lds_limits_nb<D, 5>());
  also(raise_lds_limits_nb<D, 6>());
  also(raise_lds_limits_nb<D, 7>());
  also(raise_lds_limits_nb<D, 8>());
  return e;
}
hipError_t configure_sgmv_shrink_lds() {
  const hipError_t e = raise_lds_limits_dtype<F16>();
  return e != hipSuccess ? e : raise_lds_limits_dtype<BF16>();
}

int sgmv_shrink_lds_kparts(const SgmvArgs& a, size_t room) { return lds_launch_shape(a, room).kparts; }

bool sgmv_shrink_lds_applies(const SgmvArgs& a) {
  return a.a_layout == LORAX_A_RH && a.d_in % kLdsKc == 0 && a.d_out % 8 == 0 && a.d_out >= 8 && a.d_out <= 128;
}

hipError_t launch_sgmv_shrink_lds(const SgmvArgs& a, hipStream_t stream) {
  return a.dtype == LORAX_F16 ? launch_lds_dtype<F16>(a, stream) : launch_lds_dtype<BF16>(a, stream);
}

}  // namespace lorax
