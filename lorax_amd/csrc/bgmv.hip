// BGMV for gfx950: per-token gathered LoRA matrix-vector products for decode batches.
//
// Semantics follow the reference kernels in punica_kernels/bgmv/bgmv_impl.cuh:
//   shrink (:15-143):  v[b, j] += T(scale * sum_k A[idx][layer, j, k] * x[b, k])
//   expand (:146-192): y[b, j] += T(scale * sum_k B[idx][layer, j, k] * v[b, k])
// for every token b whose idx = indices[b] is >= 0 (:24-27, :157-159).
//
// The reference launches one block per (output element, token) for shrink and one
// per (32 outputs, token) for expand, so every token re-reads its adapter's weights.
// Here the tokens of one adapter are grouped inside the kernel (group_tokens) and a
// workgroup streams the adapter's rows once for up to kGroup tokens, with 16-byte
// loads, fp32 accumulation in registers and one wave reduction per output.
#include <utility>

#include "kernels.h"
#include "sgmv_tiles.h"

namespace lorax {

constexpr int kBgmvThreads = 256;
constexpr int kGroup = 4;  // tokens sharing one pass over an adapter's weights

template <int N>
struct Pow2Ceil {
  static constexpr int value = N <= 1 ? 1 : 2 * Pow2Ceil<(N + 1) / 2>::value;
};

// ---------------------------------------------------------------------------------
// Shrink: rows of A are h_in long (thousands of elements); a workgroup owns RS rows
// of one adapter and NT tokens and walks the hidden dimension once.
// ---------------------------------------------------------------------------------
template <typename D, int RS, int NT>
__device__ __forceinline__ void bgmv_shrink_body(typename D::E* __restrict__ Y,
                                                 const typename D::E* __restrict__ X,
                                                 const typename D::E* __restrict__ A,
                                                 const int (&toks)[kGroup], int h_in, int row0,
                                                 int64_t y_offset, int64_t y_stride, float scale,
                                                 bool accumulate_into_y, float* red) {
  using vec8 = typename D::vec8;
  using E = typename D::E;
  const int tid = threadIdx.x;

  // The thread that will write output (j, g) fetches the old value now, so that the
  // read-modify-write at the end does not add a memory round trip.
  E* yp = nullptr;
  E y_old = static_cast<E>(0.f);
  if (tid < RS * NT) {
    const int j = tid / NT;
    const int g = tid % NT;
    int tok = toks[0];
#pragma unroll
    for (int q = 1; q < NT; ++q)
      if (g == q) tok = toks[q];
    yp = Y + static_cast<int64_t>(tok) * y_stride + y_offset + row0 + j;
    if (accumulate_into_y) y_old = *yp;
  }

  float acc[RS][NT];
#pragma unroll
  for (int j = 0; j < RS; ++j)
#pragma unroll
    for (int g = 0; g < NT; ++g) acc[j][g] = 0.f;

  const E* xrow[NT];
#pragma unroll
  for (int g = 0; g < NT; ++g) xrow[g] = X + static_cast<int64_t>(toks[g]) * h_in;

  // Two hidden-dimension steps per trip: all loads of the trip are issued before the first
  // one is consumed (the scheduling barrier keeps the compiler from sinking them to their
  // uses), so a trip costs one memory round trip instead of one per row.
  constexpr int kStep = kBgmvThreads * 8;
  for (int k = tid * 8; k < h_in; k += 2 * kStep) {
    vec8 xv[2][NT];
    vec8 wv[2][RS];
    const bool second = k + kStep < h_in;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int ku = k + u * kStep;
#pragma unroll
      for (int g = 0; g < NT; ++g) xv[u][g] = (u == 0 || second) ? load8<D>(xrow[g] + ku) : zero8<D>();
#pragma unroll
      for (int j = 0; j < RS; ++j)
        wv[u][j] = (u == 0 || second) ? load8<D>(A + static_cast<int64_t>(j) * h_in + ku) : zero8<D>();
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int j = 0; j < RS; ++j)
#pragma unroll
        for (int g = 0; g < NT; ++g) acc[j][g] = dot8<D>(wv[u][j], xv[u][g], acc[j][g]);
  }

  // Wave reduction of the RS*NT sums, then across the four waves through LDS.
  constexpr int NV = Pow2Ceil<RS * NT>::value;
  float vals[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) vals[i] = 0.f;
#pragma unroll
  for (int j = 0; j < RS; ++j)
#pragma unroll
    for (int g = 0; g < NT; ++g) vals[j * NT + g] = acc[j][g];
  transpose_reduce<NV>(vals);
  const int lane = lane_id();
  const int wave = tid / kWave;
  if ((lane & (kWave / NV - 1)) == 0) red[wave * NV + transpose_reduce_index<NV>(lane)] = vals[0];
  __syncthreads();
  if (tid < RS * NT) {
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < kBgmvThreads / kWave; ++w) s += red[w * NV + tid];
    *yp = accumulate<D>(y_old, s * scale);
  }
}

// Problem, token chunk and row block / column slice of this workgroup (see BgmvBatch).  Wave-uniform.
struct BatchSlot {
  int problem, chunk, sub;
};
__device__ __forceinline__ BatchSlot batch_slot(const BgmvBatch& batch, int count) {
  const int v = static_cast<int>(xcd_virtual_id());
  if (count == 1) {  // the drop-in single-problem call: no table walk in front of the first useful load
    const int subs = batch.run_subs[0];
    return BatchSlot{0, v / subs, v % subs};
  }
  // Lane i looks at problem i: the five table entries of all problems arrive in one trip to the kernel arguments
  // (a walk with the scalar unit asks for them one after the other, each answer deciding the next question - a
  // handful of dependent cache misses in front of the first useful load of every CU's first workgroup).
  const int i = lane_id() < kMaxBgmvProblems ? lane_id() : kMaxBgmvProblems - 1;
  const int run_end = batch.run_end[i], base = batch.base[i], subs = batch.run_subs[i];
  const int sub_lo = batch.sub_lo[i], sub_hi = batch.sub_hi[i];
  const bool mine = lane_id() < kMaxBgmvProblems && i + 1 < count;
  // first problem of the run that holds v: run_end does not decrease with the problem number
  const int first = __popcll(__ballot(mine && v >= run_end));
  const int rem = v - read_lane(base, first);
  const int run_subs = read_lane(subs, first);
  const int chunk = rem / run_subs, s = rem % run_subs;
  // inside the run, sub_hi increases and the run's last problem has sub_hi = run_subs > s
  const int run_stop = read_lane(run_end, first);
  const int p = first + __popcll(__ballot(mine && i >= first && run_end == run_stop && s >= sub_hi));
  return BatchSlot{p, chunk, s - read_lane(sub_lo, p)};
}

// Problem `p` of a batch, fetched the same way: lane i asks for the fields of problem i before anybody knows p,
// and the fields of the problem the workgroup turns out to serve are read from that lane.  Indexing the kernel
// arguments with p instead is one more dependent trip to memory in front of the routing record.  Wave-uniform.
// Used by the single-launch kernels, whose workgroups are alone on their CU (9.8 -> 9.2 us per decode launch);
// in the shrink and expand kernels the seventeen registers it holds cost a wave per SIMD and more than it saves
// (expand 27.0 -> 28.3 us on the mixed-rank decode batch), so they index the arguments.
__device__ __forceinline__ int64_t read_lane64(int64_t v, int src) {
  const uint32_t lo = static_cast<uint32_t>(read_lane(static_cast<int>(static_cast<uint32_t>(v)), src));
  const uint32_t hi = static_cast<uint32_t>(read_lane(static_cast<int>(static_cast<uint64_t>(v) >> 32), src));
  return static_cast<int64_t>((static_cast<uint64_t>(hi) << 32) | lo);
}
struct ProblemFields {  // one lane's copy of problem min(lane, 15)
  int64_t y, x, w_ptrs, indices, y_offset, y_stride, plan;
  int width, narrow, num_groups;
};
__device__ __forceinline__ ProblemFields preload_problems(const BgmvBatch& batch) {
  const BgmvProblem& q = batch.p[lane_id() < kMaxBgmvProblems ? lane_id() : kMaxBgmvProblems - 1];
  return ProblemFields{reinterpret_cast<int64_t>(q.y), reinterpret_cast<int64_t>(q.x),
                       reinterpret_cast<int64_t>(q.w_ptrs), reinterpret_cast<int64_t>(q.indices), q.y_offset,
                       q.y_stride, reinterpret_cast<int64_t>(q.plan), q.width, q.narrow, q.num_groups};
}
__device__ __forceinline__ BgmvProblem select_problem(const ProblemFields& f, int p) {
  BgmvProblem P;
  P.y = reinterpret_cast<void*>(read_lane64(f.y, p));
  P.x = reinterpret_cast<const void*>(read_lane64(f.x, p));
  P.w_ptrs = reinterpret_cast<const int64_t*>(read_lane64(f.w_ptrs, p));
  P.indices = reinterpret_cast<const int64_t*>(read_lane64(f.indices, p));
  P.y_offset = read_lane64(f.y_offset, p);
  P.y_stride = read_lane64(f.y_stride, p);
  P.width = read_lane(f.width, p);
  P.narrow = read_lane(f.narrow, p);
  P.plan = reinterpret_cast<const int64_t*>(read_lane64(f.plan, p));
  P.num_groups = read_lane(f.num_groups, p);
  return P;
}

// The two fields of a problem that stand between batch_slot and the routing record, fetched like batch_slot's
// tables (lane i: problem i) and with them: the record's address is then known one trip to memory after the
// workgroup starts, and the record travels together with the problem's other fields, which the scalar unit reads
// from the kernel arguments once the problem's number is known.
struct PlanOfLane {
  int64_t plan;
  int num_groups;
};
__device__ __forceinline__ PlanOfLane preload_plans(const BgmvBatch& batch) {
  const BgmvProblem& q = batch.p[lane_id() < kMaxBgmvProblems ? lane_id() : kMaxBgmvProblems - 1];
  return PlanOfLane{reinterpret_cast<int64_t>(q.plan), q.num_groups};
}

// Resolves the token chunk of workgroup row `row` and the address of its adapter's stack.
// With a routing plan (built once per batch next to the index tables) this is one 64-byte
// record: [ntok, tok0..tok3, address of the A stack, address of the B^T stack, reserved];
// without one, the chunk is found by scanning indices[] (group_tokens).  Returns the number of
// tokens, 0 if the workgroup has nothing to do.  Wave-uniform.
// `plan` / `num_groups` are the problem's fields of that name, handed over separately because the callers have
// them before the rest of the problem (PlanOfLane).
__device__ __forceinline__ int resolve_chunk(const BgmvProblem& P, const int64_t* plan, int num_groups, int num_tokens,
                                             bool expand, int row, int (&toks)[kGroup], int64_t& stack_addr) {
  if (plan != nullptr) {
    if (row >= num_groups) return 0;
    const int64_t* rec = plan + static_cast<int64_t>(row) * kPlanRecordWords;
    const int n = static_cast<int>(rec[0]);
#pragma unroll
    for (int g = 0; g < kGroup; ++g) toks[g] = static_cast<int>(rec[1 + g]);
    stack_addr = rec[expand ? 6 : 5];
    // Stacked weights ([num_adapters, r, h_in] / [num_adapters, h_out, r] tensors, one entry per adapter): the
    // record names the entry, not its address; a planned problem carries the tensors' bases in the table fields
    // it has no other use for.
    const int64_t base = expand ? reinterpret_cast<int64_t>(P.indices) : reinterpret_cast<int64_t>(P.w_ptrs);
    if (base != 0) stack_addr = base + stack_addr * P.narrow * static_cast<int64_t>(P.width) * 2;
    return n;
  }
  int64_t idx;
  const int n = group_tokens<kGroup>(P.indices, num_tokens, row, idx, toks);
  if (n == 0) return 0;
  stack_addr = P.w_ptrs[idx];
  return n;
}

template <typename D, int RS>
__global__ __launch_bounds__(kBgmvThreads) void bgmv_shrink_kernel(
    const BgmvBatch batch, int count, int num_tokens, int h_in, int64_t layer_idx, float scale,
    int accumulate_into_y) {
  __shared__ float red[(kBgmvThreads / kWave) * Pow2Ceil<RS * kGroup>::value];
  using E = typename D::E;
  const PlanOfLane plans = preload_plans(batch);
  const BatchSlot slot = batch_slot(batch, count);
  const BgmvProblem& P = batch.p[slot.problem];
  const int r = P.narrow;
  const int row0 = slot.sub * RS;
  int toks[kGroup];
  int64_t stack_addr;
  const int n = resolve_chunk(P, reinterpret_cast<const int64_t*>(read_lane64(plans.plan, slot.problem)),
                              read_lane(plans.num_groups, slot.problem), num_tokens, false, slot.chunk, toks,
                              stack_addr);
  if (n == 0) return;
  const E* A = reinterpret_cast<const E*>(stack_addr) + (layer_idx * r + row0) * static_cast<int64_t>(h_in);
  E* Y = static_cast<E*>(P.y);
  const E* X = static_cast<const E*>(P.x);
  const bool acc_y = accumulate_into_y != 0;
  switch (n) {
    case 1:
      bgmv_shrink_body<D, RS, 1>(Y, X, A, toks, h_in, row0, P.y_offset, P.y_stride, scale, acc_y, red);
      break;
    case 2:
      bgmv_shrink_body<D, RS, 2>(Y, X, A, toks, h_in, row0, P.y_offset, P.y_stride, scale, acc_y, red);
      break;
    case 3:
      bgmv_shrink_body<D, RS, 3>(Y, X, A, toks, h_in, row0, P.y_offset, P.y_stride, scale, acc_y, red);
      break;
    default:
      bgmv_shrink_body<D, RS, 4>(Y, X, A, toks, h_in, row0, P.y_offset, P.y_stride, scale, acc_y, red);
      break;
  }
}

// ---------------------------------------------------------------------------------
// SGMV shrink for a handful of rows: the same streaming body, with the token chunks cut from the
// segments (4 consecutive rows of one segment) instead of gathered by adapter.  A prefill batch of a
// few dozen tokens has too few 16-row MFMA tiles to occupy the chip and K would have to be split
// across workgroups; here every (chunk, RS rows of A) pair is a workgroup of its own and the whole
// workgroup splits K.
// ---------------------------------------------------------------------------------
template <typename D, int RS>
__global__ __launch_bounds__(kBgmvThreads) void sgmv_shrink_rows_kernel(
    typename D::E* __restrict__ V, const typename D::E* __restrict__ X, const int64_t* __restrict__ W,
    const int32_t* __restrict__ s_start, const int32_t* __restrict__ s_end, int num_segments, int num_tokens,
    int h_in, int r, int64_t layer_idx, float scale, int accumulate_into_v) {
  __shared__ float red[(kBgmvThreads / kWave) * Pow2Ceil<RS * kGroup>::value];
  using E = typename D::E;
  const bool acc_v = accumulate_into_v != 0;
  const int subs = r / RS;
  const int v = static_cast<int>(xcd_virtual_id());
  const int chunk = v / subs;
  const int row0 = (v % subs) * RS;
  const int64_t pre = preload_segment_entry(W, num_segments);
  RowTile rt;
  if (!find_row_tile(s_start, s_end, num_segments, num_tokens, kGroup, chunk, rt)) return;
  const int n = rt.row_end - rt.row0;
  int toks[kGroup];
#pragma unroll
  for (int g = 0; g < kGroup; ++g) toks[g] = rt.row0 + min(g, n - 1);
  const E* A = reinterpret_cast<const E*>(segment_entry(pre, W, rt.seg)) + (layer_idx * r + row0) * static_cast<int64_t>(h_in);
  switch (n) {
    case 1:
      bgmv_shrink_body<D, RS, 1>(V, X, A, toks, h_in, row0, 0, r, scale, acc_v, red);
      break;
    case 2:
      bgmv_shrink_body<D, RS, 2>(V, X, A, toks, h_in, row0, 0, r, scale, acc_v, red);
      break;
    case 3:
      bgmv_shrink_body<D, RS, 3>(V, X, A, toks, h_in, row0, 0, r, scale, acc_v, red);
      break;
    default:
      bgmv_shrink_body<D, RS, 4>(V, X, A, toks, h_in, row0, 0, r, scale, acc_v, red);
      break;
  }
}

template <typename D>
static hipError_t launch_shrink_rows_dtype(const SgmvArgs& a, hipStream_t stream) {
  const int64_t chunks = (a.num_tokens + kGroup - 1) / kGroup + a.num_segments;  // upper bound
  const int rs = chunks * (a.d_out / 8) >= 512 ? 8 : (chunks * (a.d_out / 4) >= 512 ? 4 : 2);
  const dim3 grid(static_cast<unsigned>(chunks * (a.d_out / rs)));
  auto args = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(kBgmvThreads), 0, stream, static_cast<typename D::E*>(a.y),
                       static_cast<const typename D::E*>(a.x), a.w_ptrs, a.s_start, a.s_end, a.num_segments,
                       static_cast<int>(a.num_tokens), a.d_in, a.d_out, a.layer_idx, a.scale, a.accumulate);
  };
  if (rs == 8) args(sgmv_shrink_rows_kernel<D, 8>);
  else if (rs == 4) args(sgmv_shrink_rows_kernel<D, 4>);
  else args(sgmv_shrink_rows_kernel<D, 2>);
  return hipGetLastError();
}

// v[s:e] += T(scale * x[s:e] @ A_i^T) for [L, r, h_in] stacks, r a multiple of 8; meant for short batches.
hipError_t launch_sgmv_shrink_rows(const SgmvArgs& a, hipStream_t stream) {
  return a.dtype == LORAX_F16 ? launch_shrink_rows_dtype<F16>(a, stream) : launch_shrink_rows_dtype<BF16>(a, stream);
}

// ---------------------------------------------------------------------------------
// Expand: rows of B^T are only r long, adjacent output columns are adjacent in memory.
// CP lanes (a power of two >= r/8) cover one column with one 16-byte load each, so a
// wave reads a contiguous run of 64/CP columns per step; the CP partial dot products
// meet in a sub-wave shuffle and the first lane of the group updates y.
// ---------------------------------------------------------------------------------
template <typename D, int CP, int U, int NT>
__device__ __forceinline__ void bgmv_expand_body(typename D::E* __restrict__ Y,
                                                 const typename D::E* __restrict__ V,
                                                 const typename D::E* __restrict__ B,
                                                 const int (&toks)[kGroup], int r, int h_out,
                                                 int col0, int64_t y_offset, int64_t y_stride,
                                                 float scale, bool accumulate_into_y) {
  using vec8 = typename D::vec8;
  using E = typename D::E;
  constexpr int kCols = kBgmvThreads / CP;  // columns per step of the workgroup
  const int tid = threadIdx.x;
  const int part = tid % CP;
  const bool has_k = part * 8 < r;

  vec8 vv[NT];
#pragma unroll
  for (int g = 0; g < NT; ++g) {
    vv[g] = zero8<D>();
    if (has_k) vv[g] = load8<D>(V + static_cast<int64_t>(toks[g]) * r + part * 8);
  }

  vec8 wv[U];
  const int colbase = col0 + tid / CP;  // the lane group's column of step u is colbase + u * kCols
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int c = colbase + u * kCols;
    wv[u] = zero8<D>();
    if (has_k && c < h_out) wv[u] = load8<D>(B + static_cast<int64_t>(c) * r + part * 8);
  }
  // The y of step u belongs to lane u % CP of the column's lane group (after the shuffles every lane of
  // the group holds the column's sum): a lane keeps ceil(U / CP) old values per token instead of U.
  constexpr int UY = (U + CP - 1) / CP;
  E yv[UY][NT];
#pragma unroll
  for (int k = 0; k < UY; ++k) {
    const int u = part + k * CP;
    const int c = colbase + u * kCols;
#pragma unroll
    for (int g = 0; g < NT; ++g) {
      yv[k][g] = static_cast<E>(0.f);
      if (u < U && c < h_out && accumulate_into_y)
        yv[k][g] = Y[static_cast<int64_t>(toks[g]) * y_stride + y_offset + c];
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    float s[NT];
#pragma unroll
    for (int g = 0; g < NT; ++g) s[g] = dot8<D>(wv[u], vv[g], 0.f);
#pragma unroll
    for (int g = 0; g < NT; ++g) s[g] = group_sum<CP>(s[g]);
    const int c = colbase + u * kCols;
    if (part == u % CP && c < h_out) {
#pragma unroll
      for (int g = 0; g < NT; ++g)
        Y[static_cast<int64_t>(toks[g]) * y_stride + y_offset + c] = accumulate<D>(yv[u / CP][g], s[g] * scale);
    }
  }
}

// The same with y moved in whole 16-byte pieces (every problem's y rows 16-byte aligned: y_offset and y_stride
// multiples of 8).  Above, a lane reads and writes single elements of y, so a wave spends U * NT load and as many
// store instructions of 32-128 useful bytes on y, more instructions than it spends on B^T.  Here the sums change
// lanes through a piece of LDS private to the wave: per step the wave's lane groups hold 64 / CP ADJACENT columns,
// so once all steps' sums are written as [token][step][column], item i is 8 (or 4, at 16 lanes per column) adjacent
// columns of one token and step, and lane i % 64 owns it: one 16-byte load of the old y, issued in front with the
// loads of B^T, and one 16-byte store.  Same sums, same roundings: the result equals the scalar path's bit for bit.
template <typename D, int CP, int U, int NT>
__device__ __forceinline__ void bgmv_expand_body_vec(typename D::E* __restrict__ Y,
                                                     const typename D::E* __restrict__ V,
                                                     const typename D::E* __restrict__ B,
                                                     const int (&toks)[kGroup], int r, int h_out,
                                                     int col0, int64_t y_offset, int64_t y_stride,
                                                     float scale, bool accumulate_into_y, float* wave_sums) {
  using vec8 = typename D::vec8;
  using E = typename D::E;
  constexpr int GPW = kWave / CP;           // adjacent columns per step of one wave
  constexpr int VC = GPW >= 8 ? 8 : 4;      // columns per y access
  constexpr int PIECES = GPW / VC;          // y accesses per token and step
  constexpr int ITEMS = NT * U * PIECES;
  constexpr int KI = (ITEMS + kWave - 1) / kWave;
  typedef E vecy __attribute__((ext_vector_type(VC)));
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int part = tid % CP;
  const int ql = lane / CP;  // the lane group's column inside the wave's run
  const bool has_k = part * 8 < r;

  vec8 vv[NT];
#pragma unroll
  for (int g = 0; g < NT; ++g) {
    vv[g] = zero8<D>();
    if (has_k) vv[g] = load8<D>(V + static_cast<int64_t>(toks[g]) * r + part * 8);
  }
  vec8 wv[U];
  // A wave's U steps cover U * GPW adjacent columns (the scalar path deals the steps kCols apart): the B^T rows of
  // one step are as contiguous as there, and the wave's y accesses for one token are one run of whole cache lines.
  const int colbase = col0 + wave * U * GPW + ql;  // the lane group's column of step u is colbase + u * GPW
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int c = colbase + u * GPW;
    wv[u] = zero8<D>();
    if (has_k && c < h_out) wv[u] = load8<D>(B + static_cast<int64_t>(c) * r + part * 8);
  }
  // this lane's items: i = (token * U + step) * PIECES + piece
  vecy yold[KI];
  E* yp[KI];
  bool live[KI];
#pragma unroll
  for (int k = 0; k < KI; ++k) {
    const int i = lane + k * kWave;
    const int piece = i % PIECES;
    const int u = (i / PIECES) % U;
    const int g = i / (PIECES * U);
    const int c = col0 + (wave * U + u) * GPW + piece * VC;
    live[k] = i < ITEMS && c < h_out;  // h_out is a multiple of 8: a piece is inside or outside as a whole
    // (the values are made opaque so that the optimiser keeps a select chain instead of turning toks[] into an
    // array in memory indexed by the lane's g)
    int tok = toks[0];
#pragma unroll
    for (int q = 1; q < NT; ++q) {
      int t = toks[q];
      asm volatile("" : "+v"(t));
      tok = g == q ? t : tok;
    }
    yp[k] = Y + static_cast<int64_t>(tok) * y_stride + y_offset + c;
#pragma unroll
    for (int e = 0; e < VC; ++e) yold[k][e] = static_cast<E>(0.f);
    if (live[k] && accumulate_into_y) yold[k] = *(const LORAX_GLOBAL vecy*)(yp[k]);
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    float s[NT];
#pragma unroll
    for (int g = 0; g < NT; ++g) s[g] = dot8<D>(wv[u], vv[g], 0.f);
#pragma unroll
    for (int g = 0; g < NT; ++g) s[g] = group_sum<CP>(s[g]);
    if (part == u % CP) {
#pragma unroll
      for (int g = 0; g < NT; ++g) wave_sums[(g * U + u) * GPW + ql] = s[g] * scale;
    }
  }
  // Writer and reader are lanes of one wave and a wave's LDS accesses execute in order: only the compiler has
  // to be kept from moving the reads up.
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
  for (int k = 0; k < KI; ++k) {
    if (live[k]) {
      const float* d = wave_sums + (lane + k * kWave) * VC;
      vecy out;
#pragma unroll
      for (int e = 0; e < VC; e += 4) {
        const f32x4 q = *reinterpret_cast<const f32x4*>(d + e);
#pragma unroll
        for (int t = 0; t < 4; ++t) out[e + t] = accumulate<D>(yold[k][e + t], q[t]);
      }
      *(LORAX_GLOBAL vecy*)(yp[k]) = out;
    }
  }
}

template <typename D, int CP, int U, int NT, bool VY>
__device__ __forceinline__ void bgmv_expand_tokens(typename D::E* Y, const typename D::E* V, const typename D::E* B,
                                                   const int (&toks)[kGroup], int r, int h_out, int col0,
                                                   int64_t y_offset, int64_t y_stride, float scale, bool acc_y,
                                                   float* wave_sums) {
  if constexpr (VY)
    bgmv_expand_body_vec<D, CP, U, NT>(Y, V, B, toks, r, h_out, col0, y_offset, y_stride, scale, acc_y, wave_sums);
  else
    bgmv_expand_body<D, CP, U, NT>(Y, V, B, toks, r, h_out, col0, y_offset, y_stride, scale, acc_y);
}

template <typename D, int CP, int U, bool VY>
__device__ __forceinline__ void bgmv_expand_problem(const BgmvProblem& P, const BatchSlot& slot, int n,
                                                    const int (&toks)[kGroup], int64_t stack_addr,
                                                    int64_t layer_idx, float scale, bool acc_y, float* wave_sums) {
  using E = typename D::E;
  const int h_out = P.width;
  const int r = P.narrow;
  const int col0 = slot.sub * (kBgmvThreads / CP) * U;  // U = expand_steps(CP, the launch's U)
  const E* B = reinterpret_cast<const E*>(stack_addr) + layer_idx * h_out * static_cast<int64_t>(r);
  E* Y = static_cast<E*>(P.y);
  const E* V = static_cast<const E*>(P.x);
  switch (n) {
    case 1:
      bgmv_expand_tokens<D, CP, U, 1, VY>(Y, V, B, toks, r, h_out, col0, P.y_offset, P.y_stride, scale, acc_y, wave_sums);
      break;
    case 2:
      bgmv_expand_tokens<D, CP, U, 2, VY>(Y, V, B, toks, r, h_out, col0, P.y_offset, P.y_stride, scale, acc_y, wave_sums);
      break;
    case 3:
      bgmv_expand_tokens<D, CP, U, 3, VY>(Y, V, B, toks, r, h_out, col0, P.y_offset, P.y_stride, scale, acc_y, wave_sums);
      break;
    default:
      bgmv_expand_tokens<D, CP, U, 4, VY>(Y, V, B, toks, r, h_out, col0, P.y_offset, P.y_stride, scale, acc_y, wave_sums);
      break;
  }
}

// Steps (columns per lane group) of an expand workgroup: ranks of 32 and more (4+ lanes per column) take
// twice the launch's U - their lanes keep few old y values, so the registers allow it, and a wave then has
// twice the bytes in flight.
__host__ __device__ constexpr int expand_steps(int lanes_per_column, int u) {
  return lanes_per_column >= 4 ? 2 * u : u;
}

// Lanes per column of a rank: the power of two >= r / 8.
__host__ __device__ __forceinline__ int expand_lanes_per_column(int r) {
  const int chunks = r / 8;
  return chunks <= 1 ? 1 : (chunks <= 2 ? 2 : (chunks <= 4 ? 4 : (chunks <= 8 ? 8 : 16)));
}

// One launch serves problems of different ranks: the workgroup picks the body for its problem's rank.
// VY: y moves in 16-byte pieces (bgmv_expand_body_vec); each wave has kGroup * U * 64 floats of LDS for its sums
// (one lane per column, the widest case; with 4 and more lanes per column the steps double and the columns per
// step shrink by more).
template <typename D, int U, bool VY>
__global__ __launch_bounds__(kBgmvThreads) void bgmv_expand_kernel(const BgmvBatch batch, int count,
                                                                   int num_tokens, int64_t layer_idx, float scale,
                                                                   int accumulate_into_y) {
  constexpr int kWaveSums = kGroup * U * kWave;
  __shared__ __attribute__((aligned(16))) float sums[VY ? (kBgmvThreads / kWave) * kWaveSums : 4];
  float* wave_sums = sums + (VY ? (threadIdx.x / kWave) * kWaveSums : 0);
  const bool acc_y = accumulate_into_y != 0;
  const PlanOfLane plans = preload_plans(batch);
  const BatchSlot vb = batch_slot(batch, count);
  const BgmvProblem& P = batch.p[vb.problem];
  // the routing record is asked for before the problem's rank is looked at: it travels with the problem's fields
  int toks[kGroup];
  int64_t stack;
  const int n = resolve_chunk(P, reinterpret_cast<const int64_t*>(read_lane64(plans.plan, vb.problem)),
                              read_lane(plans.num_groups, vb.problem), num_tokens, true, vb.chunk, toks, stack);
  if (n == 0) return;
  switch (expand_lanes_per_column(P.narrow)) {
    case 1:
      bgmv_expand_problem<D, 1, U, VY>(P, vb, n, toks, stack, layer_idx, scale, acc_y, wave_sums);
      break;
    case 2:
      bgmv_expand_problem<D, 2, U, VY>(P, vb, n, toks, stack, layer_idx, scale, acc_y, wave_sums);
      break;
    case 4:
      bgmv_expand_problem<D, 4, expand_steps(4, U), VY>(P, vb, n, toks, stack, layer_idx, scale, acc_y, wave_sums);
      break;
    case 8:
      bgmv_expand_problem<D, 8, expand_steps(8, U), VY>(P, vb, n, toks, stack, layer_idx, scale, acc_y, wave_sums);
      break;
    default:
      bgmv_expand_problem<D, 16, expand_steps(16, U), VY>(P, vb, n, toks, stack, layer_idx, scale, acc_y, wave_sums);
      break;
  }
}

// ---------------------------------------------------------------------------------
// Shrink and expand of one projection in ONE launch, for ranks whose A slab is small enough
// that every column slice can afford to recompute the shrink (rank 8 and 16): a workgroup
// issues the loads of its slice of B^T and of the old y first (they do not depend on v), runs
// the whole shrink of its token chunk (all R rows, full hidden dimension; the slab is shared
// through L2 by the slices of the chunk, which the XCD-aware numbering puts on one XCD), rounds
// v to the storage type exactly where the two-launch path would store it, and finishes with
// the expand of its columns.  v never goes to memory and one launch boundary disappears.
// ---------------------------------------------------------------------------------
template <typename D, int R, int U, int NBLK, int NT, bool VEC4>
__device__ __forceinline__ void bgmv_lora_body(typename D::E* __restrict__ Y,
                                               const typename D::E* __restrict__ X,
                                               const typename D::E* __restrict__ A,
                                               const typename D::E* __restrict__ B,
                                               const int (&toks)[kGroup], int h_in, int h_out, int col0,
                                               int col_end, int64_t y_offset, int64_t y_stride, float scale,
                                               float* red, typename D::E* vsh) {
  using vec8 = typename D::vec8;
  using E = typename D::E;
  constexpr int CP = R / 8;
  constexpr int kCols = kBgmvThreads / CP;     // columns per step of the workgroup
  constexpr int kBlock = kCols * U;            // columns per expand block
  constexpr int kSteps = R <= 8 ? 2 : 1;       // hidden-dimension steps per trip (register budget)
  const int tid = threadIdx.x;
  const int part = tid % CP;

  E* yrow[NT];
#pragma unroll
  for (int g = 0; g < NT; ++g) yrow[g] = Y + static_cast<int64_t>(toks[g]) * y_stride + y_offset;

  // (1) the first trip of the shrink's operands goes out first: loads return in order and these are
  // needed first, so the dot products run while the expand's operands are still arriving.
  float acc[R][NT];
#pragma unroll
  for (int j = 0; j < R; ++j)
#pragma unroll
    for (int g = 0; g < NT; ++g) acc[j][g] = 0.f;
  const E* xrow[NT];
#pragma unroll
  for (int g = 0; g < NT; ++g) xrow[g] = X + static_cast<int64_t>(toks[g]) * h_in;
  constexpr int kStep = kBgmvThreads * 8;
  vec8 xv[kSteps][NT];
  vec8 av[kSteps][R];
  auto load_trip = [&](int k) {
#pragma unroll
    for (int u = 0; u < kSteps; ++u) {
      // a step past the end re-reads the slab's first chunk and is masked to zero
      const bool live = k + u * kStep < h_in;
      const int ku = live ? k + u * kStep : 0;
#pragma unroll
      for (int g = 0; g < NT; ++g) xv[u][g] = keep_if<D>(live, load8<D>(xrow[g] + ku));
#pragma unroll
      for (int j = 0; j < R; ++j) av[u][j] = load8<D>(A + static_cast<int64_t>(j) * h_in + ku);
    }
  };
  auto dot_trip = [&]() {
#pragma unroll
    for (int u = 0; u < kSteps; ++u)
#pragma unroll
      for (int j = 0; j < R; ++j)
#pragma unroll
        for (int g = 0; g < NT; ++g) acc[j][g] = dot8<D>(av[u][j], xv[u][g], acc[j][g]);
  };
  load_trip(tid * 8);

  // (2) every B^T vector of the workgroup's column range and the old y: they do not depend on v, and
  // being cold they are the long pole of the expand.  Clamped, not predicated.
  // VEC4 (every y row 8-byte aligned, h_out a multiple of 4): a lane owns U = 4 adjacent columns, so
  // the old y of a block is one 8-byte load per token and the new y one 8-byte store, and all of it
  // is fetched here, ahead of the shrink's arithmetic.  Otherwise lanes take columns kCols apart and
  // y moves element by element, one block ahead of the arithmetic.
  typedef E vec4 __attribute__((ext_vector_type(4)));
  static_assert(!VEC4 || U == 4, "the vector path moves four columns per lane");
  auto column = [&](int blk, int u) {
    return VEC4 ? col0 + blk * kBlock + (tid / CP) * U + u : col0 + blk * kBlock + u * kCols + tid / CP;
  };
  vec8 wv[NBLK][U];
#pragma unroll
  for (int blk = 0; blk < NBLK; ++blk)
#pragma unroll
    for (int u = 0; u < U; ++u)
      wv[blk][u] = load8<D>(B + static_cast<int64_t>(min(column(blk, u), h_out - 1)) * R + part * 8);
  vec4 yq[VEC4 ? NBLK : 1][NT];
  if constexpr (VEC4) {
#pragma unroll
    for (int blk = 0; blk < NBLK; ++blk) {
      const int cc = min(column(blk, 0), h_out - 4);
#pragma unroll
      for (int g = 0; g < NT; ++g) yq[blk][g] = *(const LORAX_GLOBAL vec4*)(yrow[g] + cc);
    }
  }
  // the old y of one block (warm: the base projection has just written it)
  auto load_y = [&](int blk, E(&yv)[U][NT]) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int cc = min(column(blk, u), h_out - 1);
#pragma unroll
      for (int g = 0; g < NT; ++g) yv[u][g] = yrow[g][cc];
    }
  };

  // shrink: all R rows of the slab against the chunk's tokens
  __builtin_amdgcn_sched_barrier(0);
  dot_trip();
  for (int k = tid * 8 + kSteps * kStep; k < h_in; k += kSteps * kStep) {
    load_trip(k);
    __builtin_amdgcn_sched_barrier(0);
    dot_trip();
  }

  // (3) workgroup-wide sums -> v in LDS, rounded to the storage type
  constexpr int NV = Pow2Ceil<R * NT>::value;
  float vals[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) vals[i] = 0.f;
#pragma unroll
  for (int j = 0; j < R; ++j)
#pragma unroll
    for (int g = 0; g < NT; ++g) vals[g * R + j] = acc[j][g];
  transpose_reduce<NV>(vals);
  const int lane = lane_id();
  const int wave = tid / kWave;
  if ((lane & (kWave / NV - 1)) == 0) red[wave * NV + transpose_reduce_index<NV>(lane)] = vals[0];
  __syncthreads();
  if (tid < R * NT) {
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < kBgmvThreads / kWave; ++w) s += red[w * NV + tid];
    vsh[tid] = from_f32<D>(s);  // index g * R + j
  }
  __syncthreads();
  vec8 vv[NT];
#pragma unroll
  for (int g = 0; g < NT; ++g) vv[g] = *reinterpret_cast<const vec8*>(vsh + g * R + part * 8);

  // (4) expand, block by block, the next block's y in flight while one is computed
  auto finish_block = [&](int blk, const vec8(&w)[U], const E(&yv)[U][NT]) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float s[NT];
#pragma unroll
      for (int g = 0; g < NT; ++g) s[g] = dot8<D>(w[u], vv[g], 0.f);
#pragma unroll
      for (int g = 0; g < NT; ++g) s[g] = group_sum<CP>(s[g]);
      const int col = column(blk, u);
      if (part == 0 && col < col_end) {
#pragma unroll
        for (int g = 0; g < NT; ++g) yrow[g][col] = accumulate<D>(yv[u][g], s[g] * scale);
      }
    }
  };
  if constexpr (VEC4) {
#pragma unroll
    for (int blk = 0; blk < NBLK; ++blk) {
      float s[U][NT];
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int g = 0; g < NT; ++g) s[u][g] = dot8<D>(wv[blk][u], vv[g], 0.f);
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int g = 0; g < NT; ++g) s[u][g] = group_sum<CP>(s[u][g]);
      const int col = column(blk, 0);
      if (part == 0 && col < col_end) {
#pragma unroll
        for (int g = 0; g < NT; ++g) {
          vec4 out;
#pragma unroll
          for (int u = 0; u < U; ++u) out[u] = accumulate<D>(yq[blk][g][u], s[u][g] * scale);
          *(LORAX_GLOBAL vec4*)(yrow[g] + col) = out;
        }
      }
    }
  } else {
    E ya[U][NT], yb[U][NT];
    load_y(0, ya);
    if constexpr (NBLK == 1) finish_block(0, wv[0], ya);
#pragma unroll
    for (int blk = 0; blk + 1 < NBLK; blk += 2) {
      if (col0 + blk * kBlock < col_end) {
        load_y(blk + 1, yb);
        __builtin_amdgcn_sched_barrier(0);
        finish_block(blk, wv[blk], ya);
        if (blk + 2 < NBLK) load_y(blk + 2, ya);
        __builtin_amdgcn_sched_barrier(0);
        finish_block(blk + 1, wv[blk + 1], yb);
      }
    }
  }
}

template <typename D, int R, int U, int NBLK, bool VEC4>
__device__ __forceinline__ void bgmv_lora_tokens(int n, typename D::E* Y, const typename D::E* X,
                                                 const typename D::E* A, const typename D::E* B,
                                                 const int (&toks)[kGroup], int h_in, int h_out, int col0, int col_end,
                                                 int64_t y_offset, int64_t y_stride, float scale, float* red,
                                                 typename D::E* vsh) {
  switch (n) {
    case 1:
      bgmv_lora_body<D, R, U, NBLK, 1, VEC4>(Y, X, A, B, toks, h_in, h_out, col0, col_end, y_offset, y_stride, scale, red,
                                             vsh);
      break;
    case 2:
      bgmv_lora_body<D, R, U, NBLK, 2, VEC4>(Y, X, A, B, toks, h_in, h_out, col0, col_end, y_offset, y_stride, scale, red,
                                             vsh);
      break;
    case 3:
      bgmv_lora_body<D, R, U, NBLK, 3, VEC4>(Y, X, A, B, toks, h_in, h_out, col0, col_end, y_offset, y_stride, scale, red,
                                             vsh);
      break;
    default:
      bgmv_lora_body<D, R, U, NBLK, 4, VEC4>(Y, X, A, B, toks, h_in, h_out, col0, col_end, y_offset, y_stride, scale, red,
                                             vsh);
      break;
  }
}

// Workgroup placement for a batch of one wide and several narrow projections (q with k and v) when the
// launch has between one and two workgroups per CU.  The hardware hands workgroup h to XCD h % 8, and
// inside an XCD the workgroup in slot s = h / 8 shares its CU with the one in slot s + 32 (measured: 32
// CUs per XCD are filled once before any gets a second workgroup).  Two workgroups on a CU halve each
// other's vector-ALU rate, and the launch ends with its slowest CU, so the wide projection's workgroups
// are put into the slots that stay alone on their CU and the narrow ones into the shared slots.
// XCD k owns the token chunks [k * chunks_per_xcd, ...); problem 0 is the wide one.  Returns false for
// a slot without work.
__device__ __forceinline__ bool balanced_slot(int count, int chunks, int chunks_per_xcd, VirtualBlock& vb) {
  constexpr int kCusPerXcd = 32;
  const int xcd = blockIdx.x % kXcds, slot = blockIdx.x / kXcds;
  const int slots = chunks_per_xcd * count;       // per XCD, between 33 and 64
  const int first = xcd * chunks_per_xcd;
  const int heavy = max(min(chunks - first, chunks_per_xcd), 0);  // wide-projection workgroups of this XCD
  const int light = heavy * (count - 1);
  const int shared = slots - kCusPerXcd;          // slots [0, shared) pair with [32, 32 + shared)
  const int alone = kCusPerXcd - shared;          // slots [shared, 32)
  const int heavy_alone = min(heavy, alone);
  int h = -1, l = -1;                             // index among the XCD's heavy / light workgroups
  if (slot >= shared && slot < kCusPerXcd) {
    const int u = slot - shared;
    if (u < heavy_alone) h = u; else l = u - heavy_alone;
  } else {
    const int i = slot < shared ? slot : shared + (slot - kCusPerXcd);
    const int heavy_shared = heavy - heavy_alone;
    if (i < heavy_shared) h = heavy_alone + i; else l = (alone - heavy_alone) + (i - heavy_shared);
  }
  vb.x = 0;
  if (h >= 0) {
    if (h >= heavy) return false;
    vb.y = first + h;
    vb.z = 0;
    return true;
  }
  if (l >= light) return false;
  vb.y = first + l / (count - 1);
  vb.z = 1 + l % (count - 1);
  return true;
}

template <typename D, int R, int U, int NBLK, bool VEC4>
__global__ __launch_bounds__(kBgmvThreads) void bgmv_lora_kernel(const BgmvBatch batch, int h_in,
                                                                 int64_t layer_idx, float scale, int count,
                                                                 int balanced_chunks, int chunks_per_xcd) {
  using E = typename D::E;
  __shared__ float red[(kBgmvThreads / kWave) * Pow2Ceil<R * kGroup>::value];
  __shared__ __attribute__((aligned(16))) E vsh[R * kGroup];
  const ProblemFields fields = preload_problems(batch);  // before anything waits: see select_problem
  VirtualBlock vb;
  if (balanced_chunks > 0) {
    if (!balanced_slot(count, balanced_chunks, chunks_per_xcd, vb)) return;
  } else {
    vb = xcd_virtual_block();
  }
  const BgmvProblem P = select_problem(fields, vb.z);
  const int h_out = P.width;
  constexpr int cols_per_wg = (kBgmvThreads / (R / 8)) * U * NBLK;
  const int col0 = vb.x * cols_per_wg;
  if (col0 >= h_out || vb.y >= P.num_groups) return;
  const int col_end = min(col0 + cols_per_wg, h_out);
  const int64_t* rec = P.plan + static_cast<int64_t>(vb.y) * kPlanRecordWords;
  const int n = static_cast<int>(rec[0]);
  if (n <= 0) return;  // an all-zero record: padding of a plan kept at a fixed size for graph replay
  int toks[kGroup];
#pragma unroll
  for (int g = 0; g < kGroup; ++g) toks[g] = static_cast<int>(rec[1 + g]);
  // (stacked weights: the record names the adapter's entry of the [num_adapters, R, h_in] / [num_adapters, h_out, R]
  // tensors whose bases the problem carries, see resolve_chunk)
  const int64_t a_base = reinterpret_cast<int64_t>(P.w_ptrs), b_base = reinterpret_cast<int64_t>(P.indices);
  const int64_t a_addr = a_base != 0 ? a_base + rec[5] * R * static_cast<int64_t>(h_in) * 2 : rec[5];
  const int64_t b_addr = b_base != 0 ? b_base + rec[6] * R * static_cast<int64_t>(h_out) * 2 : rec[6];
  const E* A = reinterpret_cast<const E*>(a_addr) + layer_idx * R * static_cast<int64_t>(h_in);
  const E* B = reinterpret_cast<const E*>(b_addr) + layer_idx * h_out * static_cast<int64_t>(R);
  E* Y = static_cast<E*>(P.y);
  const E* X = static_cast<const E*>(P.x);
  // A narrow projection batched with wide ones (k and v next to q) fills one expand block only: it runs the
  // one-block body, which neither loads nor multiplies the three empty blocks.
  constexpr int kBlockCols = (kBgmvThreads / (R / 8)) * U;
  if (NBLK > 1 && col_end - col0 <= kBlockCols)
    bgmv_lora_tokens<D, R, U, 1, VEC4>(n, Y, X, A, B, toks, h_in, h_out, col0, col_end, P.y_offset, P.y_stride, scale,
                                       red, vsh);
  else
    bgmv_lora_tokens<D, R, U, NBLK, VEC4>(n, Y, X, A, B, toks, h_in, h_out, col0, col_end, P.y_offset, P.y_stride,
                                          scale, red, vsh);
}

// ---------------------------------------------------------------------------------
// Shrink and expand of a SHORT prefill batch in one launch: the body above with the token chunks cut from the
// segments (4 consecutive rows of one segment) instead of gathered by adapter.  A prefill batch of a few dozen
// rows is bound by launches - zero-fill, shrink and expand take about 4 us each for a megabyte of traffic - so
// the whole update of up to four projections that share x goes out as one.
// ---------------------------------------------------------------------------------
template <typename D, int R, int U, int NBLK, bool VEC4>
__global__ __launch_bounds__(kBgmvThreads) void sgmv_lora_rows_kernel(
    const SgmvLoraBatch batch, const typename D::E* __restrict__ X, const int32_t* __restrict__ s_start,
    const int32_t* __restrict__ s_end, int num_segments, int num_tokens, int h_in, int64_t layer_idx, float scale) {
  using E = typename D::E;
  __shared__ float red[(kBgmvThreads / kWave) * Pow2Ceil<R * kGroup>::value];
  __shared__ __attribute__((aligned(16))) E vsh[R * kGroup];
  const VirtualBlock vb = xcd_virtual_block();  // x: column slice, y: row chunk, z: projection
  // lane i fetches problem i's fields, the workgroup's own are read from lane z (see select_problem)
  const SgmvLoraProblem& mine = batch.p[lane_id() < kMaxSgmvLoraProblems ? lane_id() : kMaxSgmvLoraProblems - 1];
  SgmvLoraProblem P;
  P.y = reinterpret_cast<void*>(read_lane64(reinterpret_cast<int64_t>(mine.y), vb.z));
  P.a_ptrs = reinterpret_cast<const int64_t*>(read_lane64(reinterpret_cast<int64_t>(mine.a_ptrs), vb.z));
  P.b_ptrs = reinterpret_cast<const int64_t*>(read_lane64(reinterpret_cast<int64_t>(mine.b_ptrs), vb.z));
  P.y_offset = read_lane64(mine.y_offset, vb.z);
  P.y_stride = read_lane64(mine.y_stride, vb.z);
  P.h_out = read_lane(mine.h_out, vb.z);
  const int h_out = P.h_out;
  constexpr int cols_per_wg = (kBgmvThreads / (R / 8)) * U * NBLK;
  const int col0 = vb.x * cols_per_wg;
  if (col0 >= h_out) return;
  const int col_end = min(col0 + cols_per_wg, h_out);
  const int64_t pre_a = preload_segment_entry(P.a_ptrs, num_segments);
  const int64_t pre_b = preload_segment_entry(P.b_ptrs, num_segments);
  RowTile rt;
  if (!find_row_tile(s_start, s_end, num_segments, num_tokens, kGroup, vb.y, rt)) return;
  const int n = rt.row_end - rt.row0;
  int toks[kGroup];
#pragma unroll
  for (int g = 0; g < kGroup; ++g) toks[g] = rt.row0 + min(g, n - 1);
  const E* A = reinterpret_cast<const E*>(segment_entry(pre_a, P.a_ptrs, rt.seg)) + layer_idx * R * static_cast<int64_t>(h_in);
  const E* B = reinterpret_cast<const E*>(segment_entry(pre_b, P.b_ptrs, rt.seg)) + layer_idx * h_out * static_cast<int64_t>(R);
  bgmv_lora_tokens<D, R, U, NBLK, VEC4>(n, static_cast<E*>(P.y), X, A, B, toks, h_in, h_out, col0, col_end, P.y_offset,
                                        P.y_stride, scale, red, vsh);
}

template <typename D, int R, int NBLK>
static hipError_t launch_sgmv_lora_blk(const SgmvLoraArgs& a, hipStream_t stream) {
  constexpr int U = 4;
  constexpr int cols_per_wg = (kBgmvThreads / (R / 8)) * U * NBLK;
  int wide = 0;
  bool vec4 = true;  // 8-byte y accesses need every problem's rows 8-byte aligned and no ragged last column group
  for (int i = 0; i < a.count; ++i) {
    const SgmvLoraProblem& p = a.batch.p[i];
    wide = p.h_out > wide ? p.h_out : wide;
    vec4 = vec4 && p.h_out % 4 == 0 && p.y_stride % 4 == 0 && p.y_offset % 4 == 0 &&
           reinterpret_cast<uintptr_t>(p.y) % 8 == 0;
  }
  const int64_t chunks = (a.num_tokens + kGroup - 1) / kGroup + a.num_segments;  // upper bound
  const dim3 grid((wide + cols_per_wg - 1) / cols_per_wg, static_cast<unsigned>(chunks), a.count);
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(kBgmvThreads), 0, stream, a.batch, static_cast<const typename D::E*>(a.x),
                       a.s_start, a.s_end, a.num_segments, static_cast<int>(a.num_tokens), a.h_in, a.layer_idx, a.scale);
  };
  if (vec4) launch(sgmv_lora_rows_kernel<D, R, U, NBLK, true>);
  else launch(sgmv_lora_rows_kernel<D, R, U, NBLK, false>);
  return hipGetLastError();
}

template <typename D, int R>
static hipError_t launch_sgmv_lora_r(const SgmvLoraArgs& a, hipStream_t stream) {
  // column slices as wide as the launch affords, as in launch_lora_r: every slice repeats the shrink
  constexpr int cols4 = (kBgmvThreads / (R / 8)) * 4 * 4;
  const int64_t chunks = (a.num_tokens + kGroup - 1) / kGroup;
  int64_t wgs4 = 0;
  for (int i = 0; i < a.count; ++i) wgs4 += chunks * ((a.batch.p[i].h_out + cols4 - 1) / cols4);
  if (wgs4 >= 200) return launch_sgmv_lora_blk<D, R, 4>(a, stream);
  if (wgs4 >= 100) return launch_sgmv_lora_blk<D, R, 2>(a, stream);
  return launch_sgmv_lora_blk<D, R, 1>(a, stream);
}

// y[s:e, window] += T(scale * T(x[s:e] @ A_i^T) @ B_i^T) per segment, ranks 8 and 16, short batches.
hipError_t launch_sgmv_lora_rows(const SgmvLoraArgs& a, hipStream_t stream) {
  if (a.dtype == LORAX_F16)
    return a.rank == 8 ? launch_sgmv_lora_r<F16, 8>(a, stream) : launch_sgmv_lora_r<F16, 16>(a, stream);
  return a.rank == 8 ? launch_sgmv_lora_r<BF16, 8>(a, stream) : launch_sgmv_lora_r<BF16, 16>(a, stream);
}

// ---------------------------------------------------------------------------------
// Host-side launchers
// ---------------------------------------------------------------------------------
// Fills the workgroup numbering of a batch (see BgmvBatch); subs_of(problem) is the number of row
// blocks / column slices of one token chunk.  Returns the number of workgroups.
template <typename SubsOf>
static int64_t number_workgroups(BgmvArgs& a, SubsOf subs_of) {
  auto chunks_of = [&](int i) {
    return a.batch.p[i].plan != nullptr ? static_cast<int64_t>(a.batch.p[i].num_groups) : a.num_tokens;
  };
  int64_t total = 0;
  for (int first = 0; first < a.count;) {
    int last = first;
    while (!tuning().bgmv_no_runs && last + 1 < a.count && chunks_of(last + 1) == chunks_of(first)) ++last;
    int run_subs = 0;
    for (int i = first; i <= last; ++i) {
      a.batch.sub_lo[i] = run_subs;
      run_subs += subs_of(a.batch.p[i]);
      a.batch.sub_hi[i] = run_subs;
    }
    const int64_t end = total + chunks_of(first) * run_subs;
    for (int i = first; i <= last; ++i) {
      a.batch.base[i] = static_cast<int>(total < INT32_MAX ? total : INT32_MAX);
      a.batch.run_subs[i] = run_subs > 0 ? run_subs : 1;
      a.batch.run_end[i] = static_cast<int>(end < INT32_MAX ? end : INT32_MAX);
    }
    total = end;
    first = last + 1;
  }
  return total;
}

template <typename D, int RS>
static hipError_t launch_shrink_rs(BgmvArgs a, hipStream_t stream) {
  const int64_t total = number_workgroups(a, [](const BgmvProblem& p) { return p.narrow / RS; });
  if (total == 0) return hipSuccess;
  if (total >= INT32_MAX) return hipErrorInvalidValue;
  hipLaunchKernelGGL((bgmv_shrink_kernel<D, RS>), dim3(static_cast<unsigned>(total)), dim3(kBgmvThreads), 0, stream,
                     a.batch, a.count, static_cast<int>(a.num_tokens), a.wide_max, a.layer_idx, a.scale,
                     a.accumulate);
  return hipGetLastError();
}

template <typename D>
static hipError_t launch_shrink(const BgmvArgs& a, hipStream_t stream) {
  // Rows per workgroup: 8 when the grid is large enough to fill 256 CUs several times
  // over, fewer rows (more workgroups) for small batches.
  const int64_t wgs8 = a.work_rows * (a.narrow_sum / 8);
  int rs = wgs8 >= 2048 ? 8 : (wgs8 >= 512 ? 4 : 2);
  if (tuning().bgmv_shrink_rows > 0) rs = tuning().bgmv_shrink_rows;
  switch (rs) {
    case 8:
      return launch_shrink_rs<D, 8>(a, stream);
    case 4:
      return launch_shrink_rs<D, 4>(a, stream);
    default:
      return launch_shrink_rs<D, 2>(a, stream);
  }
}

template <typename D, int U>
static hipError_t launch_expand_u(BgmvArgs a, hipStream_t stream) {
  const int64_t total = number_workgroups(a, [](const BgmvProblem& p) {
    const int lanes = expand_lanes_per_column(p.narrow);
    const int cols_per_wg = (kBgmvThreads / lanes) * expand_steps(lanes, U);
    return (p.width + cols_per_wg - 1) / cols_per_wg;
  });
  if (total == 0) return hipSuccess;
  if (total >= INT32_MAX) return hipErrorInvalidValue;
  // 16-byte y accesses need every problem's rows 16-byte aligned (the widths are multiples of 8)
  bool vec_y = !tuning().bgmv_scalar_y;
  for (int i = 0; i < a.count; ++i) {
    const BgmvProblem& p = a.batch.p[i];
    vec_y = vec_y && p.y_stride % 8 == 0 && p.y_offset % 8 == 0 && reinterpret_cast<uintptr_t>(p.y) % 16 == 0;
  }
  if (vec_y)
    hipLaunchKernelGGL((bgmv_expand_kernel<D, U, true>), dim3(static_cast<unsigned>(total)), dim3(kBgmvThreads), 0,
                       stream, a.batch, a.count, static_cast<int>(a.num_tokens), a.layer_idx, a.scale, a.accumulate);
  else
    hipLaunchKernelGGL((bgmv_expand_kernel<D, U, false>), dim3(static_cast<unsigned>(total)), dim3(kBgmvThreads), 0,
                       stream, a.batch, a.count, static_cast<int>(a.num_tokens), a.layer_idx, a.scale, a.accumulate);
  return hipGetLastError();
}

template <typename D>
static hipError_t launch_expand(const BgmvArgs& a, hipStream_t stream) {
  // Columns per lane group.  Narrow slices win: the launch is a long list of independent small
  // workgroups and the CUs overlap their routing-record and weight round trips across workgroups.
  int64_t bytes = 0;
  for (int i = 0; i < a.count; ++i)
    bytes += a.work_rows * a.batch.p[i].width * static_cast<int64_t>(a.batch.p[i].narrow) * 2;
  int u = bytes >= (32ll << 20) ? 4 : 2;
  if (a.batch.p[0].plan == nullptr) u = 4;  // every workgroup scans indices[] for its chunk: fewer of them
  if (tuning().bgmv_expand_cols > 0) u = tuning().bgmv_expand_cols;
  if (u >= 8) return launch_expand_u<D, 8>(a, stream);
  if (u <= 2) return launch_expand_u<D, 2>(a, stream);
  return launch_expand_u<D, 4>(a, stream);
}

template <typename D, int R, int NBLK>
static hipError_t launch_lora_blk(const BgmvArgs& a, hipStream_t stream) {
  constexpr int U = 4;
  constexpr int cols_per_wg = (kBgmvThreads / (R / 8)) * U * NBLK;
  BgmvBatch batch = a.batch;
  dim3 grid((a.wide_max + cols_per_wg - 1) / cols_per_wg, static_cast<unsigned>(a.grid_rows), a.count);
  // One wide projection batched with narrow ones, one column slice each, one to two workgroups per CU:
  // place the wide projection's workgroups on CUs of their own (balanced_slot).
  int balanced_chunks = 0, chunks_per_xcd = 0;
  if (grid.x == 1 && a.count > 1 && !tuning().bgmv_no_balance) {
    int widest = 0;
    for (int i = 1; i < a.count; ++i)
      if (batch.p[i].width > batch.p[widest].width) widest = i;
    bool same_chunks = true;
    for (int i = 0; i < a.count; ++i) same_chunks = same_chunks && batch.p[i].num_groups == batch.p[0].num_groups;
    const int per_xcd = (static_cast<int>(a.grid_rows) + kXcds - 1) / kXcds;
    const int slots = per_xcd * a.count;
    if (same_chunks && slots > 32 && slots <= 64) {
      std::swap(batch.p[0], batch.p[widest]);  // problems are independent: their order is free
      balanced_chunks = static_cast<int>(a.grid_rows);
      chunks_per_xcd = per_xcd;
      grid = dim3(kXcds * slots);
    }
  }
  // 8-byte y accesses need every problem's rows 8-byte aligned and no ragged last column group
  bool vec4 = true;
  for (int i = 0; i < a.count; ++i) {
    const BgmvProblem& p = batch.p[i];
    vec4 = vec4 && p.width % 4 == 0 && p.y_stride % 4 == 0 && p.y_offset % 4 == 0 &&
           reinterpret_cast<uintptr_t>(p.y) % 8 == 0;
  }
  if (vec4)
    hipLaunchKernelGGL((bgmv_lora_kernel<D, R, U, NBLK, true>), grid, dim3(kBgmvThreads), 0, stream, batch, a.h_in,
                       a.layer_idx, a.scale, a.count, balanced_chunks, chunks_per_xcd);
  else
    hipLaunchKernelGGL((bgmv_lora_kernel<D, R, U, NBLK, false>), grid, dim3(kBgmvThreads), 0, stream, batch,
                       a.h_in, a.layer_idx, a.scale, a.count, balanced_chunks, chunks_per_xcd);
  return hipGetLastError();
}

template <typename D, int R>
static hipError_t launch_lora_r(const BgmvArgs& a, hipStream_t stream) {
  // Every column slice of a projection repeats the shrink (its A slab comes from L2 after the first
  // slice), so slices are as wide as the launch can afford: a workgroup covers NBLK expand blocks of
  // 4 columns per lane group and holds all their B^T vectors in registers from the start.  A CU
  // streams only a small share of the chip's bandwidth, so the slices are narrowed until the
  // launch has workgroups for most of the 256 CUs.
  constexpr int cols4 = (kBgmvThreads / (R / 8)) * 4 * 4;
  int64_t wgs4 = 0;
  for (int i = 0; i < a.count; ++i) wgs4 += a.grid_rows * ((a.batch.p[i].width + cols4 - 1) / cols4);
  int nblk = wgs4 >= 200 ? 4 : (wgs4 >= 100 ? 2 : 1);
  if (tuning().bgmv_lora_blocks > 0) nblk = tuning().bgmv_lora_blocks;
  if (nblk >= 4) return launch_lora_blk<D, R, 4>(a, stream);
  if (nblk >= 2) return launch_lora_blk<D, R, 2>(a, stream);
  return launch_lora_blk<D, R, 1>(a, stream);
}

// y += (x A^T) B^T for planned problems of rank 8 or 16 (a.narrow); a.wide_max is the widest h_out.
hipError_t launch_bgmv_lora(const BgmvArgs& a, hipStream_t stream) {
  if (a.dtype == LORAX_F16)
    return a.narrow == 8 ? launch_lora_r<F16, 8>(a, stream) : launch_lora_r<F16, 16>(a, stream);
  return a.narrow == 8 ? launch_lora_r<BF16, 8>(a, stream) : launch_lora_r<BF16, 16>(a, stream);
}

hipError_t launch_bgmv(const BgmvArgs& a, hipStream_t stream) {
  if (a.dtype == LORAX_F16)
    return a.expand ? launch_expand<F16>(a, stream) : launch_shrink<F16>(a, stream);
  return a.expand ? launch_expand<BF16>(a, stream) : launch_shrink<BF16>(a, stream);
}

}  // namespace lorax
