// Internal interface between the C ABI (capi.hip) and the kernel launchers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/lorax_hip.h"
#include "common.h"

namespace lorax {

// One BGMV problem of a batched launch: its own output, input, pointer table and routing.
// `width` is the problem's wide dimension (h_out of an expand, the shared h_in of a shrink) and
// `narrow` its LoRA rank; problems of one launch may differ in rank.
struct BgmvProblem {
  void* y;
  const void* x;
  const int64_t* w_ptrs;
  const int64_t* indices;
  int64_t y_offset;
  int64_t y_stride;
  int width;
  int narrow;
  const int64_t* plan;  // optional routing plan: num_groups records of kPlanRecordWords int64
  int num_groups;
};

constexpr int kMaxBgmvProblems = 16;
constexpr int kMaxFusedBgmvProblems = 4;  // the single-launch shrink+expand keeps its batch small
constexpr int kPlanRecordWords = 8;

// Workgroup numbering of the shrink and expand launches (one-dimensional grid).  Consecutive problems
// with the same number of token chunks (the projections of one rank group: same routing) form a run.  A
// run owns the ids [base, run_end); inside it an id is chunk * run_subs + s, and s in [sub_lo[i], sub_hi[i])
// is row block / column slice s - sub_lo[i] of problem i.  All workgroups of one token chunk are then
// neighbours - on one XCD, sharing the chunk's input rows through its L2 - and every launched workgroup
// has a problem, a chunk and a slice of its own, whatever the mix of ranks, widths and routings.
struct BgmvBatch {
  BgmvProblem p[kMaxBgmvProblems];
  int run_end[kMaxBgmvProblems];
  int base[kMaxBgmvProblems];
  int run_subs[kMaxBgmvProblems];
  int sub_lo[kMaxBgmvProblems];
  int sub_hi[kMaxBgmvProblems];
};

struct BgmvArgs {
  BgmvBatch batch;
  int count;          // problems in the batch (grid z)
  bool expand;        // bgmv_impl.cuh:204: h_in < h_out
  int narrow;         // largest LoRA rank of the batch (the fused kernel: the rank)
  int narrow_sum;     // sum of the problems' ranks
  int wide_max;       // shrink: h_in; expand and fused: widest h_out of the batch
  int h_in;           // fused shrink+expand only: hidden size of x
  int64_t num_tokens;
  int64_t grid_rows;  // workgroup rows: tokens when chunks are found by scanning, else plan records
  int64_t work_rows;  // estimate of the rows that have work (sizes the rows-per-workgroup choice)
  int64_t layer_idx;
  float scale;
  int accumulate;     // 0 = overwrite the routed rows of y, 1 = add to y
  int dtype;
};

// Projections that share x, the segment tables and the rank, shrunk in one launch (the LDS-staged kernel
// treats them as one problem whose rank is the sum): outputs and pointer tables per projection.
constexpr int kMaxShrinkGroup = 4;
struct ShrinkGroup {
  void* v[kMaxShrinkGroup];
  const int64_t* w[kMaxShrinkGroup];
  int count;
  int rank;  // of each projection
};

struct SgmvArgs {
  void* y;        // v for shrink, y for expand
  const void* x;  // x for shrink, v for expand
  const int64_t* w_ptrs;
  const int32_t* s_start;
  const int32_t* s_end;
  int num_segments;
  int64_t num_tokens;
  int d_in;
  int d_out;
  int a_layout;  // shrink: LORAX_A_*; expand: LORAX_B_*
  int64_t y_offset;
  int64_t y_stride;
  int64_t layer_idx;
  int dtype;
  ShrinkGroup group;  // shrink of several projections: count > 1, d_out = count * rank; else unused
  float scale;     // shrink: factor applied to the fp32 sums before rounding (1 in the reference's calls)
  int accumulate;  // 1 = add to the destination (the reference's only mode), 0 = overwrite the rows of the segments
  // scratch of the shrink's split-K (the caller's tmp, or the library's static array): fp32 partial tiles and one
  // arrival counter per row tile; null = no scratch, the launch does not split K across workgroups
  float* partials;
  size_t partial_bytes;
  uint32_t* counters;
  size_t num_counters;
  // optional row-tile plan of the caller (lorax_sgmv_tiles_t): device records, their number, their height bound
  const int32_t* tiles;
  int num_tiles;
  int tile_rows;
};

// Shrink and expand of a short prefill batch in one launch (bgmv.hip): up to four projections that share x and
// the segment tables, each with its own stack tables and column window of y.
constexpr int kMaxSgmvLoraProblems = 4;
struct SgmvLoraProblem {
  void* y;
  const int64_t* a_ptrs;  // [num_segments] addresses of [L, r, h_in] stacks
  const int64_t* b_ptrs;  // [num_segments] addresses of [L, h_out, r] stacks
  int64_t y_offset;
  int64_t y_stride;
  int h_out;
};
struct SgmvLoraBatch {
  SgmvLoraProblem p[kMaxSgmvLoraProblems];
};
struct SgmvLoraArgs {
  SgmvLoraBatch batch;
  int count;
  const void* x;
  const int32_t* s_start;
  const int32_t* s_end;
  int num_segments;
  int64_t num_tokens;
  int h_in;
  int rank;
  int64_t layer_idx;
  float scale;
  int dtype;
};
hipError_t launch_sgmv_lora_rows(const SgmvLoraArgs& a, hipStream_t stream);

// Launch parameters that can be overridden from the environment for tuning runs, read once per process;
// 0 (unset) = the launcher's heuristic.
struct Tuning {
  int bgmv_lora_blocks;  // LORAX_BGMV_LORA_BLOCKS: expand blocks per workgroup of the single-launch BGMV (1, 2, 4)
  int bgmv_shrink_rows;  // LORAX_BGMV_SHRINK_ROWS: rows of A per workgroup of the BGMV shrink (2, 4, 8)
  int shrink_ksplit;     // LORAX_SHRINK_KSPLIT: K splits (parts) across workgroups of the SGMV shrinks
  int shrink_mb;         // LORAX_SHRINK_MB: 16-row blocks per row tile of the SGMV shrink (1, 2, 4)
  int shrink_waves;      // LORAX_SHRINK_WAVES: waves per workgroup of the register-operand SGMV shrink
  int expand_rows;       // LORAX_EXPAND_ROWS: rows per tile of the SGMV expand
  int shrink_no_rotate;  // LORAX_SHRINK_NO_ROTATE: SGMV shrinks whose tiles all walk the hidden dimension from k = 0
  int shrink_lds;  // LORAX_SHRINK_LDS: 1 = always take the LDS-staged shrink where it applies, -1 = never
  int shrink_lds_kb;  // LORAX_SHRINK_LDS_KB: LDS budget of the staged shrink's buffers
  int bgmv_expand_cols;  // LORAX_BGMV_EXPAND_COLS: columns per lane group of the BGMV expand (4, 8, 16)
  int expand_panels;  // LORAX_EXPAND_PANELS: column panels per wave of the transposed-B expand
  int bgmv_no_runs;   // LORAX_BGMV_NO_RUNS: number workgroups problem by problem
  int bgmv_no_balance;  // LORAX_BGMV_NO_BALANCE: plain workgroup numbering in the single-launch BGMV
  int shrink_rows_max;  // LORAX_SHRINK_ROWS_MAX: largest token count served by the streaming SGMV shrink (-1 = never)
  int shrink_rows;      // LORAX_SHRINK_ROWS: rows per tile of the LDS-staged SGMV shrink (below its buffers' height)
  int bgmv_scalar_y;    // LORAX_BGMV_SCALAR_Y: BGMV expand that moves y element by element even where rows are aligned
};
const Tuning& tuning();
// lorax_set_fixed_order_shrink: the SGMV shrinks walk the hidden dimension from k = 0 in every tile and never cut
// it across workgroups.
bool fixed_order_shrink();

hipError_t launch_bgmv(const BgmvArgs& a, hipStream_t stream);
hipError_t launch_bgmv_lora(const BgmvArgs& a, hipStream_t stream);
hipError_t launch_sgmv_shrink(const SgmvArgs& a, hipStream_t stream);
hipError_t launch_sgmv_expand(const SgmvArgs& a, hipStream_t stream);
hipError_t launch_sgmv_expand_t(const SgmvArgs& a, hipStream_t stream);  // B stacks stored as [L, h_out, r]
// LDS-staged shrink (sgmv_shrink_lds.hip): [L, r, h_in] layout, h_in a multiple of 128.
bool sgmv_shrink_lds_applies(const SgmvArgs& a);
hipError_t launch_sgmv_shrink_lds(const SgmvArgs& a, hipStream_t stream);
// Per-device set-up of the LDS-staged shrink on the current device (the dynamic LDS limit of every instantiation),
// so that no launch has first-call state; a launch that finds it missing does it itself.
hipError_t configure_sgmv_shrink_lds();
// Streaming shrink for a handful of rows (bgmv.hip): [L, r, h_in] layout, any h_in the BGMV kernels take.
hipError_t launch_sgmv_shrink_rows(const SgmvArgs& a, hipStream_t stream);

// Which kernel serves an SGMV shrink call (launch_sgmv_shrink dispatches on it; the C ABI derives from it
// which shapes it accepts).
enum class ShrinkRoute {
  kNone,       // no kernel takes the shape
  kRows,       // streaming kernel for a few hundred rows, [L, r, h_in]
  kLds,        // LDS-staged MFMA kernel, [L, r, h_in], h_in a multiple of 128; launches of few row tiles cut K
               // into parts and keep the parts' fp32 sums in the scratch
  kRegisters,  // register-operand MFMA kernel, [L, r, h_in], r a multiple of 16; may split K across workgroups
               // (fp32 partial tiles and arrival counters in the scratch)
  kNarrowRows  // [L, h_in, r] layout (rank 8 in the reference)
};
ShrinkRoute sgmv_shrink_route(const SgmvArgs& a);

// Layout of the shrink scratch, the same inside the caller's 8 MiB tmp buffer and inside the library's static
// array: fp32 partial tiles first, then the arrival counters.
constexpr size_t kShrinkScratchBytes = 8u << 20;
constexpr size_t kShrinkCounterBytes = 64u << 10;
constexpr size_t kPartialBytes = kShrinkScratchBytes - kShrinkCounterBytes;
constexpr size_t kNumCounters = kShrinkCounterBytes / sizeof(uint32_t);
// K splits the register-operand shrink would use for this call given its scratch (1 = none).
int sgmv_shrink_ksplit(const SgmvArgs& a);
// Parts the LDS-staged shrink would cut the hidden dimension into given `room` bytes for their fp32 sums.
int sgmv_shrink_lds_kparts(const SgmvArgs& a, size_t room);

}  // namespace lorax
