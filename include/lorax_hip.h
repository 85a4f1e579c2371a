/*
 * lorax_hip.h - C ABI of liblorax_hip.so, the gfx950 (MI355X) implementation of the
 * multi-adapter LoRA hot path of predibase/lorax (BGMV decode, SGMV prefill).
 *
 * Every entry point replaces one function of the reference's pybind module
 * `punica_kernels` (server/punica_kernels/punica_kernels/punica_ops.cc:446-459).
 * All pointers are device pointers in the current HIP device's memory unless the
 * comment says otherwise.  `stream` is a hipStream_t passed as void* (NULL = the
 * default stream).  No entry point allocates, frees or synchronises, and none keeps state
 * between calls; every one is safe to call while `stream` is being captured into a HIP graph.
 *
 * Return value: 0 on success, a LORAX_E* code otherwise; the message for the last
 * failure on the calling thread is returned by lorax_last_error().  Errors are
 * reported synchronously from host-side argument validation and from the launch
 * call itself, never later.
 *
 * Element types: x, y, v and all weights share one 16-bit float type (`dtype`);
 * accumulation is fp32.  Rounding points follow the reference's BGMV kernels
 * (bgmv_impl.cuh:141,189-190) and its per-adapter fallback loop
 * (lorax_server/utils/layers.py:206-210,190): the fp32 dot product is rounded to
 * `dtype`, then added to the destination in fp32 and rounded again.
 */
#ifndef LORAX_HIP_H
#define LORAX_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LORAX_OK 0
#define LORAX_EINVAL 1     /* bad argument (null pointer, negative size, bad dtype)         */
#define LORAX_ENOKERNEL 2  /* shape outside what the kernels cover ("No suitable kernel.") */
#define LORAX_ELAUNCH 3    /* the HIP runtime refused the launch                            */
#define LORAX_ETMPSIZE 4   /* tmp buffer size does not match the reference's contract       */
#define LORAX_ESPACE 5     /* an output buffer of the caller is too small; sizes are reported */

#define LORAX_F16 0
#define LORAX_BF16 1

/* A layouts accepted by lorax_sgmv_shrink (one adapter's stack, row-major):
 *   LORAX_A_RH: [num_layers, r, h_in]  - what the reference's custom sgmv_shrink reads
 *                                        (sgmv_flashinfer.cuh:13-353; ranks 16..128)
 *   LORAX_A_HR: [num_layers, h_in, r]  - what its cutlass grouped GEMM reads
 *                                        (sgmv_cutlass.cuh:46; rank 8)               */
#define LORAX_A_RH 0
#define LORAX_A_HR 1

/* B layouts accepted by lorax_sgmv_expand (one adapter's stack, row-major):
 *   LORAX_B_RH: [num_layers, r, h_out] - what the reference's cutlass grouped GEMM reads
 *                                        (sgmv_cutlass.cuh:46-47; adapters/lora.py:274-281)
 *   LORAX_B_HR: [num_layers, h_out, r] - the transposed stack the reference keeps for BGMV decode
 *                                        (adapters/lora.py:117-126, weights_b_t); the faster
 *                                        one here: a column panel is one contiguous run      */
#define LORAX_B_RH 0
#define LORAX_B_HR 1

/* Size in bytes of the shrink scratch the reference API passes around
 * (lorax_server/utils/punica.py:145-147; checked at punica_ops.cc:389-390). */
#define LORAX_SHRINK_TMP_BYTES (8 * 1024 * 1024)

/*
 * BGMV, both directions.  Replaces dispatch_bgmv (punica_ops.cc:291-334) and the
 * kernels behind it (bgmv/bgmv_impl.cuh:15-285).
 *
 *   for every token b in [0, num_tokens) with idx = indices[b] >= 0:
 *     W = (dtype*)w_ptrs[idx] + layer_idx * h_out * h_in          // [h_out, h_in]
 *     y[b * y_stride + y_offset + j] += dtype(scale * sum_k W[j, k] * x[b * h_in + k])
 *   tokens with indices[b] < 0 are not touched and w_ptrs is not read for them.
 *
 * h_in < h_out selects "expand" (h_in is the LoRA rank), otherwise "shrink"
 * (h_out is the rank), as bgmv_impl.cuh:204.  The rank must be a multiple of 8 in
 * [8, 128]; the wide dimension a multiple of 8, below 65536 for a shrink (punica_ops.cc:310) and
 * below 2^20 for an expand (so that the LM head of a large-vocabulary model is served too).
 * The reference binds y_offset = 0 and y_stride = h_out (punica_ops.cc:318); other
 * values let a caller write one projection's slice of a fused q/k/v or gate/up
 * output in place.
 */
int lorax_bgmv(void* y, const void* x, const int64_t* w_ptrs, const int64_t* indices,
               int64_t num_tokens, int32_t h_in, int32_t h_out, int64_t y_offset,
               int64_t y_stride, int64_t layer_idx, float scale, int32_t dtype, void* stream);

/*
 * Several BGMV problems in one launch.  No counterpart in the reference, whose caller issues
 * one dispatch_bgmv per projection and rank group (lorax_server/utils/layers.py:143-164); it
 * exists because a decode-size BGMV is shorter than a launch, so the projections that share an
 * input (q/k/v, gate/up) are better issued together.
 *
 * `problems` is a HOST array of `num_problems` (<= 16) descriptors; the pointers inside are
 * device pointers.  All problems share num_tokens, layer_idx, scale, dtype and the direction
 * (h_in < h_out means expand).  Shrink problems share h_in and may differ in rank (their h_out);
 * expand problems may differ in rank (the problem's own h_in field) and in h_out - so the rank
 * groups of a multi-rank batch (lorax_server/adapters/lora.py:339-348, one kernel call per rank
 * in the reference) go out in ONE shrink launch and ONE expand launch.  Each problem is computed
 * exactly as by lorax_bgmv.  accumulate = 0 stores dtype(sum) instead of adding it (meant for
 * shrink launches, so that the caller need not zero v first; an expand launch takes it too); rows
 * of tokens whose index is negative are not written in either mode.
 *
 * Routing plan (optional).  Finding which tokens share an adapter costs every workgroup a scan
 * of indices[]; a caller that builds the index tables on the host anyway (as the reference does,
 * lorax_server/adapters/lora.py:354-375) can hand over the result instead: `plan` points to
 * num_groups records of 8 int64 in device memory,
 *   [0] number of tokens in the chunk (1..4)   [1..4] their row numbers (unused ones repeat [1])
 *   [5] device address of the adapter's A stack [L, r, h_in]  (read by shrink launches)
 *   [6] device address of the adapter's B^T stack [L, h_out, r] (read by expand launches)
 *   [7] reserved
 * where every chunk holds tokens of ONE adapter and every routed token is in exactly one chunk.
 * A record whose word [0] is 0 is padding and is skipped, so a plan can be kept at a fixed number of
 * records for graph replay (the reference pads its tables the same way, utils/graph.py:71-73,421-425).
 * With a plan, w_ptrs and indices are not read and may be NULL.
 *
 * Stacked weights.  The reference's newer path keeps preloaded adapters in ONE tensor per layer and projection,
 * lora_a [num_adapters, r, h_in] and lora_b [num_adapters, h_out, r] (lorax_server/models/model.py:289-334,
 * utils/punica.py:689-748), and routes with an entry number per token.  A planned problem serves it directly:
 * with a_stack (shrink launches) / b_stack (expand launches) set to the tensor's base address, plan words [5] and
 * [6] hold the adapter's ENTRY NUMBER instead of an address, layer_idx must be 0, and one plan - built once per
 * batch from the per-token entry numbers - serves every layer and projection.
 */
typedef struct lorax_bgmv_problem {
  void* y;                /* [num_tokens, y_stride] output                         */
  const void* x;          /* [num_tokens, h_in] input                              */
  const int64_t* w_ptrs;  /* device addresses of the adapters' [L, h_out, h_in] stacks */
  const int64_t* indices; /* [num_tokens] index into w_ptrs, negative = no adapter */
  int64_t y_offset;       /* first output column inside a row of y                 */
  int64_t y_stride;       /* row pitch of y in elements                            */
  int32_t h_out;
  const int64_t* plan;    /* optional routing plan (see above), else NULL          */
  int32_t num_groups;     /* records in plan                                       */
  int32_t h_in;           /* this problem's input width; 0 = the call's h_in       */
  const void* a_stack;    /* stacked weights (see above), else NULL                */
  const void* b_stack;
} lorax_bgmv_problem_t;

int lorax_bgmv_multi(const lorax_bgmv_problem_t* problems, int32_t num_problems, int64_t num_tokens,
                     int32_t h_in, int64_t layer_idx, float scale, int32_t accumulate, int32_t dtype,
                     void* stream);

/*
 * Shrink and expand of up to 4 projections in one launch: for every planned token chunk
 *   y[t, y_offset : y_offset + h_out] += dtype(scale * dtype(x[t] @ A^T) @ B^T)
 * with A and B^T taken from plan words [5] and [6].  No counterpart in the reference (it is the
 * pair add_lora_a_bgmv + add_lora_b_bgmv of lorax_server/utils/layers.py:146-164 without the
 * intermediate v tensor and the second launch).  Every problem needs a routing plan; the rank r
 * must be 8 or 16, because each column slice of a projection recomputes the shrink and the
 * adapter's A slab has to be small for that to pay.  The intermediate x @ A^T is rounded to
 * dtype exactly as the two-call sequence rounds it when it stores v.
 */
int lorax_bgmv_lora_multi(const lorax_bgmv_problem_t* problems, int32_t num_problems, int64_t num_tokens,
                          int32_t h_in, int32_t r, int64_t layer_idx, float scale, int32_t dtype,
                          void* stream);

/*
 * SGMV shrink.  Replaces sgmv_shrink (punica_ops.cc:369-411,
 * sgmv_flashinfer/sgmv_all.cu:10-65) for a_layout = LORAX_A_RH and the shrink
 * direction of sgmv_cutlass (punica_ops.cc:338-367, sgmv/sgmv_cutlass.cuh:132-178)
 * for a_layout = LORAX_A_HR.
 *
 *   for every segment i in [0, num_segments) with s_end[i] > s_start[i]:
 *     A = (dtype*)w_ptrs[i] + layer_idx * r * h_in
 *     v[s_start[i]:s_end[i], :] += dtype(x[s_start[i]:s_end[i], :] @ A_as_[h_in, r])
 *   empty or negative segments are skipped without reading w_ptrs[i]
 *   (sgmv_cutlass.cuh:39-44).  Rows at or beyond num_tokens are never accessed.
 *   `scale` multiplies the fp32 sums before they are rounded (1 in every call of the reference's
 *   legacy path; the `scaling` argument of lorax_server/utils/ops/sgmv_shrink.py:101-196).
 *
 * r must be a multiple of 8 in [8, 128]; h_in a multiple of 8; LORAX_A_RH with a rank that is not a
 * multiple of 16 additionally needs h_in to be a multiple of 128 or num_tokens <= 512.
 *
 * `tmp`/`tmp_bytes` is the caller's scratch, with the reference's sizes (8 MiB for LORAX_A_RH, punica_ops.cc:
 * 389-390; lorax_sgmv_tmp_size(num_segments) for LORAX_A_HR, punica_ops.cc:359).  For LORAX_A_RH the launch
 * may write it (fp32 partial sums, and arrival counters, when the hidden dimension is split across workgroups:
 * batches of roughly 500 to 2000 rows, and h_in that is not a multiple of 128); nothing is expected in it on
 * entry and nothing of value is left in it.  As in the reference, two shrinks that are in flight at the same time (different streams) must
 * not share one tmp buffer.
 */
int lorax_sgmv_shrink(void* v, const void* x, const int64_t* w_ptrs, const int32_t* s_start,
                      const int32_t* s_end, int32_t num_segments, int64_t num_tokens,
                      int32_t h_in, int32_t r, int32_t a_layout, int64_t layer_idx, float scale,
                      void* tmp, int64_t tmp_bytes, int32_t dtype, void* stream);

/*
 * lorax_sgmv_shrink without a tmp argument and without any allocation.  It has no counterpart in the reference;
 * it is for callers that cannot allocate device memory or hand a scratch buffer over: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  Whenever it returns LORAX_OK the result is
 * bit-identical to lorax_sgmv_shrink's on the same arguments.  The scratch is an array of LORAX_SHRINK_TMP_BYTES
 * (8 MiB) inside the library's own device image, one copy per GPU, held until the process ends; its address on a
 * device is looked up on the first call there (or by lorax_init).
 *
 * Limit: a launch that splits the hidden dimension across workgroups (batches of fewer than 192 row tiles, i.e.
 * up to a few thousand rows) keeps one fp32 copy of v per part in the array, and all parts of the split the
 * launcher chooses for the shape must fit: parts * num_tokens * 16 * ceil(r / 16) * 4 bytes <= 8 MiB - 64 KiB.
 * A call beyond that fails with LORAX_ESPACE and launches nothing (lorax_sgmv_shrink runs the same call with a
 * shallower split, which is slower; here that never happens silently).  In practice only shapes served by the
 * register-operand kernel (h_in not a multiple of 128) with around ten thousand rows reach the limit; calls that
 * do not split - most - use no scratch and have no limit.  All calls on one GPU share that GPU's array: calls
 * that overlap in time on one GPU (different streams or threads) race; calls on one stream, or ordered by events,
 * do not.  Nothing needs to be cleared between calls (the arrival counters are cleared by every launch that uses
 * them, partial sums are written before they are read).
 */
int lorax_sgmv_shrink_static(void* v, const void* x, const int64_t* w_ptrs, const int32_t* s_start,
                             const int32_t* s_end, int32_t num_segments, int64_t num_tokens, int32_t h_in,
                             int32_t r, int32_t a_layout, int64_t layer_idx, float scale, int32_t dtype,
                             void* stream);

/*
 * Row-tile plan of an SGMV launch (optional; no counterpart in the reference's custom shrink, which searches its
 * tiles on the device, sgmv_flashinfer.cuh:41-60; its cutlass path precomputes a problem table on the device,
 * sgmv/sgmv_cutlass.cuh:30-52).  The segment kernels cut every segment into row tiles.  Given only s_start / s_end in device
 * memory, every workgroup finds its tile by scanning those tables and the grid is sized for an upper bound of the
 * tile count.  A caller that knows the segment lengths on the host can pass the finished list instead:
 * `tiles` points to num_tiles records in DEVICE memory, each rows [row0, row_end) of segment `seg` (an index into
 * the call's s_start / s_end / w_ptrs tables; row0 >= s_start[seg], row_end <= s_end[seg]), `index` the tile's
 * number inside its segment.  Every row of every non-empty segment must be in exactly one tile, and no tile may
 * be higher than tile_rows.  lorax_sgmv_plan_tiles builds such a list from host copies of the tables (and
 * lorax_build_batch_tables emits one per rank group).  Records are clamped on the device to the call's
 * num_segments, num_tokens and tile_rows, and a tile whose segment has a null table entry is skipped, so a wrong
 * plan gives wrong results but reads and writes x, v and y inside the call's bounds only (a tile may not name a
 * segment whose table entry dangles: the entry is dereferenced, as it would be for a non-empty segment).  The results do not depend on how a batch is cut into tiles, except that the shrink's last
 * rounding can (its sums over the hidden dimension are added in an order that depends on the tile, see
 * lorax_sgmv_shrink_multi).
 */
typedef struct lorax_sgmv_tile {
  int32_t seg;
  int32_t row0;
  int32_t row_end;
  int32_t index;
} lorax_sgmv_tile_t;

typedef struct lorax_sgmv_tiles {
  const lorax_sgmv_tile_t* tiles; /* device memory, 16-byte aligned */
  int32_t num_tiles;
  int32_t tile_rows;              /* upper bound of row_end - row0 over the list */
} lorax_sgmv_tiles_t;

#define LORAX_TILES_SHRINK 0 /* for lorax_sgmv_shrink_multi: tiles of at most 64 rows                    */
#define LORAX_TILES_EXPAND 1 /* for lorax_sgmv_expand_planned: tiles of about 256 rows                   */

/*
 * Builds a tile plan on the HOST: s_start / s_end are host copies of the segment tables of the launch (empty and
 * negative segments get no tile, bounds are clamped to [0, num_tokens]).  Writes up to `capacity` records to
 * `tiles` (host memory; the caller uploads them), the number of records to *num_tiles and the bound of their
 * heights to *tile_rows.  `rank` is the LoRA rank of the launch (shrink tiles are not made lower than a quarter
 * of it; 0 = unknown).  Returns LORAX_ESPACE, with *num_tiles set, when capacity is too small (or tiles NULL).
 */
int lorax_sgmv_plan_tiles(const int32_t* s_start, const int32_t* s_end, int32_t num_segments, int64_t num_tokens,
                          int32_t kind, int32_t rank, lorax_sgmv_tile_t* tiles, int32_t capacity,
                          int32_t* num_tiles, int32_t* tile_rows);

/*
 * SGMV shrink of up to 4 projections that share x, the segments and the rank (q/k/v, gate/up), LORAX_A_RH
 * stacks: problem p gets v_p[s:e, :] += dtype(scale * x[s:e, :] @ A_p^T) exactly as from lorax_sgmv_shrink
 * with (v_p, w_ptrs_p).  The reference launches one shrink per projection (lorax_server/utils/layers.py:
 * 121-133, punica_ops.cc:369-411) and reads x once per launch; here, when num_problems * r <= 128, h_in is a
 * multiple of 128 and the batch has more than 512 rows, the projections run as ONE launch that reads x once
 * (their A matrices are stacked into one rank-(num_problems * r) tile).  Otherwise the call issues one
 * launch per projection.  `tmp`/`tmp_bytes`: at least LORAX_SHRINK_TMP_BYTES of scratch, as for lorax_sgmv_shrink
 * with LORAX_A_RH; a larger buffer is accepted and changes nothing (a launch that splits the hidden dimension
 * across workgroups keeps its fp32 partial sums in the first 8 MiB, so that the result does not depend on the
 * buffer's size).  num_problems = 1 is allowed.
 * accumulate = 1 adds to v as lorax_sgmv_shrink does; accumulate = 0 stores dtype(scale * x @ A^T) into the rows
 * of the segments instead, so the caller need not zero v first (rows outside every segment keep their contents;
 * lorax_sgmv_expand reads no others).  The reference zero-fills v before every shrink (punica.py:176-178).
 * `tiles`: optional row-tile plan (LORAX_TILES_SHRINK) for the call's segment tables, or NULL; it is used by the
 * one-launch path and ignored otherwise.
 * Order of the sums: a row tile walks the hidden dimension from a starting point that depends on the tile (its
 * adapter's stack address, its number inside the segment, the XCD it runs on), and launches with few tiles cut
 * the hidden dimension into parts whose fp32 sums are added afterwards.  A call is deterministic, but the last
 * rounding of an element of v can differ between two batches that hold the same row (within the parity
 * tolerance by a wide margin: one spacing of dtype on a few percent of the elements).
 * lorax_set_fixed_order_shrink(1) trades speed for reproducibility: every tile then walks from k = 0 and no launch
 * cuts the hidden dimension, so a row's result depends on nothing but the row and its adapter.
 */
typedef struct {
  void* v;               /* [num_tokens, r] */
  const int64_t* w_ptrs; /* [num_segments] addresses of [num_layers, r, h_in] stacks */
} lorax_sgmv_shrink_problem_t;

int lorax_sgmv_shrink_multi(const lorax_sgmv_shrink_problem_t* problems, int32_t num_problems, const void* x,
                            const int32_t* s_start, const int32_t* s_end, int32_t num_segments,
                            int64_t num_tokens, int32_t h_in, int32_t r, int64_t layer_idx, float scale,
                            int32_t accumulate, void* tmp, int64_t tmp_bytes, const lorax_sgmv_tiles_t* tiles,
                            int32_t dtype, void* stream);

/* Process-wide switch (default 0): 1 = the SGMV shrinks add their sums over the hidden dimension in one fixed
 * order whatever the batch (see lorax_sgmv_shrink_multi).  Returns the previous value.  Not meant to be flipped
 * while launches are being issued from other threads. */
int lorax_set_fixed_order_shrink(int32_t on);

/*
 * Shrink and expand of a SHORT prefill batch in one launch, for up to 4 projections that share x and the
 * segment tables:
 *   y_p[s:e, y_offset_p : y_offset_p + h_out_p] += dtype(scale * dtype(x[s:e] @ A_p,i^T) @ B_p,i^T)   per segment i
 * with A_p,i = a_ptrs_p[i] ([num_layers, r, h_in] stack) and B_p,i = b_ptrs_p[i] ([num_layers, h_out, r] stack).
 * No counterpart in the reference: it is the sequence zero-fill, sgmv_shrink, sgmv_cutlass of
 * lorax_server/utils/layers.py:114-142 (punica.py:170-196) without the intermediate tensor and two of the three
 * launches, for batches that are bound by launches rather than bytes.  The intermediate x @ A^T is rounded to
 * dtype exactly where the two-call sequence rounds it when it stores v.  r must be 8 or 16 and num_tokens at
 * most 512; empty and negative segments are skipped without reading their table entries' stacks.
 */
typedef struct lorax_sgmv_lora_problem {
  void* y;                /* [num_tokens, y_stride]                                  */
  const int64_t* a_ptrs;  /* [num_segments] device addresses of [L, r, h_in] stacks  */
  const int64_t* b_ptrs;  /* [num_segments] device addresses of [L, h_out, r] stacks */
  int64_t y_offset;
  int64_t y_stride;
  int32_t h_out;
} lorax_sgmv_lora_problem_t;

int lorax_sgmv_lora_multi(const lorax_sgmv_lora_problem_t* problems, int32_t num_problems, const void* x,
                          const int32_t* s_start, const int32_t* s_end, int32_t num_segments, int64_t num_tokens,
                          int32_t h_in, int32_t r, int64_t layer_idx, float scale, int32_t dtype, void* stream);

/*
 * SGMV expand.  Replaces the expand direction of sgmv_cutlass (punica_ops.cc:338-367,
 * sgmv/sgmv_cutlass.cuh:86-131).
 *
 *   for every segment i with s_end[i] > s_start[i]:
 *     B = (dtype*)w_ptrs[i] + layer_idx * r * h_out                  // [r, h_out] (LORAX_B_RH)
 *     y[s:e, y_offset : y_offset + h_out] += dtype(v[s:e, :] @ B)    // row pitch y_stride
 *   With b_layout = LORAX_B_HR the stack holds B^T, [h_out, r] per layer, and the result is the same.
 *   accumulate = 1 is the reference's only mode; accumulate = 0 stores dtype(v @ B) into the rows of the
 *   segments instead of adding it (add_inputs=False of lorax_server/utils/ops/sgmv_expand.py:106-121).
 *
 * r must be a multiple of 8 in [8, 128]; h_out, y_offset and y_stride multiples of 8; y_stride < 2^24
 * (a row tile of y is addressed with 32-bit element offsets).
 */
int lorax_sgmv_expand(void* y, const void* v, const int64_t* w_ptrs, const int32_t* s_start,
                      const int32_t* s_end, int32_t num_segments, int64_t num_tokens, int32_t r,
                      int32_t h_out, int32_t b_layout, int64_t y_offset, int64_t y_stride,
                      int64_t layer_idx, int32_t accumulate, void* tmp, int64_t tmp_bytes,
                      int32_t dtype, void* stream);

/*
 * lorax_sgmv_expand over B^T stacks (LORAX_B_HR) with a row-tile plan (LORAX_TILES_EXPAND) and without the tmp
 * argument, which that kernel has no use for.  No counterpart in the reference.  Same result as lorax_sgmv_expand,
 * bit for bit (every element of the update is one dot product over r whatever the tiling); `tiles` may be NULL.
 */
int lorax_sgmv_expand_planned(void* y, const void* v, const int64_t* w_ptrs, const int32_t* s_start,
                              const int32_t* s_end, int32_t num_segments, int64_t num_tokens, int32_t r,
                              int32_t h_out, int64_t y_offset, int64_t y_stride, int64_t layer_idx,
                              int32_t accumulate, const lorax_sgmv_tiles_t* tiles, int32_t dtype, void* stream);

/* Bytes of grouped-GEMM argument scratch for `num_problems` segments.  Replaces
 * sgmv_tmp_size (sgmv/sgmv_cutlass.cuh:54-58): 3 pointers + 3 int64 + one
 * 3 x int32 problem size per segment = 60 * num_problems. */
size_t lorax_sgmv_tmp_size(int32_t num_problems);

/*
 * Routing tables of one batch for ALL layer types, built on the host into one packed buffer (one
 * host-to-device copy).  Replaces, per step, find_segments (lorax_server/utils/segments.py:6-34) and
 * the table building of BatchLoraWeights.load for every layer type (lorax_server/adapters/lora.py:
 * 290-396: grouping of segments by rank, pointer tables, segment bounds, per-token indices), and adds the
 * routing plan of lorax_bgmv_multi / lorax_bgmv_lora_multi.  Runs on the CPU; touches no GPU state.
 *
 * adapter_indices[num_tokens]: adapter of every token (any value; tokens of adapters without an entry
 *   are not routed).  entries: for layer type 0, 1, ... the adapters that have weights for it
 *   (entry_counts[t] of them, sorted by `adapter`), with the device addresses of their resident stacks.
 * Outputs: segment_bounds[num_tokens + 1] / segment_owners[num_tokens] (first *num_segments + 1 / *num_segments
 *   used); `groups`: one descriptor per (layer type, rank), ranks in order of first appearance, with byte
 *   offsets into `packed`.  Returns LORAX_ESPACE when `packed` or `groups` is too small (or NULL), with
 *   *packed_bytes and *num_groups set to what is needed.
 * Segment tables (use_sgmv = 1) keep the segments of one adapter next to each other (the order of a group's
 *   segments is free).  A group with at least 32 segments of at most 4 rows - decode tokens inside a prefill
 *   batch - lists those after the longer ones and also gets a routing plan over their rows (records as for
 *   lorax_bgmv_multi): a caller may run lorax_sgmv_shrink / lorax_sgmv_expand over the first
 *   num_long_segments entries and lorax_bgmv_multi over the plan, on the same v and y, instead of the segment
 *   kernels over the whole table.  The reference routes every row of such a batch through its segment kernels
 *   (lorax_server/adapters/lora.py:279, server/lorax_server/models/flash_causal_lm.py:1594).
 * Every segment-table group also carries the row-tile plans of its first num_long_segments segments for
 *   lorax_sgmv_shrink_multi and lorax_sgmv_expand_planned (the builder has the segment lengths anyway).
 */
typedef struct lorax_adapter_entry {
  int64_t adapter; /* adapter index as it appears in adapter_indices            */
  int64_t a_addr;  /* device address of the [L, r, h_in] stack                   */
  int64_t b_addr;  /* device address of the [L, h_out, r] stack                  */
  int32_t rank;
  int32_t reserved;
} lorax_adapter_entry_t;

typedef struct lorax_table_group {
  int32_t layer_type;   /* index into entry_counts                                       */
  int32_t rank;
  int32_t use_sgmv;     /* 1: segment tables (prefill, or a rank above 128); 0: per-token */
  int32_t num_segments; /* entries of the group's pointer tables                          */
  int32_t num_chunks;   /* routing-plan records: of all routed tokens (use_sgmv = 0), of the rows of
                           the group's short segments (use_sgmv = 1, 0 = no such plan)            */
  int32_t num_long_segments; /* use_sgmv = 1 with a plan: the tables list the segments of more than 4
                           rows first, this many; the plan covers the rest.  Else num_segments    */
  int64_t a_ptr_off;    /* int64[num_segments] stack addresses per segment                */
  int64_t b_ptr_off;
  int64_t starts_off;   /* int32[num_segments] (use_sgmv = 1), else -1                    */
  int64_t ends_off;
  int64_t indices_off;  /* int64[num_tokens] slot in the group's tables or -1 (use_sgmv = 0) */
  int64_t plan_off;     /* int64[num_chunks][8] routing plan, -1 = none                   */
  /* use_sgmv = 1: row-tile plans over the first num_long_segments entries of the tables (lorax_sgmv_tile_t
     records at these offsets; -1 = none) */
  int64_t shrink_tiles_off;
  int64_t expand_tiles_off;
  int32_t num_shrink_tiles;
  int32_t shrink_tile_rows;
  int32_t num_expand_tiles;
  int32_t expand_tile_rows;
} lorax_table_group_t;

int lorax_build_batch_tables(const int64_t* adapter_indices, int64_t num_tokens,
                             const lorax_adapter_entry_t* entries, const int32_t* entry_counts,
                             int32_t num_layer_types, int32_t prefill, int32_t* segment_bounds,
                             int64_t* segment_owners, int32_t* num_segments, void* packed,
                             int64_t packed_capacity, int64_t* packed_bytes, lorax_table_group_t* groups,
                             int32_t group_capacity, int32_t* num_groups);

/*
 * Per-device set-up: looks up the address of the static scratch of lorax_sgmv_shrink_static on `device`.
 * Nothing is allocated (every other entry point takes its scratch from the caller, as the reference does,
 * punica.py:145-167).  Optional: lorax_sgmv_shrink_static does the same on its first call on a device.
 */
int lorax_init(int32_t device);

/* Device memory the library itself holds per GPU, in bytes (the static scratch). */
size_t lorax_workspace_bytes(void);

/* Message of the last error on this thread ("" if none).  Host pointer, valid until
 * the next failing call on the same thread. */
const char* lorax_last_error(void);

/* Library version string (host pointer, static). */
const char* lorax_version(void);

#ifdef __cplusplus
}
#endif
#endif /* LORAX_HIP_H */
