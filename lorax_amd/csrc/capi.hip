// C ABI of liblorax_hip.so: argument validation, error reporting and dispatch to the kernel launchers.  The checks mirror the TORCH_CHECKs
// of the reference's pybind layer (punica_kernels/punica_ops.cc:291-411); what that
// layer reads from tensor metadata arrives here as plain integers.
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>

#include "kernels.h"

namespace lorax {
namespace {

constexpr int kMaxDevices = 64;
constexpr int kMaxRank = 128;  // BGMV_MAX_RANK / MAX_RANK_CUSTOM, punica.py:37-39

// Scratch of lorax_sgmv_shrink_static: device memory that exists from the moment the library is loaded, so that
// entry point never allocates.  Same layout as the caller's tmp of lorax_sgmv_shrink (kernels.h).  Every GPU
// holds its own copy at its own address; in host code the array's name is only a handle for the runtime (passed
// to a kernel it would be a host address and the kernel would fault), so the device address is asked for once
// per device and kept.
static __device__ __align__(256) unsigned char scratch[kShrinkScratchBytes];
std::atomic<unsigned char*> g_scratch_ptr[kMaxDevices];

thread_local char g_error[512] = "";
std::atomic<int> g_fixed_order_shrink{0};

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

#ifdef LORAX_TUNING_ENV
int env_int(const char* name) {
  const char* s = getenv(name);
  return s ? atoi(s) : 0;
}
#endif

// Address of `scratch` on `device`, asked for on first use with that device current.  Two threads that race here
// ask twice and store the same address, which is harmless.
int resolve_scratch(int device, unsigned char** out) {
  if (device < 0 || device >= kMaxDevices) return fail(LORAX_EINVAL, "device %d out of range", device);
  unsigned char* p = g_scratch_ptr[device].load(std::memory_order_acquire);
  if (p == nullptr) {
    int prev = 0;
    hipError_t e = hipGetDevice(&prev);
    if (e != hipSuccess) return fail(LORAX_ELAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
    if (prev != device) {
      e = hipSetDevice(device);
      if (e != hipSuccess) return fail(LORAX_ELAUNCH, "hipSetDevice(%d): %s", device, hipGetErrorString(e));
    }
    void* addr = nullptr;
    e = hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch));
    if (prev != device) (void)hipSetDevice(prev);
    if (e != hipSuccess || addr == nullptr)
      return fail(LORAX_ELAUNCH, "hipGetSymbolAddress(scratch) on device %d: %s", device, hipGetErrorString(e));
    p = static_cast<unsigned char*>(addr);
    g_scratch_ptr[device].store(p, std::memory_order_release);
  }
  *out = p;
  return LORAX_OK;
}

int check_common(const void* y, const void* x, const void* w_ptrs, int dtype) {
  if (y == nullptr || x == nullptr || w_ptrs == nullptr)
    return fail(LORAX_EINVAL, "null pointer argument (y=%p x=%p w_ptrs=%p)", y, x, w_ptrs);
  if (!aligned16(y) || !aligned16(x))
    return fail(LORAX_EINVAL, "y and x must be 16-byte aligned (y=%p x=%p)", y, x);
  if (dtype != LORAX_F16 && dtype != LORAX_BF16)
    return fail(LORAX_ENOKERNEL, "No suitable kernel. dtype=%d (only f16=0 and bf16=1)", dtype);
  return LORAX_OK;
}

}  // namespace

// Launch parameters are the launchers' own heuristics in the product build; a tuning build
// (-DLORAX_TUNING_ENV) lets LORAX_* environment variables override them, read once per process.
const Tuning& tuning() {
#ifndef LORAX_TUNING_ENV
  static const Tuning t = {};
#else
  static const Tuning t = {env_int("LORAX_BGMV_LORA_BLOCKS"), env_int("LORAX_BGMV_SHRINK_ROWS"), env_int("LORAX_SHRINK_KSPLIT"),
                           env_int("LORAX_SHRINK_MB"), env_int("LORAX_SHRINK_WAVES"), env_int("LORAX_EXPAND_ROWS"),
                           env_int("LORAX_SHRINK_NO_ROTATE"), env_int("LORAX_SHRINK_LDS"), env_int("LORAX_SHRINK_LDS_KB"), env_int("LORAX_BGMV_EXPAND_COLS"), env_int("LORAX_EXPAND_PANELS"), env_int("LORAX_BGMV_NO_RUNS"), env_int("LORAX_BGMV_NO_BALANCE"), env_int("LORAX_SHRINK_ROWS_MAX"), env_int("LORAX_SHRINK_ROWS"), env_int("LORAX_BGMV_SCALAR_Y")};
#endif
  return t;
}

bool fixed_order_shrink() { return g_fixed_order_shrink.load(std::memory_order_relaxed) != 0; }

}  // namespace lorax

using namespace lorax;

namespace {

// Validates one batch of BGMV problems that share num_tokens, direction and layer and launches it.
// Problem i maps its own h_in (the call's h_in where the field is 0) to its own h_out; shrink problems
// share h_in and may differ in rank (h_out), expand problems may differ in rank (h_in) and width.
int bgmv_batch(const lorax_bgmv_problem_t* problems, int32_t count, int64_t num_tokens, int32_t h_in,
               int64_t layer_idx, float scale, int32_t accumulate, int32_t dtype, void* stream) {
  if (count < 0 || count > kMaxBgmvProblems)
    return fail(LORAX_EINVAL, "num_problems=%d (at most %d per launch)", count, kMaxBgmvProblems);
  if (num_tokens < 0) return fail(LORAX_EINVAL, "num_tokens=%lld is negative", (long long)num_tokens);
  if (count == 0 || num_tokens == 0) return LORAX_OK;
  if (problems == nullptr) return fail(LORAX_EINVAL, "null pointer argument (problems)");
  if (layer_idx < 0) return fail(LORAX_EINVAL, "layer_idx=%lld is negative", (long long)layer_idx);
  BgmvArgs a{};
  a.count = count;
  a.expand = (problems[0].h_in > 0 ? problems[0].h_in : h_in) < problems[0].h_out;  // bgmv_impl.cuh:204
  a.wide_max = a.expand ? 0 : h_in;
  a.num_tokens = num_tokens;
  a.layer_idx = layer_idx;
  a.scale = scale;
  a.accumulate = accumulate;
  a.dtype = dtype;
  const bool planned = problems[0].plan != nullptr;
  for (int i = 0; i < count; ++i) {
    const lorax_bgmv_problem_t& q = problems[i];
    if ((q.plan != nullptr) != planned)
      return fail(LORAX_EINVAL, "problems of one launch must all carry a plan or none");
    if (planned) {
      if (int rc = check_common(q.y, q.x, q.plan, dtype)) return rc;
      if (q.num_groups < 0 || q.num_groups > 65535)
        return fail(LORAX_EINVAL, "num_groups=%d out of range", q.num_groups);
      if (q.num_groups > a.grid_rows) a.grid_rows = q.num_groups;
    } else {
      if (int rc = check_common(q.y, q.x, q.w_ptrs, dtype)) return rc;
      if (q.indices == nullptr) return fail(LORAX_EINVAL, "null pointer argument (indices)");
    }
    const int h_out = q.h_out;
    const int q_in = q.h_in > 0 ? q.h_in : h_in;
    const bool expand = q_in < h_out;
    const int narrow = expand ? q_in : h_out;
    const int wide = expand ? h_out : q_in;
    // bgmv_config.h:12-86 (narrow side 8..128).  The reference also wants both dims below 65536
    // (punica_ops.cc:310), which shuts out the LM head of models with large vocabularies and sends it to the
    // dense loop; here the wide side of an expand may be up to 2^20.
    const int wide_limit = expand ? (1 << 20) : 65536;
    if (q_in <= 0 || h_out <= 0 || wide >= wide_limit || narrow % 8 != 0 || narrow > kMaxRank || wide % 8 != 0)
      return fail(LORAX_ENOKERNEL, "No suitable kernel. h_in=%d h_out=%d dtype=%d", q_in, h_out, dtype);
    if (expand != a.expand)
      return fail(LORAX_EINVAL, "problems of one launch must share the direction (problem %d: h_in=%d h_out=%d)", i,
                  q_in, h_out);
    if (!expand && q_in != h_in)
      return fail(LORAX_EINVAL, "shrink problems of one launch share h_in=%d (problem %d: h_in=%d)", h_in, i, q_in);
    if (q.y_offset < 0 || q.y_stride < q.y_offset + h_out)
      return fail(LORAX_EINVAL, "y_offset=%lld y_stride=%lld do not hold h_out=%d columns",
                  (long long)q.y_offset, (long long)q.y_stride, h_out);
    if (a.expand && h_out > a.wide_max) a.wide_max = h_out;
    if (narrow > a.narrow) a.narrow = narrow;
    a.narrow_sum += narrow;
    // a planned problem reads neither table; its stacked-weight base (if any) travels in the field of the
    // direction's table instead (bgmv.hip: resolve_chunk)
    const int64_t* tab_a = planned ? static_cast<const int64_t*>(expand ? nullptr : q.a_stack) : q.w_ptrs;
    const int64_t* tab_b = planned ? static_cast<const int64_t*>(expand ? q.b_stack : nullptr) : q.indices;
    if (planned && ((expand ? q.b_stack : q.a_stack) != nullptr) && !aligned16(expand ? q.b_stack : q.a_stack))
      return fail(LORAX_EINVAL, "stacked weights must be 16-byte aligned (problem %d)", i);
    a.batch.p[i] = BgmvProblem{q.y, q.x, tab_a, tab_b, q.y_offset, q.y_stride, wide, narrow, q.plan, q.num_groups};
  }
  if (!planned) a.grid_rows = num_tokens;
  a.work_rows = planned ? a.grid_rows : (num_tokens + 1) / 2;
  if (a.grid_rows == 0) return LORAX_OK;
  if (accumulate != 0 && accumulate != 1)
    return fail(LORAX_EINVAL, "accumulate=%d (0 = overwrite, 1 = add)", accumulate);
  if (num_tokens > 65535)
    return fail(LORAX_ENOKERNEL, "No suitable kernel. num_tokens=%lld exceeds 65535", (long long)num_tokens);
  const hipError_t e = launch_bgmv(a, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(LORAX_ELAUNCH, "bgmv launch failed: %s", hipGetErrorString(e));
  return LORAX_OK;
}

// Copies a caller's row-tile plan into the launch arguments (null = the kernels search their tiles themselves).
int take_tiles(const lorax_sgmv_tiles_t* tiles, SgmvArgs& a) {
  if (tiles == nullptr || tiles->tiles == nullptr) return LORAX_OK;
  if (tiles->num_tiles < 0 || tiles->tile_rows < 1 || !aligned16(tiles->tiles))
    return fail(LORAX_EINVAL, "tile plan: num_tiles=%d tile_rows=%d tiles=%p (16-byte aligned records, tile_rows >= 1)",
                tiles->num_tiles, tiles->tile_rows, (const void*)tiles->tiles);
  a.tiles = reinterpret_cast<const int32_t*>(tiles->tiles);
  a.num_tiles = tiles->num_tiles;
  a.tile_rows = tiles->tile_rows;
  return LORAX_OK;
}

// Shape checks and launch shared by lorax_sgmv_shrink and lorax_sgmv_shrink_static.  `scratch_buf` is
// kShrinkScratchBytes of device memory (partial tiles, then arrival counters) or null.  A launch splits the hidden
// dimension across workgroups only as far as the scratch has room for (sgmv_shrink_ksplit, the K parts of the
// LDS-staged kernel).  With `whole_split` a call whose split would have to be cut back for lack of room is refused
// instead of being run with the shallower split.
int sgmv_shrink_checked(void* v, const void* x, const int64_t* w_ptrs, const int32_t* s_start, const int32_t* s_end,
                        int32_t num_segments, int64_t num_tokens, int32_t h_in, int32_t r, int32_t a_layout,
                        int64_t layer_idx, float scale, int32_t accumulate, void* scratch_buf, bool whole_split,
                        int32_t dtype, void* stream) {
  if (accumulate != 0 && accumulate != 1)
    return fail(LORAX_EINVAL, "accumulate=%d (0 = overwrite, 1 = add)", accumulate);
  if (int rc = check_common(v, x, w_ptrs, dtype)) return rc;
  if (s_start == nullptr || s_end == nullptr)
    return fail(LORAX_EINVAL, "null pointer argument (s_start=%p s_end=%p)", s_start, s_end);
  if (layer_idx < 0) return fail(LORAX_EINVAL, "layer_idx=%lld is negative", (long long)layer_idx);
  // [L, r, h_in]: multiples of 16 as in the reference (sgmv_config.h:10-15), and any multiple of 8 where the
  // LDS-staged kernel or the streaming kernel applies (sgmv_shrink_route decides, below)
  if (r < 8 || r > kMaxRank || r % 8 != 0 || h_in <= 0 || h_in % 8 != 0 || num_tokens > INT32_MAX / 2)
    return fail(LORAX_ENOKERNEL, "No suitable kernel. dtype=%d d_in=%d d_out=%d layout=%d", dtype, h_in,
                r, a_layout);
  SgmvArgs a{};
  a.y = v;
  a.x = x;
  a.w_ptrs = w_ptrs;
  a.s_start = s_start;
  a.s_end = s_end;
  a.num_segments = num_segments;
  a.num_tokens = num_tokens;
  a.d_in = h_in;
  a.d_out = r;
  a.a_layout = a_layout;
  a.layer_idx = layer_idx;
  a.dtype = dtype;
  a.scale = scale;
  a.accumulate = accumulate;
  if (scratch_buf != nullptr) {
    a.partials = static_cast<float*>(scratch_buf);
    a.partial_bytes = kPartialBytes;
    a.counters = reinterpret_cast<uint32_t*>(static_cast<unsigned char*>(scratch_buf) + kPartialBytes);
    a.num_counters = kNumCounters;
  }
  const ShrinkRoute route = sgmv_shrink_route(a);
  if (route == ShrinkRoute::kNone)
    return fail(LORAX_ENOKERNEL, "No suitable kernel. dtype=%d d_in=%d d_out=%d layout=%d", dtype, h_in, r, a_layout);
  if (whole_split && (route == ShrinkRoute::kLds || route == ShrinkRoute::kRegisters)) {
    SgmvArgs roomy = a;
    roomy.partial_bytes = SIZE_MAX / 2;
    const int want = route == ShrinkRoute::kLds ? sgmv_shrink_lds_kparts(a, SIZE_MAX / 2) : sgmv_shrink_ksplit(roomy);
    const int get = route == ShrinkRoute::kLds ? sgmv_shrink_lds_kparts(a, kPartialBytes) : sgmv_shrink_ksplit(a);
    if (want != get)
      return fail(LORAX_ESPACE,
                  "batch too large for the static scratch: %d parts of num_tokens * r * 4 = %lld bytes each, limit %zu "
                  "(num_tokens=%lld r=%d); call lorax_sgmv_shrink with a tmp buffer instead",
                  want, (long long)(num_tokens * r * 4), kPartialBytes, (long long)num_tokens, r);
  }
  const hipError_t e = launch_sgmv_shrink(a, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(LORAX_ELAUNCH, "sgmv_shrink launch failed: %s", hipGetErrorString(e));
  return LORAX_OK;
}

// Shape checks and launch shared by lorax_sgmv_expand and lorax_sgmv_expand_planned.
int sgmv_expand_checked(void* y, const void* v, const int64_t* w_ptrs, const int32_t* s_start, const int32_t* s_end,
                        int32_t num_segments, int64_t num_tokens, int32_t r, int32_t h_out, int32_t b_layout,
                        int64_t y_offset, int64_t y_stride, int64_t layer_idx, int32_t accumulate,
                        const lorax_sgmv_tiles_t* tiles, int32_t dtype, void* stream) {
  if (accumulate != 0 && accumulate != 1)
    return fail(LORAX_EINVAL, "accumulate=%d (0 = overwrite, 1 = add)", accumulate);
  if (b_layout != LORAX_B_RH && b_layout != LORAX_B_HR) return fail(LORAX_EINVAL, "b_layout=%d", b_layout);
  if (num_segments < 0 || num_tokens < 0)
    return fail(LORAX_EINVAL, "negative size (num_segments=%d num_tokens=%lld)", num_segments,
                (long long)num_tokens);
  if (num_segments == 0 || num_tokens == 0) return LORAX_OK;
  if (int rc = check_common(y, v, w_ptrs, dtype)) return rc;
  if (s_start == nullptr || s_end == nullptr)
    return fail(LORAX_EINVAL, "null pointer argument (s_start=%p s_end=%p)", s_start, s_end);
  if (layer_idx < 0) return fail(LORAX_EINVAL, "layer_idx=%lld is negative", (long long)layer_idx);
  if (r < 8 || r > kMaxRank || r % 8 != 0 || h_out <= 0 || h_out % 8 != 0 ||
      num_tokens > INT32_MAX / 2)
    return fail(LORAX_ENOKERNEL, "No suitable kernel. dtype=%d d_in=%d d_out=%d", dtype, r, h_out);
  if (y_offset < 0 || y_offset % 8 != 0 || y_stride % 8 != 0 || y_stride < y_offset + h_out)
    return fail(LORAX_EINVAL, "y_offset=%lld y_stride=%lld must be multiples of 8 holding h_out=%d columns",
                (long long)y_offset, (long long)y_stride, h_out);
  if (y_stride >= (1ll << 24))
    return fail(LORAX_EINVAL, "y_stride=%lld: rows of y hold fewer than 2^24 elements", (long long)y_stride);
  SgmvArgs a{};
  a.y = y;
  a.x = v;
  a.w_ptrs = w_ptrs;
  a.s_start = s_start;
  a.s_end = s_end;
  a.num_segments = num_segments;
  a.num_tokens = num_tokens;
  a.d_in = r;
  a.d_out = h_out;
  a.y_offset = y_offset;
  a.y_stride = y_stride;
  a.layer_idx = layer_idx;
  a.dtype = dtype;
  a.a_layout = b_layout;
  a.accumulate = accumulate;
  if (int rc = take_tiles(tiles, a)) return rc;
  if (a.tiles != nullptr && a.num_tiles == 0) return LORAX_OK;  // a plan without tiles: no segment has rows
  const hipError_t e = b_layout == LORAX_B_HR ? launch_sgmv_expand_t(a, static_cast<hipStream_t>(stream))
                                              : launch_sgmv_expand(a, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(LORAX_ELAUNCH, "sgmv_expand launch failed: %s", hipGetErrorString(e));
  return LORAX_OK;
}

}  // namespace

extern "C" {

int lorax_bgmv(void* y, const void* x, const int64_t* w_ptrs, const int64_t* indices,
               int64_t num_tokens, int32_t h_in, int32_t h_out, int64_t y_offset,
               int64_t y_stride, int64_t layer_idx, float scale, int32_t dtype, void* stream) {
  if (num_tokens == 0) return LORAX_OK;
  const lorax_bgmv_problem_t one{y, x, w_ptrs, indices, y_offset, y_stride, h_out, nullptr, 0, 0, nullptr, nullptr};
  return bgmv_batch(&one, 1, num_tokens, h_in, layer_idx, scale, 1, dtype, stream);
}

int lorax_bgmv_multi(const lorax_bgmv_problem_t* problems, int32_t num_problems, int64_t num_tokens,
                     int32_t h_in, int64_t layer_idx, float scale, int32_t accumulate, int32_t dtype,
                     void* stream) {
  return bgmv_batch(problems, num_problems, num_tokens, h_in, layer_idx, scale, accumulate, dtype, stream);
}

int lorax_sgmv_shrink(void* v, const void* x, const int64_t* w_ptrs, const int32_t* s_start,
                      const int32_t* s_end, int32_t num_segments, int64_t num_tokens,
                      int32_t h_in, int32_t r, int32_t a_layout, int64_t layer_idx, float scale,
                      void* tmp, int64_t tmp_bytes, int32_t dtype, void* stream) {
  if (num_segments < 0 || num_tokens < 0)
    return fail(LORAX_EINVAL, "negative size (num_segments=%d num_tokens=%lld)", num_segments,
                (long long)num_tokens);
  // Same contract as the reference: the custom kernel wants the 8 MiB buffer
  // (punica_ops.cc:389-390), the cutlass path 60 bytes per problem (punica_ops.cc:359).
  if (a_layout == LORAX_A_RH) {
    if (tmp_bytes != LORAX_SHRINK_TMP_BYTES)
      return fail(LORAX_ETMPSIZE, "CHECK_EQ(tmp.size(0), 8 * 1024 * 1024) failed. %lld vs %d",
                  (long long)tmp_bytes, LORAX_SHRINK_TMP_BYTES);
  } else if (a_layout == LORAX_A_HR) {
    if (tmp_bytes != static_cast<int64_t>(lorax_sgmv_tmp_size(num_segments)))
      return fail(LORAX_ETMPSIZE, "CHECK_EQ(tmp.size(0), sgmv_tmp_size(num_problems)) failed. %lld vs %zu",
                  (long long)tmp_bytes, lorax_sgmv_tmp_size(num_segments));
  } else {
    return fail(LORAX_EINVAL, "a_layout=%d (0 = [L,r,h_in], 1 = [L,h_in,r])", a_layout);
  }
  if (num_segments == 0 || num_tokens == 0) return LORAX_OK;
  if (tmp == nullptr && tmp_bytes > 0) return fail(LORAX_EINVAL, "null pointer argument (tmp)");
  // Split-K scratch: the caller's 8 MiB buffer, as in the reference (sgmv_all.cu:10-65 takes its partial sums
  // and its barrier words from tmp).  Its contents are never assumed: the counters are cleared by the launch.
  void* scratch_buf = (a_layout == LORAX_A_RH && aligned16(tmp)) ? tmp : nullptr;
  return sgmv_shrink_checked(v, x, w_ptrs, s_start, s_end, num_segments, num_tokens, h_in, r, a_layout, layer_idx,
                             scale, 1, scratch_buf, false, dtype, stream);
}

int lorax_sgmv_shrink_static(void* v, const void* x, const int64_t* w_ptrs, const int32_t* s_start,
                             const int32_t* s_end, int32_t num_segments, int64_t num_tokens, int32_t h_in,
                             int32_t r, int32_t a_layout, int64_t layer_idx, float scale, int32_t dtype,
                             void* stream) {
  if (num_segments < 0 || num_tokens < 0)
    return fail(LORAX_EINVAL, "negative size (num_segments=%d num_tokens=%lld)", num_segments,
                (long long)num_tokens);
  if (a_layout != LORAX_A_RH && a_layout != LORAX_A_HR)
    return fail(LORAX_EINVAL, "a_layout=%d (0 = [L,r,h_in], 1 = [L,h_in,r])", a_layout);
  if (num_segments == 0 || num_tokens == 0) return LORAX_OK;
  int device = 0;
  const hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return fail(LORAX_ELAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
  unsigned char* buf = nullptr;
  if (int rc = resolve_scratch(device, &buf)) return rc;
  return sgmv_shrink_checked(v, x, w_ptrs, s_start, s_end, num_segments, num_tokens, h_in, r, a_layout, layer_idx,
                             scale, 1, buf, true, dtype, stream);
}

int lorax_sgmv_shrink_multi(const lorax_sgmv_shrink_problem_t* problems, int32_t num_problems, const void* x,
                            const int32_t* s_start, const int32_t* s_end, int32_t num_segments,
                            int64_t num_tokens, int32_t h_in, int32_t r, int64_t layer_idx, float scale,
                            int32_t accumulate, void* tmp, int64_t tmp_bytes, const lorax_sgmv_tiles_t* tiles,
                            int32_t dtype, void* stream) {
  if (accumulate != 0 && accumulate != 1)
    return fail(LORAX_EINVAL, "accumulate=%d (0 = overwrite, 1 = add)", accumulate);
  if (num_problems < 1 || num_problems > kMaxShrinkGroup)
    return fail(LORAX_EINVAL, "num_problems=%d (1 to %d per call)", num_problems, kMaxShrinkGroup);
  if (problems == nullptr) return fail(LORAX_EINVAL, "null pointer argument (problems)");
  // One launch where the LDS-staged kernel takes the stacked rank and the batch is past the streaming
  // kernel's range; otherwise one launch per projection, with the same result.
  const int rows_max = tuning().shrink_rows_max != 0 ? tuning().shrink_rows_max : 512;
  const bool stacked = r >= 8 && r % 8 == 0 && num_problems * r <= kMaxRank && h_in > 0 &&
                       h_in % 128 == 0 && num_tokens > rows_max && tuning().shrink_lds >= 0;
  if (!stacked) {
    for (int i = 0; i < num_problems; ++i) {
      if (tmp_bytes < LORAX_SHRINK_TMP_BYTES)
        return fail(LORAX_ETMPSIZE, "CHECK_GE(tmp.size(0), 8 * 1024 * 1024) failed. %lld vs %d", (long long)tmp_bytes,
                    LORAX_SHRINK_TMP_BYTES);
      if (num_segments < 0 || num_tokens < 0)
        return fail(LORAX_EINVAL, "negative size (num_segments=%d num_tokens=%lld)", num_segments, (long long)num_tokens);
      if (num_segments == 0 || num_tokens == 0) continue;
      if (tmp == nullptr) return fail(LORAX_EINVAL, "null pointer argument (tmp)");
      const int rc = sgmv_shrink_checked(problems[i].v, x, problems[i].w_ptrs, s_start, s_end, num_segments, num_tokens,
                                         h_in, r, LORAX_A_RH, layer_idx, scale, accumulate, aligned16(tmp) ? tmp : nullptr,
                                         false, dtype, stream);
      if (rc != LORAX_OK) return rc;
    }
    return LORAX_OK;
  }
  if (num_segments < 0 || num_tokens < 0)
    return fail(LORAX_EINVAL, "negative size (num_segments=%d num_tokens=%lld)", num_segments, (long long)num_tokens);
  if (tmp_bytes < LORAX_SHRINK_TMP_BYTES)
    return fail(LORAX_ETMPSIZE, "CHECK_GE(tmp.size(0), 8 * 1024 * 1024) failed. %lld vs %d", (long long)tmp_bytes,
                LORAX_SHRINK_TMP_BYTES);
  if (num_segments == 0) return LORAX_OK;
  for (int i = 0; i < num_problems; ++i)
    if (int rc = check_common(problems[i].v, x, problems[i].w_ptrs, dtype)) return rc;
  if (s_start == nullptr || s_end == nullptr || tmp == nullptr)
    return fail(LORAX_EINVAL, "null pointer argument (s_start=%p s_end=%p tmp=%p)", s_start, s_end, tmp);
  if (layer_idx < 0) return fail(LORAX_EINVAL, "layer_idx=%lld is negative", (long long)layer_idx);
  if (num_tokens > INT32_MAX / 2)
    return fail(LORAX_ENOKERNEL, "No suitable kernel. dtype=%d d_in=%d d_out=%d layout=%d", dtype, h_in, r, LORAX_A_RH);
  SgmvArgs a{};
  a.y = problems[0].v;
  a.x = x;
  a.w_ptrs = problems[0].w_ptrs;
  a.s_start = s_start;
  a.s_end = s_end;
  a.num_segments = num_segments;
  a.num_tokens = num_tokens;
  a.d_in = h_in;
  a.d_out = num_problems * r;
  a.a_layout = LORAX_A_RH;
  a.layer_idx = layer_idx;
  a.dtype = dtype;
  a.scale = scale;
  a.accumulate = accumulate;
  if (aligned16(tmp)) {  // fp32 partial tiles of a launch that splits K
    a.partials = static_cast<float*>(tmp);
    a.partial_bytes = static_cast<size_t>(tmp_bytes);
  }
  a.group.count = num_problems;
  a.group.rank = r;
  for (int i = 0; i < num_problems; ++i) {
    a.group.v[i] = problems[i].v;
    a.group.w[i] = problems[i].w_ptrs;
  }
  if (int rc = take_tiles(tiles, a)) return rc;
  if (a.tiles != nullptr && a.num_tiles == 0) return LORAX_OK;  // a plan without tiles: no segment has rows
  const hipError_t e = launch_sgmv_shrink_lds(a, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(LORAX_ELAUNCH, "sgmv_shrink launch failed: %s", hipGetErrorString(e));
  return LORAX_OK;
}

int lorax_sgmv_expand(void* y, const void* v, const int64_t* w_ptrs, const int32_t* s_start,
                      const int32_t* s_end, int32_t num_segments, int64_t num_tokens, int32_t r,
                      int32_t h_out, int32_t b_layout, int64_t y_offset, int64_t y_stride,
                      int64_t layer_idx, int32_t accumulate, void* tmp, int64_t tmp_bytes, int32_t dtype,
                      void* stream) {
  if (num_segments >= 0 && tmp_bytes != static_cast<int64_t>(lorax_sgmv_tmp_size(num_segments)))  // punica_ops.cc:359
    return fail(LORAX_ETMPSIZE, "CHECK_EQ(tmp.size(0), sgmv_tmp_size(num_problems)) failed. %lld vs %zu",
                (long long)tmp_bytes, lorax_sgmv_tmp_size(num_segments));
  if (num_segments > 0 && num_tokens > 0 && tmp == nullptr && tmp_bytes > 0)
    return fail(LORAX_EINVAL, "null pointer argument (tmp)");
  return sgmv_expand_checked(y, v, w_ptrs, s_start, s_end, num_segments, num_tokens, r, h_out, b_layout, y_offset,
                             y_stride, layer_idx, accumulate, nullptr, dtype, stream);
}

int lorax_sgmv_expand_planned(void* y, const void* v, const int64_t* w_ptrs, const int32_t* s_start,
                              const int32_t* s_end, int32_t num_segments, int64_t num_tokens, int32_t r,
                              int32_t h_out, int64_t y_offset, int64_t y_stride, int64_t layer_idx,
                              int32_t accumulate, const lorax_sgmv_tiles_t* tiles, int32_t dtype, void* stream) {
  return sgmv_expand_checked(y, v, w_ptrs, s_start, s_end, num_segments, num_tokens, r, h_out, LORAX_B_HR, y_offset,
                             y_stride, layer_idx, accumulate, tiles, dtype, stream);
}

int lorax_bgmv_lora_multi(const lorax_bgmv_problem_t* problems, int32_t num_problems, int64_t num_tokens,
                          int32_t h_in, int32_t r, int64_t layer_idx, float scale, int32_t dtype,
                          void* stream) {
  if (num_problems < 0 || num_problems > kMaxFusedBgmvProblems)
    return fail(LORAX_EINVAL, "num_problems=%d (at most %d per launch)", num_problems, kMaxFusedBgmvProblems);
  if (num_tokens < 0) return fail(LORAX_EINVAL, "num_tokens=%lld is negative", (long long)num_tokens);
  if (num_problems == 0 || num_tokens == 0) return LORAX_OK;
  if (problems == nullptr) return fail(LORAX_EINVAL, "null pointer argument (problems)");
  if (layer_idx < 0) return fail(LORAX_EINVAL, "layer_idx=%lld is negative", (long long)layer_idx);
  if ((r != 8 && r != 16) || h_in <= 0 || h_in % 8 != 0 || h_in >= 65536)
    return fail(LORAX_ENOKERNEL, "No suitable kernel. fused shrink+expand covers rank 8 and 16, h_in=%d r=%d", h_in, r);
  BgmvArgs a{};
  a.count = num_problems;
  a.expand = true;
  a.narrow = r;
  a.h_in = h_in;
  a.num_tokens = num_tokens;
  a.layer_idx = layer_idx;
  a.scale = scale;
  a.accumulate = 1;
  a.dtype = dtype;
  for (int i = 0; i < num_problems; ++i) {
    const lorax_bgmv_problem_t& q = problems[i];
    if (int rc = check_common(q.y, q.x, q.plan, dtype)) return rc;
    if (q.num_groups < 0 || q.num_groups > 65535) return fail(LORAX_EINVAL, "num_groups=%d out of range", q.num_groups);
    if (q.h_out <= 0 || q.h_out % 8 != 0 || q.h_out >= 65536)
      return fail(LORAX_ENOKERNEL, "No suitable kernel. h_in=%d h_out=%d dtype=%d", h_in, q.h_out, dtype);
    if (q.y_offset < 0 || q.y_stride < q.y_offset + q.h_out)
      return fail(LORAX_EINVAL, "y_offset=%lld y_stride=%lld do not hold h_out=%d columns", (long long)q.y_offset,
                  (long long)q.y_stride, q.h_out);
    if (q.num_groups > a.grid_rows) a.grid_rows = q.num_groups;
    if (q.h_out > a.wide_max) a.wide_max = q.h_out;
    if ((q.a_stack == nullptr) != (q.b_stack == nullptr) || !aligned16(q.a_stack) || !aligned16(q.b_stack))
      return fail(LORAX_EINVAL, "a_stack and b_stack go together and must be 16-byte aligned (problem %d)", i);
    a.batch.p[i] = BgmvProblem{q.y,        q.x,        static_cast<const int64_t*>(q.a_stack), static_cast<const int64_t*>(q.b_stack),
                               q.y_offset, q.y_stride, q.h_out, r, q.plan, q.num_groups};
  }
  if (a.grid_rows == 0) return LORAX_OK;
  const hipError_t e = launch_bgmv_lora(a, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(LORAX_ELAUNCH, "bgmv launch failed: %s", hipGetErrorString(e));
  return LORAX_OK;
}

int lorax_sgmv_lora_multi(const lorax_sgmv_lora_problem_t* problems, int32_t num_problems, const void* x,
                          const int32_t* s_start, const int32_t* s_end, int32_t num_segments, int64_t num_tokens,
                          int32_t h_in, int32_t r, int64_t layer_idx, float scale, int32_t dtype, void* stream) {
  if (num_problems < 1 || num_problems > kMaxSgmvLoraProblems)
    return fail(LORAX_EINVAL, "num_problems=%d (1 to %d per launch)", num_problems, kMaxSgmvLoraProblems);
  if (num_segments < 0 || num_tokens < 0)
    return fail(LORAX_EINVAL, "negative size (num_segments=%d num_tokens=%lld)", num_segments, (long long)num_tokens);
  if (num_segments == 0 || num_tokens == 0) return LORAX_OK;
  if (problems == nullptr || s_start == nullptr || s_end == nullptr)
    return fail(LORAX_EINVAL, "null pointer argument (problems=%p s_start=%p s_end=%p)", (const void*)problems,
                (const void*)s_start, (const void*)s_end);
  if (layer_idx < 0) return fail(LORAX_EINVAL, "layer_idx=%lld is negative", (long long)layer_idx);
  if ((r != 8 && r != 16) || h_in <= 0 || h_in % 8 != 0 || h_in >= 65536 || num_tokens > 512)
    return fail(LORAX_ENOKERNEL,
                "No suitable kernel. the single-launch prefill update covers rank 8 and 16 and up to 512 rows, "
                "h_in=%d r=%d num_tokens=%lld", h_in, r, (long long)num_tokens);
  SgmvLoraArgs a{};
  a.count = num_problems;
  a.x = x;
  a.s_start = s_start;
  a.s_end = s_end;
  a.num_segments = num_segments;
  a.num_tokens = num_tokens;
  a.h_in = h_in;
  a.rank = r;
  a.layer_idx = layer_idx;
  a.scale = scale;
  a.dtype = dtype;
  for (int i = 0; i < num_problems; ++i) {
    const lorax_sgmv_lora_problem_t& q = problems[i];
    if (int rc = check_common(q.y, x, q.a_ptrs, dtype)) return rc;
    if (q.b_ptrs == nullptr) return fail(LORAX_EINVAL, "null pointer argument (b_ptrs)");
    if (q.h_out <= 0 || q.h_out % 8 != 0 || q.h_out >= 65536)
      return fail(LORAX_ENOKERNEL, "No suitable kernel. h_in=%d h_out=%d dtype=%d", h_in, q.h_out, dtype);
    if (q.y_offset < 0 || q.y_stride < q.y_offset + q.h_out)
      return fail(LORAX_EINVAL, "y_offset=%lld y_stride=%lld do not hold h_out=%d columns", (long long)q.y_offset,
                  (long long)q.y_stride, q.h_out);
    a.batch.p[i] = SgmvLoraProblem{q.y, q.a_ptrs, q.b_ptrs, q.y_offset, q.y_stride, q.h_out};
  }
  const hipError_t e = launch_sgmv_lora_rows(a, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(LORAX_ELAUNCH, "sgmv_lora launch failed: %s", hipGetErrorString(e));
  return LORAX_OK;
}

size_t lorax_sgmv_tmp_size(int32_t num_problems) {
  // 3 pointers + 3 int64 leading dimensions + one (m, n, k) int32 triple per problem
  return num_problems > 0 ? static_cast<size_t>(num_problems) * (3 * 8 + 3 * 8 + 12) : 0;
}

int lorax_init(int32_t device) {
  unsigned char* p = nullptr;
  if (int rc = resolve_scratch(device, &p)) return rc;
  // Per-kernel attributes (the dynamic LDS limit of the LDS-staged shrink) on that device, so that no launch
  // has anything left to set up - the first call of every entry point may already be under stream capture.
  int prev = 0;
  hipError_t e = hipGetDevice(&prev);
  if (e != hipSuccess) return fail(LORAX_ELAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
  if (prev != device) {
    e = hipSetDevice(device);
    if (e != hipSuccess) return fail(LORAX_ELAUNCH, "hipSetDevice(%d): %s", device, hipGetErrorString(e));
  }
  e = configure_sgmv_shrink_lds();
  if (prev != device) (void)hipSetDevice(prev);
  if (e != hipSuccess) return fail(LORAX_ELAUNCH, "kernel set-up on device %d: %s", device, hipGetErrorString(e));
  return LORAX_OK;
}

int lorax_set_fixed_order_shrink(int32_t on) { return g_fixed_order_shrink.exchange(on != 0 ? 1 : 0); }

size_t lorax_workspace_bytes(void) { return kShrinkScratchBytes; }

const char* lorax_last_error(void) { return g_error; }

const char* lorax_version(void) { return "lorax_hip 0.1.0 (gfx950)"; }

}  // extern "C"
