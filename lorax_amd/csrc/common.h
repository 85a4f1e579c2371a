// Shared device helpers for the gfx950 LoRA kernels: 16-bit float element traits,
// 128-bit vector access, wave64 reductions and the token-grouping scan used by BGMV.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lorax {

constexpr int kWave = 64;

typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

// Element traits.  E is the 16-bit storage type; vec8 is eight of them (16 bytes).
// dot2(a, b, c) = c + a.lo * b.lo + a.hi * b.hi on one packed pair of 16-bit elements, fp32
// accumulate (v_dot2_f32_f16 / v_dot2_f32_bf16): two multiply-adds per instruction and no
// conversion of the operands, which is what keeps the decode kernels off the vector-ALU limit.
struct F16 {
  using E = _Float16;
  using vec8 = f16x8;
  static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    typedef _Float16 pair __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(pair, a), __builtin_bit_cast(pair, b), c, false);
  }
  static __device__ __forceinline__ f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};
struct BF16 {
  using E = __bf16;
  using vec8 = bf16x8;
  static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    typedef __bf16 pair __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(pair, a), __builtin_bit_cast(pair, b), c, false);
  }
  static __device__ __forceinline__ f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};

template <typename D>
__device__ __forceinline__ float to_f32(typename D::E v) {
  return static_cast<float>(v);
}
// Round-to-nearest-even conversion to the storage type.
template <typename D>
__device__ __forceinline__ typename D::E from_f32(float v) {
  return static_cast<typename D::E>(v);
}

// y <- D(float(y) + float(D(delta))): the reference's two rounding points
// (bgmv_impl.cuh:141, layers.py:190,210).
template <typename D>
__device__ __forceinline__ typename D::E accumulate(typename D::E y, float delta) {
  return from_f32<D>(to_f32<D>(y) + to_f32<D>(from_f32<D>(delta)));
}

// Four adjacent elements (8 bytes, 8-byte aligned) updated with one load and one store.
template <typename D>
__device__ __forceinline__ void accumulate4(typename D::E* p, f32x4 delta) {
  typedef typename D::E vec4 __attribute__((ext_vector_type(4)));
  vec4 y = *reinterpret_cast<const vec4*>(p);
#pragma unroll
  for (int i = 0; i < 4; ++i) y[i] = accumulate<D>(y[i], delta[i]);
  *reinterpret_cast<vec4*>(p) = y;
}

// The same for a destination that is overwritten: the old value counts as zero.
template <typename D>
__device__ __forceinline__ void overwrite4(typename D::E* p, f32x4 delta) {
  typedef typename D::E vec4 __attribute__((ext_vector_type(4)));
  vec4 y;
#pragma unroll
  for (int i = 0; i < 4; ++i) y[i] = from_f32<D>(delta[i]);
  *reinterpret_cast<vec4*>(p) = y;
}
template <typename D>
__device__ __forceinline__ void update4(bool add, typename D::E* p, f32x4 delta) {
  if (add) accumulate4<D>(p, delta); else overwrite4<D>(p, delta);
}

// All tensors and weight stacks live in device (global) memory.  Weight addresses arrive as
// integers, which the compiler can only treat as generic pointers (flat_load); the explicit
// address space turns every 16-byte access into global_load/global_store_dwordx4.
#define LORAX_GLOBAL __attribute__((address_space(1)))

template <typename D>
__device__ __forceinline__ typename D::vec8 load8(const typename D::E* p) {
  return *(const LORAX_GLOBAL typename D::vec8*)(p);
}
template <typename D>
__device__ __forceinline__ void store8(typename D::E* p, typename D::vec8 v) {
  *(LORAX_GLOBAL typename D::vec8*)(p) = v;
}
// c + sum of the 8 products of two 16-byte vectors.
template <typename D>
__device__ __forceinline__ float dot8(typename D::vec8 a, typename D::vec8 b, float c) {
  const u32x4 ab = __builtin_bit_cast(u32x4, a);
  const u32x4 bb = __builtin_bit_cast(u32x4, b);
#pragma unroll
  for (int i = 0; i < 4; ++i) c = D::dot2(ab[i], bb[i], c);
  return c;
}

// v if keep, else zeros - a select on registers, for masking AFTER an unconditional load.
template <typename D>
__device__ __forceinline__ typename D::vec8 keep_if(bool keep, typename D::vec8 v) {
  u32x4 bits = __builtin_bit_cast(u32x4, v);
#pragma unroll
  for (int i = 0; i < 4; ++i) bits[i] = keep ? bits[i] : 0u;
  return __builtin_bit_cast(typename D::vec8, bits);
}
template <typename D>
__device__ __forceinline__ typename D::vec8 zero8() {
  typename D::vec8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = static_cast<typename D::E>(0.0f);
  return z;
}

__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

// Cross-lane sums without the LDS crossbar.  __shfl_xor compiles to ds_bpermute_b32, an LDS instruction with an
// address register and a round trip through the LDS pipeline; every lane distance the reductions of these kernels
// use has a cheaper form on gfx950:
//   1, 2     DPP quad_perm (folds into the add that consumes it)
//   4        two DPP row shifts, each writing the banks (groups of four lanes) it serves
//   8        DPP row_ror:8
//   16, 32   v_permlane16_swap / v_permlane32_swap, which exchange half of one register with half of another:
//            with (a, b) in, r0 + r1 out is a + a(lane ^ M) in the lanes whose bit M is clear and b + b(lane ^ M)
//            in the others - the exchange step of a transposing reduction in two instructions, no select.
// Results are bit-identical to the __shfl_xor forms: the same two values are added (fp32 add commutes).
template <int CTRL, int BANKS>
__device__ __forceinline__ float dpp_move(float old, float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, v),
                                                               CTRL, 0xF, BANKS, false));
}
// v of lane (lane ^ M), M in {1, 2, 4, 8}.
template <int M>
__device__ __forceinline__ float lane_xor_dpp(float v) {
  static_assert(M == 1 || M == 2 || M == 4 || M == 8, "DPP reaches lanes of the same row of 16");
  if constexpr (M == 1) return dpp_move<0xB1, 0xF>(v, v);  // quad_perm [1, 0, 3, 2]
  if constexpr (M == 2) return dpp_move<0x4E, 0xF>(v, v);  // quad_perm [2, 3, 0, 1]
  if constexpr (M == 8) return dpp_move<0x128, 0xF>(v, v);  // row_ror:8
  // M == 4: lanes 0-3 and 8-11 of a row take lane + 4 (row_shl:4), lanes 4-7 and 12-15 take lane - 4 (row_shr:4)
  const float up = dpp_move<0x104, 0x5>(v, v);
  return dpp_move<0x114, 0xA>(up, v);
}
// keep + send(lane ^ M), where a lane keeps lo and sends hi if its bit M is clear, and keeps hi and sends lo if set.
template <int M>
__device__ __forceinline__ float fold_pair(float lo, float hi, bool upper) {
  if constexpr (M == 32) {
    const auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned, lo), __builtin_bit_cast(unsigned, hi),
                                                    false, false);
    // (elements copied out before the bit casts: a bit cast applied to r[1] directly reads r[0])
    const unsigned r0 = r[0], r1 = r[1];
    return __builtin_bit_cast(float, r0) + __builtin_bit_cast(float, r1);
  } else if constexpr (M == 16) {
    const auto r = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(unsigned, lo), __builtin_bit_cast(unsigned, hi),
                                                    false, false);
    const unsigned r0 = r[0], r1 = r[1];
    return __builtin_bit_cast(float, r0) + __builtin_bit_cast(float, r1);
  } else {
    const float keep = upper ? hi : lo;
    const float send = upper ? lo : hi;
    return keep + lane_xor_dpp<M>(send);
  }
}
// v + v(lane ^ M)
template <int M>
__device__ __forceinline__ float xor_add(float v) {
  if constexpr (M >= 16) return fold_pair<M>(v, v, false);
  else return v + lane_xor_dpp<M>(v);
}

// Inclusive prefix sum over the 64 lanes of a wave with DPP row shifts and the two row broadcasts (six VALU
// instructions of a few cycles each where six __shfl_up are six dependent trips through the LDS crossbar).
template <int CTRL, int ROWS>
__device__ __forceinline__ int dpp_add_from(int v) {
  // lanes whose source is outside the row (or whose row is masked off) add nothing
  return v + __builtin_amdgcn_update_dpp(0, v, CTRL, ROWS, 0xF, true);
}
__device__ __forceinline__ int wave_inclusive_scan(int v) {
  v = dpp_add_from<0x111, 0xF>(v);  // row_shr:1
  v = dpp_add_from<0x112, 0xF>(v);  // row_shr:2
  v = dpp_add_from<0x114, 0xF>(v);  // row_shr:4
  v = dpp_add_from<0x118, 0xF>(v);  // row_shr:8 - every row of 16 lanes now holds its own prefix sums
  v = dpp_add_from<0x142, 0xA>(v);  // row_bcast15 into rows 1 and 3: + total of the row before
  v = dpp_add_from<0x143, 0xC>(v);  // row_bcast31 into rows 2 and 3: + total of rows 0 and 1
  return v;
}
// v of lane `src`, src wave-uniform.
__device__ __forceinline__ int read_lane(int v, int src) {
  return __builtin_amdgcn_readlane(v, __builtin_amdgcn_readfirstlane(src));
}

// Sum over the 64 lanes of a wave; every lane receives the total.
__device__ __forceinline__ float wave_sum(float v) {
  v = xor_add<32>(v);
  v = xor_add<16>(v);
  v = xor_add<8>(v);
  v = xor_add<4>(v);
  v = xor_add<2>(v);
  return xor_add<1>(v);
}

// Sum over aligned groups of CP lanes (CP a power of two <= 16); every lane of a group receives its total.
// Distances from CP / 2 down to 1, the order the kernels have always added in.
template <int CP>
__device__ __forceinline__ float group_sum(float v) {
  static_assert(CP >= 1 && CP <= 16 && (CP & (CP - 1)) == 0, "CP must be a power of two <= 16");
  if constexpr (CP >= 16) v = xor_add<8>(v);
  if constexpr (CP >= 8) v = xor_add<4>(v);
  if constexpr (CP >= 4) v = xor_add<2>(v);
  if constexpr (CP >= 2) v = xor_add<1>(v);
  return v;
}

// Reduces N per-lane values across the wave with N-1+log2(64/N) exchanges instead of
// 6*N: at every step a lane hands half of its values to the partner lane and keeps
// the sum of the other half.  On return lane l holds in vals[0] the wave-wide total
// of the input value with index transpose_reduce_index<N>(l).
template <int M, int N>
__device__ __forceinline__ void transpose_reduce_step(float (&vals)[N], int n, bool upper) {
  const int half = n >> 1;
#pragma unroll
  for (int i = 0; i < N / 2; ++i) {
    if (i < half) {
      float lo = vals[i];
      float hi = vals[i + half];
      // Opaque to the optimiser: without this it rewrites "upper ? vals[i + half] : vals[i]"
      // into a load with a lane-dependent index, which costs an N-way select chain per access.
      asm volatile("" : "+v"(lo), "+v"(hi));
      vals[i] = fold_pair<M>(lo, hi, upper);
    }
  }
}
template <int N>
__device__ __forceinline__ void transpose_reduce(float (&vals)[N]) {
  static_assert(N >= 1 && N <= 64 && (N & (N - 1)) == 0, "N must be a power of two <= 64");
  const int lane = lane_id();
  // distance 32 with n = N values, 16 with N / 2, ...; once one value is left the remaining distances are plain sums
  if constexpr (N >= 2) transpose_reduce_step<32>(vals, N, (lane & 32) != 0); else vals[0] = xor_add<32>(vals[0]);
  if constexpr (N >= 4) transpose_reduce_step<16>(vals, N / 2, (lane & 16) != 0); else vals[0] = xor_add<16>(vals[0]);
  if constexpr (N >= 8) transpose_reduce_step<8>(vals, N / 4, (lane & 8) != 0); else vals[0] = xor_add<8>(vals[0]);
  if constexpr (N >= 16) transpose_reduce_step<4>(vals, N / 8, (lane & 4) != 0); else vals[0] = xor_add<4>(vals[0]);
  if constexpr (N >= 32) transpose_reduce_step<2>(vals, N / 16, (lane & 2) != 0); else vals[0] = xor_add<2>(vals[0]);
  if constexpr (N >= 64) transpose_reduce_step<1>(vals, N / 32, (lane & 1) != 0); else vals[0] = xor_add<1>(vals[0]);
}

// Index of the input value whose total lane `lane` holds after transpose_reduce<N>.
template <int N>
__device__ __forceinline__ int transpose_reduce_index(int lane) {
  int idx = 0;
  int n = N;
  int m = 32;
  for (; n > 1; n >>= 1, m >>= 1) {
    if (lane & m) idx += n >> 1;
  }
  return idx;
}

// XCD-aware workgroup numbering.  The 8 XCDs of an MI355X each have their own L2 and receive
// workgroups round-robin by linear workgroup id, so neighbours in the grid never share an L2.
// This maps the hardware id to a virtual (x, y, z) in which consecutive virtual ids - x fastest,
// then z, then y - run on ONE XCD: the workgroups that read the same activation rows (all row or
// column slices and all batched problems of one token chunk) then hit the same L2 instead of
// fetching those rows once per XCD.
constexpr unsigned kXcds = 8;

struct VirtualBlock {
  int x, y, z;
};

__device__ __forceinline__ VirtualBlock xcd_virtual_block() {
  const unsigned gx = gridDim.x, gy = gridDim.y, gz = gridDim.z;
  const unsigned n = gx * gy * gz;
  const unsigned lin = blockIdx.x + gx * (blockIdx.y + gy * blockIdx.z);
  const unsigned per = n / kXcds, rem = n % kXcds;  // XCD k runs per + (k < rem) workgroups
  const unsigned xcd = lin % kXcds, slot = lin / kXcds;
  const unsigned v = xcd * per + (xcd < rem ? xcd : rem) + slot;
  VirtualBlock b;
  b.x = static_cast<int>(v % gx);
  b.z = static_cast<int>((v / gx) % gz);
  b.y = static_cast<int>(v / (gx * gz));
  return b;
}

// The same for a one-dimensional grid: consecutive virtual ids run on one XCD.
__device__ __forceinline__ unsigned xcd_virtual_id() {
  const unsigned n = gridDim.x;
  const unsigned per = n / kXcds, rem = n % kXcds;
  const unsigned xcd = blockIdx.x % kXcds, slot = blockIdx.x / kXcds;
  return xcd * per + (xcd < rem ? xcd : rem) + slot;
}

// Token grouping for BGMV.  Tokens that share an indices[] value share one adapter; the
// tokens of one adapter are cut, in token order, into chunks of at most G and the
// first token of each chunk ("leader") processes the whole chunk, so the adapter's
// weights are fetched once per chunk instead of once per token.
//
// Called by every wave of the workgroup of token b with identical arguments; all
// results are wave-uniform.  Returns the number of tokens in b's chunk (>= 1) if b
// leads a chunk, with toks[0] = b and toks[1..] the followers in ascending order;
// returns 0 if b is a follower or has no adapter (the workgroup has nothing to do).
// idx receives indices[b].
//
// The scan reads the index array in batches of kScanBlocks * 64 entries whose loads are
// all issued before the first one is consumed, so a batch costs one memory round trip.
constexpr int kScanBlocks = 8;

template <int G>
__device__ __forceinline__ int group_tokens(const int64_t* __restrict__ indices, int num_tokens,
                                            int b, int64_t& idx, int (&toks)[G]) {
  const int lane = lane_id();
#pragma unroll
  for (int g = 0; g < G; ++g) toks[g] = b;
  const int b_blk = b & ~(kWave - 1);
  int before = 0;
  int n = 1;
  bool first_batch = true;
  for (int base = 0; base < num_tokens; base += kWave * kScanBlocks) {
    int64_t vals[kScanBlocks];
#pragma unroll
    for (int c = 0; c < kScanBlocks; ++c) {
      const int t = base + c * kWave + lane;
      vals[c] = t < num_tokens ? indices[t] : static_cast<int64_t>(-1);
    }
    if (first_batch) {
      idx = indices[b];
      if (idx < 0) return 0;
      if (G == 1) return 1;
      first_batch = false;
    }
#pragma unroll
    for (int c = 0; c < kScanBlocks; ++c) {
      const int t0 = base + c * kWave;
      if (t0 < num_tokens) {
        uint64_t mask = __ballot(vals[c] == idx);
        if (t0 < b_blk) {
          before += __popcll(mask);
        } else {
          if (t0 == b_blk) {
            const uint64_t below = (1ull << (b - b_blk)) - 1ull;
            before += __popcll(mask & below);
            if ((before % G) != 0) return 0;
            mask &= ~(below | (1ull << (b - b_blk)));
          }
          while (mask != 0 && n < G) {
            const int pos = __ffsll(static_cast<unsigned long long>(mask)) - 1;
            mask &= mask - 1;
#pragma unroll
            for (int g = 1; g < G; ++g) {
              if (g == n) toks[g] = t0 + pos;
            }
            ++n;
          }
          if (n == G) return n;
        }
      }
    }
  }
  return n;
}

}  // namespace lorax
