// Shared device helpers for the gfx950 kernels: bf16 bit handling, fixed-order reductions,
// the transcendental primitives every kernel variant of one op must share, launch checks.
//
// Determinism rules used throughout this library:
//   * compiled with -ffp-contract=off: a fused multiply-add happens only where __builtin_fmaf
//     is written, so the rounding points of every expression are the ones in the source;
//   * no atomics, no split-K, no reduction whose shape depends on a batch dimension;
//   * every reduction is one of two named orders (ix_tree8, ix_lane_tree) or a plain
//     left-to-right loop.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define IX_OK 0
#define IX_DECLINED 1
#define IX_ERR_ARG (-1)
#define IX_ERR_LAUNCH (-2)
#define IX_ERR_SIZE (-3)

#define IX_DT_F32 0
#define IX_DT_BF16 1

typedef uint16_t bf16_t;

#define IX_WAVE 64
#define IX_LOG2E 1.44269504088896340736f
#define IX_NEG_INF (-__builtin_huge_valf())

__device__ __forceinline__ float ix_bf2f(bf16_t h) { return __uint_as_float(((uint32_t)h) << 16); }

// Round-to-nearest-even fp32 -> bf16, NaN canonicalised to 0x7fc0 (the rule torch's CPU and
// GPU casts use), written with integer ops so the rounding is the same everywhere it is used.
__device__ __forceinline__ bf16_t ix_f2bf(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)0x7fc0;
  u += 0x7fffu + ((u >> 16) & 1u);
  return (bf16_t)(u >> 16);
}
// bf16-round a float and widen it back (the "x.to(bf16).float()" of the eager expressions).
__device__ __forceinline__ float ix_rbf(float f) { return ix_bf2f(ix_f2bf(f)); }

__device__ __forceinline__ uint32_t ix_pack_bf2(float lo, float hi) {
  return (uint32_t)ix_f2bf(lo) | ((uint32_t)ix_f2bf(hi) << 16);
}

// The same rounding by the hardware pack-convert (identical to ix_f2bf on every non-NaN bit pattern; a NaN
// keeps its payload instead of becoming 0x7fc0). For values that cannot be NaN unless the inputs were.
typedef __attribute__((ext_vector_type(2))) __bf16 ix_hw_bf16x2;
typedef __attribute__((ext_vector_type(2))) float ix_hw_f32x2;
__device__ __forceinline__ uint32_t ix_pack_bf2_hw(float lo, float hi) {
  const ix_hw_f32x2 v = {lo, hi};
  const ix_hw_bf16x2 r = __builtin_convertvector(v, ix_hw_bf16x2);
  return *reinterpret_cast<const uint32_t*>(&r);
}

// ix_pack_bf2 bit for bit through the hardware pack-convert: a NaN is first replaced by the quiet NaN whose upper half
// is 0x7fc0, every other pattern rounds the same way. Five instructions for the pair where the integer form takes twelve.
__device__ __forceinline__ float ix_canon_nan(float v) { return v != v ? __uint_as_float(0x7fc00000u) : v; }
__device__ __forceinline__ uint32_t ix_pack_bf2_canon_hw(float lo, float hi) {
  return ix_pack_bf2_hw(ix_canon_nan(lo), ix_canon_nan(hi));
}
// One value through the same instruction (the other half is a constant zero).
__device__ __forceinline__ bf16_t ix_f2bf_hw(float f) { return (bf16_t)(ix_pack_bf2_hw(f, 0.0f) & 0xffffu); }
// bf16-round two floats and widen them back: three instructions for the pair.
__device__ __forceinline__ void ix_rbf2_hw(float a, float b, float& ra, float& rb) {
  const uint32_t u = ix_pack_bf2_hw(a, b);
  ra = __uint_as_float(u << 16);
  rb = __uint_as_float(u & 0xffff0000u);
}

// ---- the transcendental primitives -------------------------------------------------------
// One definition each; every kernel of an op family calls these and nothing else, so prefill
// and decode, M=1 and M=4096, see the same function. ix_prim_unary (ix_prims.hip) exports
// them elementwise so a host-side checker can evaluate the same functions.
__device__ __forceinline__ float ix_exp(float x) { return expf(x); }        // ocml, <=1 ulp
__device__ __forceinline__ float ix_log(float x) { return logf(x); }        // ocml, <=1 ulp
__device__ __forceinline__ float ix_log1p(float x) { return log1pf(x); }    // ocml
// Fast exp for the vocabulary sum: one multiply and one v_exp_f32. Argument is always <= 0.
__device__ __forceinline__ float ix_exp_fast(float x) { return __builtin_amdgcn_exp2f(x * IX_LOG2E); }
// The bare hardware 2^x (about 1 ulp; results below the normal range flush to zero).
__device__ __forceinline__ float ix_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
// IEEE divide and square root (correctly rounded; hipcc's default for fp32), so 1/sqrt is
// reproducible on any IEEE host.
__device__ __forceinline__ float ix_rsqrt_ieee(float x) { return 1.0f / sqrtf(x); }
// Logistic function from the hardware 2^x and reciprocal (about 1 ulp each): 1 / (1 + 2^(-x log2 e)). Five
// instructions where the correctly rounded exp and divide take about forty; within a few fp32 ulp of them.
__device__ __forceinline__ float ix_sigmoid(float x) {
  return __builtin_amdgcn_rcpf(1.0f + ix_exp2((-x) * IX_LOG2E));
}
// SiLU x * sigmoid(x) (ATen's x / (1 + exp(-x)) up to those few ulp).
__device__ __forceinline__ float ix_silu_div(float x) { return x * ix_sigmoid(x); }
// softplus with torch's threshold 20: x > 20 -> x, else log1p(exp(x)).
__device__ __forceinline__ float ix_softplus(float x) { return x > 20.0f ? x : ix_log1p(ix_exp(x)); }

// ---- fixed-order reductions --------------------------------------------------------------
// ix_tree8: ((a0+a1)+(a2+a3))+((a4+a5)+(a6+a7))
__device__ __forceinline__ float ix_tree8(const float (&a)[8]) {
  return ((a[0] + a[1]) + (a[2] + a[3])) + ((a[4] + a[5]) + (a[6] + a[7]));
}
__device__ __forceinline__ float ix_tree8_max(const float (&a)[8]) {
  return fmaxf(fmaxf(fmaxf(a[0], a[1]), fmaxf(a[2], a[3])), fmaxf(fmaxf(a[4], a[5]), fmaxf(a[6], a[7])));
}

// ix_lane_tree<L>: adjacent-pairwise binary tree over L consecutive lanes (L a power of two,
// group aligned to L). Step s adds lane^s; fp add is commutative, so both partners hold the
// same bits after each step and every lane of the group ends with the tree's root:
//   level 1: p[2i]+p[2i+1], level 2: those pairs, ...
// The value held by lane (lane ^ S). Distances below 16 stay inside a row of 16 lanes and use the
// data-parallel-primitive lane controls of the vector ALU (no trip through the LDS crossbar):
//   1, 2: quad permutes; 8: rotate the row by 8; 4: rotate by 12 or by 4, chosen by bit 2 of the lane.
// Larger distances go through the cross-lane permute.
template <int S>
__device__ __forceinline__ float ix_xor_lane(float v) {
  const int x = __float_as_int(v);
  if constexpr (S == 1) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, x, 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
  } else if constexpr (S == 2) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, x, 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
  } else if constexpr (S == 4) {
    const int up = __builtin_amdgcn_update_dpp(0, x, 0x12C, 0xF, 0xF, true);          // row_ror:12 -> lane i reads i+4
    const int dn = __builtin_amdgcn_update_dpp(0, x, 0x124, 0xF, 0xF, true);          // row_ror:4  -> lane i reads i-4
    return __int_as_float((threadIdx.x & 4) ? dn : up);
  } else if constexpr (S == 8) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, x, 0x128, 0xF, 0xF, true));  // row_ror:8
  } else {
    return __shfl_xor(v, S, IX_WAVE);
  }
}
template <int L, int S = 1>
__device__ __forceinline__ float ix_lane_tree(float v) {
  if constexpr (S < L) {
    v = v + ix_xor_lane<S>(v);
    return ix_lane_tree<L, S * 2>(v);
  } else {
    return v;
  }
}
template <int L, int S = 1>
__device__ __forceinline__ float ix_lane_max(float v) {
  if constexpr (S < L) {
    v = fmaxf(v, ix_xor_lane<S>(v));
    return ix_lane_max<L, S * 2>(v);
  } else {
    return v;
  }
}

// ---- 8-element group loads ----------------------------------------------------------------
// Load 8 consecutive elements starting at p, of which the first `valid` (may be <=0 or >=8)
// exist; the others read as `fill`. `vec` says p is 16-byte aligned for bf16 / 32 for fp32.
__device__ __forceinline__ void ix_load8(const bf16_t* __restrict__ p, long valid, bool vec, float fill,
                                         float (&o)[8]) {
  if (vec && valid >= 8) {
    uint4 u = *reinterpret_cast<const uint4*>(p);
    o[0] = __uint_as_float(u.x << 16); o[1] = __uint_as_float(u.x & 0xffff0000u);
    o[2] = __uint_as_float(u.y << 16); o[3] = __uint_as_float(u.y & 0xffff0000u);
    o[4] = __uint_as_float(u.z << 16); o[5] = __uint_as_float(u.z & 0xffff0000u);
    o[6] = __uint_as_float(u.w << 16); o[7] = __uint_as_float(u.w & 0xffff0000u);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = (i < valid) ? ix_bf2f(p[i]) : fill;
  }
}
__device__ __forceinline__ void ix_load8(const float* __restrict__ p, long valid, bool vec, float fill,
                                         float (&o)[8]) {
  if (vec && valid >= 8) {
    float4 a = *reinterpret_cast<const float4*>(p);
    float4 b = *reinterpret_cast<const float4*>(p + 4);
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = (i < valid) ? p[i] : fill;
  }
}

// Eight bf16 held in a 16-byte register group, widened.
__device__ __forceinline__ void ix_unpack8(const uint4 u, float (&o)[8]) {
  const uint32_t q[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    o[2 * c] = __uint_as_float(q[c] << 16);
    o[2 * c + 1] = __uint_as_float(q[c] & 0xffff0000u);
  }
}

__device__ __forceinline__ void ix_store8_bf16(bf16_t* __restrict__ p, long valid, bool vec, const float (&v)[8]) {
  if (vec && valid >= 8) {
    uint4 u;
    u.x = ix_pack_bf2(v[0], v[1]); u.y = ix_pack_bf2(v[2], v[3]);
    u.z = ix_pack_bf2(v[4], v[5]); u.w = ix_pack_bf2(v[6], v[7]);
    *reinterpret_cast<uint4*>(p) = u;
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (i < valid) p[i] = ix_f2bf(v[i]);
  }
}

// Workgroup id -> position in a linear work order, for kernels that stream memory in that order. Hardware deals
// consecutive workgroup ids to the 8 XCDs round-robin; here the order is cut into 8 equal runs and XCD x walks run x,
// so every XCD (its own L2, its own path to memory) streams one contiguous region instead of every eighth piece of
// all of them. Launch ix_xcd_run_grid(total) workgroups; a workgroup past its run's end gets false and exits.
__device__ __forceinline__ bool ix_xcd_run_position(unsigned bid, unsigned total, unsigned* pos) {
  const unsigned xcd = bid & 7u, idx = bid >> 3;
  const unsigned q = total >> 3, r = total & 7u;
  const unsigned lo = q * xcd + ((r * xcd) >> 3), hi = q * (xcd + 1) + ((r * (xcd + 1)) >> 3);
  *pos = lo + idx;
  return lo + idx < hi;
}
static inline unsigned ix_xcd_run_grid(unsigned total) { return 8u * ((total + 7u) / 8u); }

static inline int ix_launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? IX_OK : IX_ERR_LAUNCH;
}
static inline bool ix_aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }
