// Zero-centred RMSNorm, the GatedDeltaNet gated output norm and the residual add + norm.
//
// Down-cast chain (skyrl/backends/skyrl_train/isoexec/ops/norms/fused_outnorm.py:16-29,113-232;
// eager form ops/norms/zero_centered_norm.py:36-37 and runtimes/megatron/gdn_fla_shim.py:390-425):
//   s    = sum_j x_j^2 in fp32          rstd = 1 / sqrt(s / N + eps)   (IEEE divide and sqrt)
//   nb   = bf16(x * rstd)
//   gam  = bf16(1 + w)  (zero-centred)   or  w
//   y    = bf16(nb * gam)
//   gated: out = bf16(y * (g / (1 + exp(-g))))   in fp32, one round
//   add : h = bf16(x + r) (fp32 add, one round), then the chain on h; h is also returned.
//
// The reduction order is a function of N alone. A row is owned by LPR = min(64, pow2ceil(N/8))
// consecutive lanes; lane l, slot i holds columns c*LPR*8 + l*8 + i; slot sums run left to right
// over chunks c (multiply rounded, then add rounded: no fused multiply-add), then ix_tree8 over
// the 8 slots, then the adjacent-pairwise lane tree over the LPR lanes. Rows only pick the grid.
#include "ix_common.h"
#include "../../include/isoexec_hip.h"

template <int LPR>
__device__ __forceinline__ float ix_row_sumsq(const bf16_t* __restrict__ xr, const bf16_t* __restrict__ rr,
                                              int N, int sub, bool vec) {
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int off = sub * 8; off < N; off += LPR * 8) {
    float x[8];
    ix_load8(xr + off, N - off, vec, 0.0f, x);
    if (rr) {
      float r[8];
      ix_load8(rr + off, N - off, vec, 0.0f, r);
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] = ix_rbf(x[i] + r[i]);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float sq = x[i] * x[i];
      acc[i] = acc[i] + sq;
    }
  }
  return ix_lane_tree<LPR>(ix_tree8(acc));
}

// MODE 0: plain; 1: gated (gate strided by token); 2: residual add (writes h too).
template <int LPR, int MODE>
__global__ __launch_bounds__(256) void k_rmsnorm(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                 bf16_t* __restrict__ out, long M, int N, float eps,
                                                 int zero_centered, const bf16_t* __restrict__ aux,
                                                 long aux_stride_t, int HV, bf16_t* __restrict__ h_out,
                                                 int vec) {
  constexpr int RPB = 256 / LPR;  // rows per workgroup
  const int tid = threadIdx.x;
  const int sub = tid % LPR;
  const long row = (long)blockIdx.x * RPB + tid / LPR;
  // Lanes of rows past M still run the shuffles (their row pointer is clamped), never store.
  const bool live = row < M;
  const long rrow = live ? row : (M - 1);
  const bf16_t* xr = x + rrow * N;
  const bf16_t* rr = nullptr;
  if (MODE == 2) rr = aux + rrow * N;
  const float s = ix_row_sumsq<LPR>(xr, rr, N, sub, vec != 0);
  const float ms = s / (float)N;
  const float rstd = ix_rsqrt_ieee(ms + eps);
  const bf16_t* gr = nullptr;
  if (MODE == 1) {
    const long t = rrow / HV, hh = rrow % HV;
    gr = aux + t * aux_stride_t + hh * N;
  }
  if (!live) return;
  bf16_t* orow = out + row * N;
  for (int off = sub * 8; off < N; off += LPR * 8) {
    float xv[8], wv[8], o[8];
    ix_load8(xr + off, N - off, vec != 0, 0.0f, xv);
    ix_load8(w + off, N - off, vec != 0, 0.0f, wv);
    if (MODE == 2) {
      float r[8];
      ix_load8(rr + off, N - off, vec != 0, 0.0f, r);
#pragma unroll
      for (int i = 0; i < 8; ++i) xv[i] = ix_rbf(xv[i] + r[i]);
      ix_store8_bf16(h_out + row * N + off, N - off, vec != 0, xv);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float nb = ix_rbf(xv[i] * rstd);
      const float gam = zero_centered ? ix_rbf(1.0f + wv[i]) : wv[i];
      o[i] = ix_rbf(nb * gam);
    }
    if (MODE == 1) {
      float g[8];
      ix_load8(gr + off, N - off, vec != 0 && (aux_stride_t % 8 == 0), 0.0f, g);
#pragma unroll
      for (int i = 0; i < 8; ++i) o[i] = o[i] * ix_silu_div(g[i]);
    }
    ix_store8_bf16(orow + off, N - off, vec != 0, o);
  }
}

// The same chain for a row that fits the registers of its lanes: N = LPR * 8 * NG columns, 16-byte aligned. Every
// operand is fetched once, all loads are issued before the first use, and the sums run in the order of ix_row_sumsq
// (chunks ascending per slot, ix_tree8, lane tree), so the results are those of k_rmsnorm.
template <int LPR, int MODE, int NG>
__global__ __launch_bounds__(256) void k_rmsnorm_reg(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                     bf16_t* __restrict__ out, long M, float eps, int zero_centered,
                                                     const bf16_t* __restrict__ aux, long aux_stride_t, int HV,
                                                     bf16_t* __restrict__ h_out) {
  constexpr int RPB = 256 / LPR, N = LPR * 8 * NG;
  const int tid = threadIdx.x;
  const int sub = tid % LPR;
  const long row = (long)blockIdx.x * RPB + tid / LPR;
  const bool live = row < M;
  const long rrow = live ? row : (M - 1);
  const bf16_t* xr = x + rrow * N + sub * 8;
  uint4 xp[NG], ap[NG], wp[NG];
#pragma unroll
  for (int c = 0; c < NG; ++c) xp[c] = *reinterpret_cast<const uint4*>(xr + c * LPR * 8);
  if (MODE == 2) {
    const bf16_t* rr = aux + rrow * N + sub * 8;
#pragma unroll
    for (int c = 0; c < NG; ++c) ap[c] = *reinterpret_cast<const uint4*>(rr + c * LPR * 8);
  }
  if (MODE == 1) {
    const long t = rrow / HV, hh = rrow % HV;
    const bf16_t* gr = aux + t * aux_stride_t + hh * N + sub * 8;
#pragma unroll
    for (int c = 0; c < NG; ++c) ap[c] = *reinterpret_cast<const uint4*>(gr + c * LPR * 8);
  }
#pragma unroll
  for (int c = 0; c < NG; ++c) wp[c] = *reinterpret_cast<const uint4*>(w + sub * 8 + c * LPR * 8);

  float xv[NG][8];
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int c = 0; c < NG; ++c) {
    ix_unpack8(xp[c], xv[c]);
    if (MODE == 2) {
      float r[8];
      ix_unpack8(ap[c], r);
#pragma unroll
      for (int i = 0; i < 8; ++i) xv[c][i] = ix_rbf(xv[c][i] + r[i]);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float sq = xv[c][i] * xv[c][i];
      acc[i] = acc[i] + sq;
    }
  }
  const float s = ix_lane_tree<LPR>(ix_tree8(acc));
  const float ms = s / (float)N;
  const float rstd = ix_rsqrt_ieee(ms + eps);
  if (!live) return;
  bf16_t* orow = out + row * N + sub * 8;
#pragma unroll
  for (int c = 0; c < NG; ++c) {
    float wv[8], o[8];
    ix_unpack8(wp[c], wv);
    if (MODE == 2) ix_store8_bf16(h_out + row * N + sub * 8 + c * LPR * 8, 8, true, xv[c]);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float nb = ix_rbf(xv[c][i] * rstd);
      const float gam = zero_centered ? ix_rbf(1.0f + wv[i]) : wv[i];
      o[i] = ix_rbf(nb * gam);
    }
    if (MODE == 1) {
      float g[8];
      ix_unpack8(ap[c], g);
#pragma unroll
      for (int i = 0; i < 8; ++i) o[i] = o[i] * ix_silu_div(g[i]);
    }
    ix_store8_bf16(orow + c * LPR * 8, 8, true, o);
  }
}

static int ix_lpr_for(int N) {
  int groups = (N + 7) / 8, l = 1;
  while (l < groups && l < 64) l <<= 1;
  return l;
}

template <int MODE>
static int ix_norm_launch(const bf16_t* x, const bf16_t* w, bf16_t* out, long M, int N, float eps, int zc,
                          const bf16_t* aux, long aux_stride_t, int HV, bf16_t* h_out, hipStream_t st) {
  if (M == 0) return IX_OK;
  const int lpr = ix_lpr_for(N);
  int vec = (N % 8 == 0) && ix_aligned(x, 16) && ix_aligned(w, 16) && ix_aligned(out, 16);
  if (MODE != 0) vec = vec && ix_aligned(aux, 16);
  if (MODE == 2) vec = vec && ix_aligned(h_out, 16);
  const long rpb = 256 / lpr;
  const long grid = (M + rpb - 1) / rpb;
  if (grid > 0x7fffffffL) return IX_DECLINED;
  // rows that fit their lanes' registers (N = lpr * 8 * {1, 2, 4, 8}), all operands 16-byte aligned
  if (vec && (MODE != 1 || aux_stride_t % 8 == 0) && N % (lpr * 8) == 0) {
    const int ng = N / (lpr * 8);
#define IX_NORM_REG(L, G)                                                                                        \
  if (lpr == L && ng == G) {                                                                                     \
    hipLaunchKernelGGL((k_rmsnorm_reg<L, MODE, G>), dim3((unsigned)grid), dim3(256), 0, st, x, w, out, M, eps,   \
                       zc, aux, aux_stride_t, HV, h_out);                                                        \
    return ix_launch_status();                                                                                   \
  }
    IX_NORM_REG(8, 1) IX_NORM_REG(16, 1) IX_NORM_REG(32, 1) IX_NORM_REG(64, 1)
    IX_NORM_REG(64, 2) IX_NORM_REG(64, 4) IX_NORM_REG(64, 8)
#undef IX_NORM_REG
  }
#define IX_NORM_CASE(L)                                                                                          \
  case L:                                                                                                        \
    hipLaunchKernelGGL((k_rmsnorm<L, MODE>), dim3((unsigned)grid), dim3(256), 0, st, x, w, out, M, N, eps, zc,   \
                       aux, aux_stride_t, HV, h_out, vec);                                                       \
    break;
  switch (lpr) {
    IX_NORM_CASE(1) IX_NORM_CASE(2) IX_NORM_CASE(4) IX_NORM_CASE(8) IX_NORM_CASE(16) IX_NORM_CASE(32)
    IX_NORM_CASE(64)
    default: return IX_ERR_ARG;
  }
#undef IX_NORM_CASE
  return ix_launch_status();
}

extern "C" int ix_rmsnorm_gamma(const void* x, const void* weight, void* out, long M, long N, float eps,
                                int zero_centered, void* stream) {
  if (!x || !weight || !out || M < 0 || N <= 0) return IX_ERR_ARG;
  if (N > (1 << 20)) return IX_DECLINED;
  return ix_norm_launch<0>((const bf16_t*)x, (const bf16_t*)weight, (bf16_t*)out, M, (int)N, eps, zero_centered,
                           nullptr, 0, 1, nullptr, (hipStream_t)stream);
}

extern "C" int ix_gated_out_norm(const void* x, const void* gate, long gate_stride_t, const void* weight,
                                 void* out, long T, long HV, long N, float eps, int zero_centered, void* stream) {
  if (!x || !gate || !weight || !out || T < 0 || HV <= 0 || N <= 0) return IX_ERR_ARG;
  if (N > (1 << 20) || HV > (1 << 20)) return IX_DECLINED;
  if (gate_stride_t < HV * N) return IX_ERR_ARG;
  return ix_norm_launch<1>((const bf16_t*)x, (const bf16_t*)weight, (bf16_t*)out, T * HV, (int)N, eps,
                           zero_centered, (const bf16_t*)gate, gate_stride_t, (int)HV, nullptr,
                           (hipStream_t)stream);
}

extern "C" int ix_add_rmsnorm_gamma(const void* x, const void* residual, const void* weight, void* out,
                                    void* h_out, long M, long N, float eps, int zero_centered, void* stream) {
  if (!x || !residual || !weight || !out || !h_out || M < 0 || N <= 0) return IX_ERR_ARG;
  if (N > (1 << 20)) return IX_DECLINED;
  return ix_norm_launch<2>((const bf16_t*)x, (const bf16_t*)weight, (bf16_t*)out, M, (int)N, eps, zero_centered,
                           (const bf16_t*)residual, 0, 1, (bf16_t*)h_out, (hipStream_t)stream);
}

// ---------------------------------------------------------------------------------------------
// The experts' combine, the residual add and the norm in one launch (the tail of every layer: moe_batch_invariant.py:
// 276-320 / moe_combine_kernel.py:36-76, then fused_add_rmsnorm.py:1-25): the token's k expert rows are summed in
// ascending expert order exactly as k_moe_combine sums them (left to right; bf16 adds, or fp32 adds and one round), the
// bf16 result takes the place of x in the residual-add form above. The [T, N] combine output is never written or read
// back. Row layout and reduction order are those of k_rmsnorm_reg<64, 2, NG>, so the results are the two launches'.
template <int NG, int KC>
__global__ __launch_bounds__(256) void k_combine_add_rmsnorm_reg(const bf16_t* __restrict__ expert_out,
                                                                 const int* __restrict__ combine_rows,
                                                                 const bf16_t* __restrict__ residual,
                                                                 const bf16_t* __restrict__ w, bf16_t* __restrict__ out,
                                                                 bf16_t* __restrict__ h_out, long M, float eps,
                                                                 int zero_centered, int fp32_acc) {
  constexpr int LPR = 64, RPB = 256 / LPR, N = LPR * 8 * NG;
  const int tid = threadIdx.x;
  const int sub = tid % LPR;
  const long row = (long)blockIdx.x * RPB + tid / LPR;
  const bool live = row < M;
  const long rrow = live ? row : (M - 1);
  long src[KC];
#pragma unroll
  for (int r = 0; r < KC; ++r) src[r] = combine_rows[rrow * KC + r];
  uint4 ap[NG], wp[NG];
  const bf16_t* rr = residual + rrow * N + sub * 8;
#pragma unroll
  for (int c = 0; c < NG; ++c) ap[c] = *reinterpret_cast<const uint4*>(rr + c * LPR * 8);
#pragma unroll
  for (int c = 0; c < NG; ++c) wp[c] = *reinterpret_cast<const uint4*>(w + sub * 8 + c * LPR * 8);
  float xv[NG][8];
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int c = 0; c < NG; ++c) {
    uint4 ep[KC];
#pragma unroll
    for (int r = 0; r < KC; ++r)
      ep[r] = *reinterpret_cast<const uint4*>(expert_out + src[r] * N + sub * 8 + c * LPR * 8);
    // Roundings inside the chain go through the hardware pack-convert (ix_rbf2_hw), which differs from ix_rbf on NaNs
    // only (it keeps a payload where ix_rbf makes 0x7fc0). A NaN stays a NaN through every add, multiply, divide and
    // square root below whatever its payload, and everything else is the same number either way, so making the NaNs
    // canonical where values are STORED (ix_pack_bf2_canon_hw) leaves every stored bit what the ix_rbf chain stores.
    float sum[8];
    ix_unpack8(ep[0], sum);
#pragma unroll
    for (int r = 1; r < KC; ++r) {
      float e[8];
      ix_unpack8(ep[r], e);
#pragma unroll
      for (int i = 0; i < 8; i += 2) {
        const float t0 = sum[i] + e[i], t1 = sum[i + 1] + e[i + 1];
        if (fp32_acc) {
          sum[i] = t0;
          sum[i + 1] = t1;
        } else {
          ix_rbf2_hw(t0, t1, sum[i], sum[i + 1]);
        }
      }
    }
    float r8[8];
    ix_unpack8(ap[c], r8);
    uint32_t hp[4];
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
      float d0, d1;
      ix_rbf2_hw(sum[i], sum[i + 1], d0, d1);      // what k_moe_combine stores
      const uint32_t u = ix_pack_bf2_canon_hw(d0 + r8[i], d1 + r8[i + 1]);  // h = bf16(x + residual)
      hp[i >> 1] = u;
      xv[c][i] = __uint_as_float(u << 16);
      xv[c][i + 1] = __uint_as_float(u & 0xffff0000u);
    }
    if (live)
      *reinterpret_cast<uint4*>(h_out + row * N + sub * 8 + c * LPR * 8) = make_uint4(hp[0], hp[1], hp[2], hp[3]);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float sq = xv[c][i] * xv[c][i];
      acc[i] = acc[i] + sq;
    }
  }
  const float s = ix_lane_tree<LPR>(ix_tree8(acc));
  const float ms = s / (float)N;
  const float rstd = ix_rsqrt_ieee(ms + eps);
  if (!live) return;
  bf16_t* orow = out + row * N + sub * 8;
#pragma unroll
  for (int c = 0; c < NG; ++c) {
    float wv[8];
    uint32_t op[4];
    ix_unpack8(wp[c], wv);
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
      float nb0, nb1, g0 = wv[i], g1 = wv[i + 1];
      ix_rbf2_hw(xv[c][i] * rstd, xv[c][i + 1] * rstd, nb0, nb1);
      if (zero_centered) ix_rbf2_hw(1.0f + wv[i], 1.0f + wv[i + 1], g0, g1);
      op[i >> 1] = ix_pack_bf2_canon_hw(nb0 * g0, nb1 * g1);
    }
    *reinterpret_cast<uint4*>(orow + c * LPR * 8) = make_uint4(op[0], op[1], op[2], op[3]);
  }
}

extern "C" int ix_moe_combine_add_rmsnorm(const void* expert_out, const int* combine_rows, long k, int fp32_acc,
                                          const void* residual, const void* weight, void* out, void* h_out, long T,
                                          long N, float eps, int zero_centered, void* stream) {
  if (!expert_out || !combine_rows || !residual || !weight || !out || !h_out || T < 0 || N <= 0 || k <= 0)
    return IX_ERR_ARG;
  if (!ix_aligned(expert_out, 16) || !ix_aligned(residual, 16) || !ix_aligned(weight, 16) || !ix_aligned(out, 16) ||
      !ix_aligned(h_out, 16))
    return IX_DECLINED;
  if (T == 0) return IX_OK;
  const long grid = (T + 3) / 4;
  if (grid > 0x7fffffffL) return IX_DECLINED;
  hipStream_t st = (hipStream_t)stream;
#define IX_CAN(NG_, KC_)                                                                                              \
  if (N == 512 * NG_ && k == KC_) {                                                                                   \
    hipLaunchKernelGGL((k_combine_add_rmsnorm_reg<NG_, KC_>), dim3((unsigned)grid), dim3(256), 0, st,                 \
                       (const bf16_t*)expert_out, combine_rows, (const bf16_t*)residual, (const bf16_t*)weight,       \
                       (bf16_t*)out, (bf16_t*)h_out, T, eps, zero_centered, fp32_acc);                                \
    return ix_launch_status();                                                                                        \
  }
  IX_CAN(2, 8) IX_CAN(4, 8) IX_CAN(8, 8) IX_CAN(2, 4) IX_CAN(4, 4) IX_CAN(8, 4) IX_CAN(4, 2) IX_CAN(1, 8) IX_CAN(1, 4)
#undef IX_CAN
  return IX_DECLINED;
}
