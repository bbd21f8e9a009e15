// GatedDeltaNet: the gated delta-rule scan, its l2norm/gating preparation and the causal
// depthwise short conv.
//
// Scan (one function for varlen prefill and T=1 decode; reference call sites
// skyrl/backends/skyrl_train/isoexec/ops/gdn/gdn_ops.py:400-441 and :513-558):
//   per (sequence, value head hv), state S [V, K] fp32, for each token t in order
//     S      <- S * exp(g_t)
//     kv[v]   = sum_k S[v,k] * k_t[k]
//     d[v]    = (v_t[v] - kv[v]) * beta_t
//     S[v,k] <- S[v,k] + d[v] * k_t[k]
//     o_t[v]  = sum_k S[v,k] * (q_t[k] * scale)
//   state loaded from pool row idx[n,0], stored to pool row idx[n,t] after token t when that
//   index is > 0; a sequence whose idx[n,0] <= 0 is skipped (its outputs are written as 0).
//
// Each state row S[v,:] evolves independently, so the work is N*HV*V row recurrences. A row is
// owned by KS = K/8 consecutive lanes, lane s holding k = 8s..8s+7 in registers for the whole
// sequence. The two dot products use one fixed order: in-lane, two fused-multiply-add chains
// (even k, odd k) joined by one add; across the KS lanes, the adjacent-pairwise tree. The
// same device function runs for every token of a prefill and for a decode step, and a "chunk"
// is only how many tokens of q/k/v/g/beta are staged per LDS fill, so chunk length, the
// prefill/decode split and batch composition cannot move a bit.
#include "ix_common.h"
#include "../../include/isoexec_hip.h"

__device__ __forceinline__ float ix_ld(const float* p) { return *p; }
__device__ __forceinline__ float ix_ld(const bf16_t* p) { return ix_bf2f(*p); }
__device__ __forceinline__ void ix_st(float* p, float v) { *p = v; }
__device__ __forceinline__ void ix_st(bf16_t* p, float v) { *p = ix_f2bf(v); }

// dot of the lane's 8-element slices: (chain over k = 0,2,4,6) + (chain over k = 1,3,5,7)
__device__ __forceinline__ float ix_dot8(const float (&s)[8], const float (&x)[8]) {
  float pa = s[0] * x[0];
  float pb = s[1] * x[1];
  pa = __builtin_fmaf(s[2], x[2], pa);
  pb = __builtin_fmaf(s[3], x[3], pb);
  pa = __builtin_fmaf(s[4], x[4], pa);
  pb = __builtin_fmaf(s[5], x[5], pb);
  pa = __builtin_fmaf(s[6], x[6], pa);
  pb = __builtin_fmaf(s[7], x[7], pb);
  return pa + pb;
}

// One token of one state-row slice. Returns o (valid in every lane of the row's group).
template <int KS>
__device__ __forceinline__ float ix_gdn_step(float (&S)[8], const float (&kk)[8], const float (&qs)[8], float vv,
                                             float eg, float bt) {
#pragma unroll
  for (int i = 0; i < 8; ++i) S[i] = S[i] * eg;
  const float kv = ix_lane_tree<KS>(ix_dot8(S, kk));
  const float d = (vv - kv) * bt;
#pragma unroll
  for (int i = 0; i < 8; ++i) S[i] = __builtin_fmaf(d, kk[i], S[i]);
  return ix_lane_tree<KS>(ix_dot8(S, qs));
}

// RPL state rows per lane group: lane group r of the workgroup owns rows r, r + 256/KS, ... Each row is
// computed exactly as with RPL = 1 (same lanes per row, same order); holding several rows per lane only
// shares the k/q fetch and gives the scheduler independent chains to interleave.
template <int KS, int RPL, typename TIO>
__global__ __launch_bounds__(256) void k_gdn_scan(const TIO* __restrict__ q, const TIO* __restrict__ k,
                                                  const TIO* __restrict__ v, const float* __restrict__ g,
                                                  const TIO* __restrict__ beta, TIO* __restrict__ o,
                                                  float* __restrict__ state, const int* __restrict__ cu,
                                                  const int* __restrict__ sidx, long sidx_stride, long q_pitch,
                                                  long k_pitch, long v_pitch, int H, int HV, int V, float scale,
                                                  int TT, unsigned xcd_total) {
  constexpr int K = KS * 8;
  constexpr int RW = 256 / KS;   // state rows per pass over the lanes
  constexpr int R = RW * RPL;    // state rows per workgroup
  extern __shared__ __align__(16) char ix_lds[];
  float* kf = reinterpret_cast<float*>(ix_lds);  // [TT][K]
  float* qf = kf + TT * K;                       // [TT][K], pre-scaled
  float* vf = qf + TT * K;                       // [TT][R]
  float* of = vf + TT * R;                       // [TT][R]
  float* egf = of + TT * R;                      // [TT]
  float* btf = egf + TT;                         // [TT]
  int* sif = reinterpret_cast<int*>(btf + TT);   // [TT]

  const int VB = V / R;
  long bid = blockIdx.x;
  {
    unsigned pos;
    if (!ix_xcd_run_position(blockIdx.x, xcd_total, &pos)) return;
    bid = pos;
  }
  const int vb = (int)(bid % VB);
  bid /= VB;
  const int hv = (int)(bid % HV);
  const int n = (int)(bid / HV);
  const int h = hv / (HV / H);
  const int tid = threadIdx.x;
  const int sub = tid % KS, r = tid / KS;
  const int vrow = vb * R + r;  // row of pass 0; pass j adds j * RW

  const int t_begin = cu[n], t_end = cu[n + 1];
  const int len = t_end - t_begin;
  if (len <= 0) return;
  // Stride 0: one row per sequence, loaded at the first token and stored once after the last.
  const long sbase = sidx_stride == 0 ? (long)n : (long)n * sidx_stride;
  const int row0 = sidx[sbase];
  if (row0 <= 0) {  // null lane: no state, outputs defined as zero
    if (!o) return;
    for (int i = tid; i < len * R; i += 256) {
      const int tt = i / R, rr = i % R;
      ix_st(o + ((long)(t_begin + tt) * HV + hv) * V + vb * R + rr, 0.0f);
    }
    return;
  }

  // q and k rows can be fetched 8 elements at a time when every row start is 16/32-byte aligned
  constexpr long AL = 16 * sizeof(TIO) / 2;
  const bool vec_qk = (q_pitch % 8 == 0) && (k_pitch % 8 == 0) && ((uintptr_t)q % AL == 0) && ((uintptr_t)k % AL == 0);
  float S[RPL][8];
#pragma unroll
  for (int j = 0; j < RPL; ++j) {
    const float* sp = state + (((long)row0 * HV + hv) * V + vrow + j * RW) * K + sub * 8;
    const float4 a = *reinterpret_cast<const float4*>(sp);
    const float4 b = *reinterpret_cast<const float4*>(sp + 4);
    S[j][0] = a.x; S[j][1] = a.y; S[j][2] = a.z; S[j][3] = a.w;
    S[j][4] = b.x; S[j][5] = b.y; S[j][6] = b.z; S[j][7] = b.w;
  }

  for (int t0 = 0; t0 < len; t0 += TT) {
    const int nt = min(TT, len - t0);
    __syncthreads();
    if (vec_qk) {  // 8 elements (16 bytes) per load
      for (int i = tid; i < nt * (K / 8); i += 256) {
        const int tt = i / (K / 8), kk = (i % (K / 8)) * 8;
        const long tok = t_begin + t0 + tt;
        float a[8], b[8];
        ix_load8(k + tok * k_pitch + h * K + kk, 8, true, 0.0f, a);
        ix_load8(q + tok * q_pitch + h * K + kk, 8, true, 0.0f, b);
        float* kd = kf + tt * K + kk;
        float* qd = qf + tt * K + kk;
        *reinterpret_cast<float4*>(kd) = make_float4(a[0], a[1], a[2], a[3]);
        *reinterpret_cast<float4*>(kd + 4) = make_float4(a[4], a[5], a[6], a[7]);
        *reinterpret_cast<float4*>(qd) = make_float4(b[0] * scale, b[1] * scale, b[2] * scale, b[3] * scale);
        *reinterpret_cast<float4*>(qd + 4) = make_float4(b[4] * scale, b[5] * scale, b[6] * scale, b[7] * scale);
      }
    } else {
      for (int i = tid; i < nt * K; i += 256) {
        const int tt = i / K, kk = i % K;
        const long tok = t_begin + t0 + tt;
        kf[i] = ix_ld(k + tok * k_pitch + h * K + kk);
        qf[i] = ix_ld(q + tok * q_pitch + h * K + kk) * scale;
      }
    }
    for (int i = tid; i < nt * R; i += 256) {
      const int tt = i / R, rr = i % R;
      vf[i] = ix_ld(v + (long)(t_begin + t0 + tt) * v_pitch + (long)hv * V + vb * R + rr);
    }
    for (int i = tid; i < nt; i += 256) {
      const long src = (long)(t_begin + t0 + i) * HV + hv;
      egf[i] = ix_exp(g[src]);
      btf[i] = ix_ld(beta + src);
      sif[i] = sidx_stride == 0 ? (t0 + i == len - 1 ? row0 : 0) : sidx[sbase + t0 + i];
    }
    __syncthreads();
    auto token = [&](int tt) {
      float kk[8], qs[8];
      {
        const float4 a = *reinterpret_cast<const float4*>(kf + tt * K + sub * 8);
        const float4 b = *reinterpret_cast<const float4*>(kf + tt * K + sub * 8 + 4);
        kk[0] = a.x; kk[1] = a.y; kk[2] = a.z; kk[3] = a.w; kk[4] = b.x; kk[5] = b.y; kk[6] = b.z; kk[7] = b.w;
        const float4 c = *reinterpret_cast<const float4*>(qf + tt * K + sub * 8);
        const float4 d = *reinterpret_cast<const float4*>(qf + tt * K + sub * 8 + 4);
        qs[0] = c.x; qs[1] = c.y; qs[2] = c.z; qs[3] = c.w; qs[4] = d.x; qs[5] = d.y; qs[6] = d.z; qs[7] = d.w;
      }
      const float eg = egf[tt], bt = btf[tt];
      float ov[RPL];
#pragma unroll
      for (int j = 0; j < RPL; ++j) ov[j] = ix_gdn_step<KS>(S[j], kk, qs, vf[tt * R + j * RW + r], eg, bt);
      if (sub == 0) {
#pragma unroll
        for (int j = 0; j < RPL; ++j) of[tt * R + j * RW + r] = ov[j];
      }
    };
    auto store_state = [&](int si) {
#pragma unroll
      for (int j = 0; j < RPL; ++j) {
        float* sp = state + (((long)si * HV + hv) * V + vrow + j * RW) * K + sub * 8;
        *reinterpret_cast<float4*>(sp) = make_float4(S[j][0], S[j][1], S[j][2], S[j][3]);
        *reinterpret_cast<float4*>(sp + 4) = make_float4(S[j][4], S[j][5], S[j][6], S[j][7]);
      }
    };
    if (sidx_stride == 0) {
      // one store, after the sequence's last token: the token loop carries no per-token check
#pragma unroll 4
      for (int tt = 0; tt < nt; ++tt) token(tt);
      if (t0 + nt == len) store_state(row0);
    } else {
      for (int tt = 0; tt < nt; ++tt) {
        token(tt);
        const int si = sif[tt];
        if (si > 0) store_state(si);
      }
    }
    __syncthreads();
    if (o) {
      for (int i = tid; i < nt * R; i += 256) {
        const int tt = i / R, rr = i % R;
        ix_st(o + ((long)(t_begin + t0 + tt) * HV + hv) * V + vb * R + rr, of[i]);
      }
    }
  }
}

// ---- the same scan with a state row held by a PAIR of lanes (K = 128) ---------------------------------------
// Lane l and lane l + 32 of a wave own one state row: the lower one k = 0..63, the upper one k = 64..127, 64
// state floats each. The row's arithmetic is that of k_gdn_scan statement for statement -- per 8-element slice the
// same two multiply-add chains and their join (ix_dot8), the adjacent-pairwise tree over the 16 slice sums, here
// three levels inside the lane (ix_tree8) and the last one across the two halves -- so the two kernels agree bit
// for bit, and which one runs is a staging choice like the time tile. What changes is the cost: 15 of the 16 tree
// adds per dot product no longer cross lanes, and a wave instruction serves 32 rows with 64 elements each instead
// of 4 rows x RPL with 8: about 9.4 instead of 11.3 vector instructions per row and token.
// Compact state form only (one pool row per sequence, stored after the last token).
__device__ __forceinline__ float ix_add_halves(float v) {
  const uint32_t u = __float_as_uint(v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);  // (own half) + (other half) or the reverse: same bits
}

template <typename TIO>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3)))
void k_gdn_scan_pairs(const TIO* __restrict__ q, const TIO* __restrict__ k, const TIO* __restrict__ v,
                      const float* __restrict__ g, const TIO* __restrict__ beta, TIO* __restrict__ o,
                      float* __restrict__ state, const int* __restrict__ cu, const int* __restrict__ sidx,
                      long q_pitch, long k_pitch, long v_pitch, int H, int HV, int V, float scale, int TT,
                      const bf16_t* __restrict__ gate, long gate_stride_t, const bf16_t* __restrict__ norm_w,
                      float norm_eps, int zero_centered) {
  constexpr int K = 128;
  constexpr int R = 128;  // state rows per workgroup: 4 waves x 32 rows
  extern __shared__ __align__(16) char ix_lds[];
  float* kf = reinterpret_cast<float*>(ix_lds);  // [TT][K]
  float* qf = kf + TT * K;                       // [TT][K], pre-scaled
  float* vf = qf + TT * K;                       // [TT][R]
  float* of = vf + TT * R;                       // [TT][R]
  float* egf = of + TT * R;                      // [TT]
  float* btf = egf + TT;                         // [TT]

  const int VB = V / R;
  long bid = blockIdx.x;
  const int vb = (int)(bid % VB);
  bid /= VB;
  const int hv = (int)(bid % HV);
  const int n = (int)(bid / HV);
  const int h = hv / (HV / H);
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int hf = lane >> 5;
  const int r = wave * 32 + (lane & 31);
  const int vrow = vb * R + r;

  const int t_begin = cu[n], t_end = cu[n + 1];
  const int len = t_end - t_begin;
  if (len <= 0) return;
  const int row0 = sidx[n];
  // What leaves for the nt tokens of the tile at t0 whose outputs stand in `of`: the outputs themselves, or, with a gate,
  // the layer's gated output norm of them (ix_gated_out_norm: RMSNorm over the head's V = 128 values, bf16(1 + w),
  // silu(gate)) instead of a launch that reads them back. A token's head is sixteen consecutive threads of eight
  // values, k_rmsnorm_reg<16, 1, 1>'s layout, and the statements are its statements on the bf16 values this kernel
  // would have stored. V == 128 there (one row block per head).
  auto emit = [&](int t0, int nt) __attribute__((always_inline)) {
    if (gate) {
      for (int i0 = 0; i0 < nt * 16; i0 += 256) {
        const int i = i0 + tid;
        const bool live_row = i < nt * 16;
        const int tt = live_row ? i >> 4 : nt - 1, sub = i & 15;  // rows past the tile run the shuffles, never store
        const long tok = t_begin + t0 + tt;
        // The roundings inside the chain are the hardware pack-convert's (ix_rbf2_hw): it differs from ix_rbf on NaNs
        // only, a NaN stays a NaN through every operation below whatever its payload, and the values that are stored
        // get their NaNs made canonical (ix_pack_bf2_canon_hw) -- the stored bits are the ix_rbf chain's. This kernel
        // is bound by vector issue, so the twenty-odd instructions less per value are time.
        float xv[8], wv[8], gv[8], acc[8];
        uint32_t op[4];
        ix_unpack8(*reinterpret_cast<const uint4*>(gate + tok * gate_stride_t + (long)hv * V + sub * 8), gv);
        ix_unpack8(*reinterpret_cast<const uint4*>(norm_w + sub * 8), wv);
#pragma unroll
        for (int j = 0; j < 8; j += 2)  // the scan's output is a bf16 tensor
          ix_rbf2_hw(of[tt * R + sub * 8 + j], of[tt * R + sub * 8 + j + 1], xv[j], xv[j + 1]);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float sq = xv[j] * xv[j];
          acc[j] = 0.0f + sq;
        }
        const float ssum = ix_lane_tree<16>(ix_tree8(acc));
        const float ms = ssum / 128.0f;
        const float rstd = ix_rsqrt_ieee(ms + norm_eps);
#pragma unroll
        for (int j = 0; j < 8; j += 2) {
          float nb0, nb1, g0 = wv[j], g1 = wv[j + 1], y0, y1;
          ix_rbf2_hw(xv[j] * rstd, xv[j + 1] * rstd, nb0, nb1);
          if (zero_centered) ix_rbf2_hw(1.0f + wv[j], 1.0f + wv[j + 1], g0, g1);
          ix_rbf2_hw(nb0 * g0, nb1 * g1, y0, y1);
          op[j >> 1] = ix_pack_bf2_canon_hw(y0 * ix_silu_div(gv[j]), y1 * ix_silu_div(gv[j + 1]));
        }
        if (live_row)
          *reinterpret_cast<uint4*>(reinterpret_cast<bf16_t*>(o) + (tok * HV + hv) * V + sub * 8) =
              make_uint4(op[0], op[1], op[2], op[3]);
      }
    } else {
      for (int i = tid; i < nt * R; i += 256) {
        const int tt = i / R, rr = i % R;
        ix_st(o + ((long)(t_begin + t0 + tt) * HV + hv) * V + vb * R + rr, of[i]);
      }
    }
  };
  if (row0 <= 0) {  // null lane: no state, outputs defined as zero (and what the norm makes of zeros)
    if (!o) return;
    for (int i = tid; i < TT * R; i += 256) of[i] = 0.0f;
    __syncthreads();
    for (int t0 = 0; t0 < len; t0 += TT) emit(t0, min(TT, len - t0));
    return;
  }
  constexpr long AL = 16 * sizeof(TIO) / 2;
  const bool vec_qk = (q_pitch % 8 == 0) && (k_pitch % 8 == 0) && ((uintptr_t)q % AL == 0) && ((uintptr_t)k % AL == 0);
  float S[64];
  float* srow = state + (((long)row0 * HV + hv) * V + vrow) * K + 64 * hf;
#pragma unroll
  for (int c = 0; c < 16; ++c) {
    const float4 a = *reinterpret_cast<const float4*>(srow + 4 * c);
    S[4 * c] = a.x; S[4 * c + 1] = a.y; S[4 * c + 2] = a.z; S[4 * c + 3] = a.w;
  }

  for (int t0 = 0; t0 < len; t0 += TT) {
    const int nt = min(TT, len - t0);
    __syncthreads();
    if (vec_qk) {  // 8 elements (16 bytes) per load
      for (int i = tid; i < nt * (K / 8); i += 256) {
        const int tt = i / (K / 8), kk = (i % (K / 8)) * 8;
        const long tok = t_begin + t0 + tt;
        float a[8], b[8];
        ix_load8(k + tok * k_pitch + h * K + kk, 8, true, 0.0f, a);
        ix_load8(q + tok * q_pitch + h * K + kk, 8, true, 0.0f, b);
        float* kd = kf + tt * K + kk;
        float* qd = qf + tt * K + kk;
        *reinterpret_cast<float4*>(kd) = make_float4(a[0], a[1], a[2], a[3]);
        *reinterpret_cast<float4*>(kd + 4) = make_float4(a[4], a[5], a[6], a[7]);
        *reinterpret_cast<float4*>(qd) = make_float4(b[0] * scale, b[1] * scale, b[2] * scale, b[3] * scale);
        *reinterpret_cast<float4*>(qd + 4) = make_float4(b[4] * scale, b[5] * scale, b[6] * scale, b[7] * scale);
      }
    } else {
      for (int i = tid; i < nt * K; i += 256) {
        const int tt = i / K, kk = i % K;
        const long tok = t_begin + t0 + tt;
        kf[i] = ix_ld(k + tok * k_pitch + h * K + kk);
        qf[i] = ix_ld(q + tok * q_pitch + h * K + kk) * scale;
      }
    }
    for (int i = tid; i < nt * R; i += 256) {
      const int tt = i / R, rr = i % R;
      vf[i] = ix_ld(v + (long)(t_begin + t0 + tt) * v_pitch + (long)hv * V + vb * R + rr);
    }
    for (int i = tid; i < nt; i += 256) {
      const long src = (long)(t_begin + t0 + i) * HV + hv;
      egf[i] = ix_exp(g[src]);
      btf[i] = ix_ld(beta + src);
    }
    __syncthreads();
#pragma unroll 2
    for (int tt = 0; tt < nt; ++tt) {
      const float eg = egf[tt], bt = btf[tt], vv = vf[tt * R + r];
      float x[64];  // this half's 64 elements of k, later of q
      const float* kp = kf + tt * K + 64 * hf;
#pragma unroll
      for (int c = 0; c < 16; ++c) {
        const float4 a = *reinterpret_cast<const float4*>(kp + 4 * c);
        x[4 * c] = a.x; x[4 * c + 1] = a.y; x[4 * c + 2] = a.z; x[4 * c + 3] = a.w;
      }
      float part[8];
#pragma unroll
      for (int sl = 0; sl < 8; ++sl) {
        float ss[8], xs[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          S[8 * sl + i] = S[8 * sl + i] * eg;
          ss[i] = S[8 * sl + i];
          xs[i] = x[8 * sl + i];
        }
        part[sl] = ix_dot8(ss, xs);
      }
      const float kv = ix_add_halves(ix_tree8(part));
      const float d = (vv - kv) * bt;
#pragma unroll
      for (int i = 0; i < 64; ++i) S[i] = __builtin_fmaf(d, x[i], S[i]);
      const float* qp = qf + tt * K + 64 * hf;
#pragma unroll
      for (int c = 0; c < 16; ++c) {
        const float4 a = *reinterpret_cast<const float4*>(qp + 4 * c);
        x[4 * c] = a.x; x[4 * c + 1] = a.y; x[4 * c + 2] = a.z; x[4 * c + 3] = a.w;
      }
#pragma unroll
      for (int sl = 0; sl < 8; ++sl) {
        float ss[8], xs[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          ss[i] = S[8 * sl + i];
          xs[i] = x[8 * sl + i];
        }
        part[sl] = ix_dot8(ss, xs);
      }
      const float ov = ix_add_halves(ix_tree8(part));
      if (hf == 0) of[tt * R + r] = ov;
    }
    if (t0 + nt == len) {
#pragma unroll
      for (int c = 0; c < 16; ++c)
        *reinterpret_cast<float4*>(srow + 4 * c) = make_float4(S[4 * c], S[4 * c + 1], S[4 * c + 2], S[4 * c + 3]);
    }
    __syncthreads();
    if (o) emit(t0, nt);
  }
}

static size_t ix_gdn_lds_bytes(int K, int R, int TT) {
  return (size_t)TT * (2 * K + 2 * R + 3) * sizeof(float);
}

template <int KS, int RPL, typename TIO>
static int ix_gdn_scan_launch_rpl(const void* q, const void* k, const void* v, const float* g, const void* beta,
                                  void* o, float* state, const int* cu, const int* sidx, long sidx_stride,
                                  long q_pitch, long k_pitch, long v_pitch, long N, int H, int HV, int V, float scale,
                                  int TT, hipStream_t st) {
  constexpr int R = (256 / KS) * RPL;
  if (V % R != 0) return IX_DECLINED;
  const long grid = N * HV * (V / R);
  if (grid > 0x7fffffffL) return IX_DECLINED;
  const size_t lds = ix_gdn_lds_bytes(KS * 8, R, TT);
  auto kern = k_gdn_scan<KS, RPL, TIO>;
  if (lds > 48 * 1024) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return IX_ERR_LAUNCH;
  }
  // workgroup order = state order in the pool, walked in 8 XCD runs (a decode step streams the pool once:
  // 0.214 -> 0.210 ms at 256 sequences)
  const unsigned xcd_total = (unsigned)grid;
  if (xcd_total > 0x7ffffff0u) return IX_DECLINED;
  hipLaunchKernelGGL(kern, dim3(ix_xcd_run_grid(xcd_total)), dim3(256), lds, st,
                     (const TIO*)q, (const TIO*)k, (const TIO*)v, g, (const TIO*)beta, (TIO*)o, state, cu, sidx,
                     sidx_stride, q_pitch, k_pitch, v_pitch, H, HV, V, scale, TT, xcd_total);
  return ix_launch_status();
}

// Rows per lane group: a staging choice like the time tile (bits 8.. of time_tile force it). More rows per
// workgroup share each k/q fetch and interleave independent chains, but leave fewer workgroups.
template <int KS, typename TIO>
static int ix_gdn_scan_launch(const void* q, const void* k, const void* v, const float* g, const void* beta,
                              void* o, float* state, const int* cu, const int* sidx, long sidx_stride,
                              long q_pitch, long k_pitch, long v_pitch, long N, int H, int HV, int V, float scale,
                              int TT, int rpl, hipStream_t st) {
  constexpr int RW = 256 / KS;
  if (V % RW != 0) return IX_DECLINED;
  const long groups = N * HV * (V / RW);  // workgroups at one row per lane group
  if (rpl <= 0) rpl = (V % (RW * 2) == 0 && groups >= 2 * 1024) ? 2 : 1;  // measured: 4 rows gain nothing over 2
  while (rpl > 1 && V % (RW * rpl) != 0) rpl >>= 1;
#define IX_RPL_CASE(R_)                                                                                          \
  case R_:                                                                                                       \
    return ix_gdn_scan_launch_rpl<KS, R_, TIO>(q, k, v, g, beta, o, state, cu, sidx, sidx_stride, q_pitch, k_pitch, \
                                               v_pitch, N, H, HV, V, scale, TT, st);
  switch (rpl) {
    IX_RPL_CASE(1)
    IX_RPL_CASE(2)
    IX_RPL_CASE(4)
    default:
      return IX_ERR_ARG;
  }
#undef IX_RPL_CASE
}

static int ix_gdn_scan_impl(const void* q, const void* k, const void* v, const float* g, const void* beta, void* o,
                            int io_dtype, long q_pitch, long k_pitch, long v_pitch, float* state_pool,
                            const int* cu_seqlens, const int* state_indices, long state_indices_stride, long N,
                            long H, long HV, long K, long V, float scale, int time_tile, const bf16_t* gate,
                            long gate_stride_t, const bf16_t* norm_w, float norm_eps, int zero_centered, void* stream) {
  if (!q || !k || !v || !g || !beta || !state_pool || !cu_seqlens || !state_indices) return IX_ERR_ARG;
  if (N < 0 || H <= 0 || HV <= 0 || K <= 0 || V <= 0 || HV % H != 0 || state_indices_stride < 0) return IX_ERR_ARG;
  if (q_pitch < H * K || k_pitch < H * K || v_pitch < HV * V) return IX_ERR_ARG;
  if (io_dtype != IX_DT_F32 && io_dtype != IX_DT_BF16) return IX_DECLINED;
  if (N == 0) return IX_OK;
  if (!ix_aligned(state_pool, 16)) return IX_DECLINED;
  const int rpl = time_tile > 0 ? (time_tile >> 8) : 0;
  // default time tile: short tiles keep more workgroups resident when there are many, long tiles
  // amortise the staging when there are few
  int TT = time_tile <= 0 ? 0 : (time_tile & 0xff);
  if (TT <= 0) TT = (N * HV * (V / 16) >= 4096) ? 16 : 64;
  if (TT > 64) TT = 64;
  hipStream_t st = (hipStream_t)stream;
  // The lane-pair layout: compact state form, K = 128, whole groups of 128 rows, and enough workgroups to fill the
  // chip (or forced by rows-per-lane-group code 16 in bits 8.. of time_tile). Same bits as the kernels below. A
  // time tile of 1 says one token per sequence (a decode step): that is a pure stream of the state, which the
  // 16-lane layout does with more waves in flight.
  if (state_indices_stride == 0 && K == 128 && V % 128 == 0 &&
      (rpl == 16 || (rpl == 0 && (time_tile & 0xff) != 1 && N * HV * (V / 128) >= 512))) {
    const long grid = N * HV * (V / 128);
    if (grid > 0x7fffffffL) return IX_DECLINED;
    const int tt = time_tile > 0 && (time_tile & 0xff) > 0 ? TT : 16;
    const size_t lds = ix_gdn_lds_bytes(128, 128, tt);
    if (io_dtype == IX_DT_BF16)
      hipLaunchKernelGGL((k_gdn_scan_pairs<bf16_t>), dim3((unsigned)grid), dim3(256), lds, st, (const bf16_t*)q,
                         (const bf16_t*)k, (const bf16_t*)v, g, (const bf16_t*)beta, (bf16_t*)o, state_pool,
                         cu_seqlens, state_indices, q_pitch, k_pitch, v_pitch, (int)H, (int)HV, (int)V, scale, tt, gate,
                         gate_stride_t, norm_w, norm_eps, zero_centered);
    else
      hipLaunchKernelGGL((k_gdn_scan_pairs<float>), dim3((unsigned)grid), dim3(256), lds, st, (const float*)q,
                         (const float*)k, (const float*)v, g, (const float*)beta, (float*)o, state_pool, cu_seqlens,
                         state_indices, q_pitch, k_pitch, v_pitch, (int)H, (int)HV, (int)V, scale, tt,
                         (const bf16_t*)nullptr, 0L, (const bf16_t*)nullptr, 0.0f, 0);
    return ix_launch_status();
  }
  if (gate) return IX_DECLINED;       // the norm rides on the lane-pair layout only
  if (rpl == 16) return IX_DECLINED;  // the lane-pair layout was asked for and does not apply
#define IX_SCAN_CASE(KSV)                                                                                         \
  if (K == KSV * 8) {                                                                                             \
    if (io_dtype == IX_DT_BF16)                                                                                   \
      return ix_gdn_scan_launch<KSV, bf16_t>(q, k, v, g, beta, o, state_pool, cu_seqlens, state_indices,         \
                                             state_indices_stride, q_pitch, k_pitch, v_pitch, N, (int)H,         \
                                             (int)HV, (int)V, scale, TT, rpl, st);                               \
    return ix_gdn_scan_launch<KSV, float>(q, k, v, g, beta, o, state_pool, cu_seqlens, state_indices,            \
                                          state_indices_stride, q_pitch, k_pitch, v_pitch, N, (int)H, (int)HV,   \
                                          (int)V, scale, TT, rpl, st);                                           \
  }
  IX_SCAN_CASE(4)
  IX_SCAN_CASE(8)
  IX_SCAN_CASE(16)
  IX_SCAN_CASE(32)
#undef IX_SCAN_CASE
  return IX_DECLINED;
}

extern "C" int ix_gdn_scan(const void* q, const void* k, const void* v, const float* g, const void* beta, void* o,
                           int io_dtype, long q_pitch, long k_pitch, long v_pitch, float* state_pool,
                           const int* cu_seqlens, const int* state_indices, long state_indices_stride, long N,
                           long H, long HV, long K, long V, float scale, int time_tile, void* stream) {
  return ix_gdn_scan_impl(q, k, v, g, beta, o, io_dtype, q_pitch, k_pitch, v_pitch, state_pool, cu_seqlens, state_indices,
                          state_indices_stride, N, H, HV, K, V, scale, time_tile, nullptr, 0, nullptr, 0.0f, 0, stream);
}

// ix_gdn_scan whose output leaves through the layer's gated output norm (ix_gated_out_norm with N = V) in the same
// launch: o receives bf16(norm(o_scan) * silu(gate)) instead of o_scan -- the bits of the two calls. Served where the
// lane-pair layout runs (one state row per sequence, K = V = 128, bf16, at least 512 (sequence, head) pairs) with
// 16-byte aligned gate rows and weight; IX_DECLINED otherwise, before anything is launched or the state is touched.
extern "C" int ix_gdn_scan_gated_norm(const void* q, const void* k, const void* v, const float* g, const void* beta,
                                      void* o, long q_pitch, long k_pitch, long v_pitch, float* state_pool,
                                      const int* cu_seqlens, const int* state_indices, long N, long H, long HV, long K,
                                      long V, float scale, int time_tile, const void* gate, long gate_stride_t,
                                      const void* norm_weight, float norm_eps, int zero_centered, void* stream) {
  if (!o || !gate || !norm_weight || gate_stride_t < HV * V) return IX_ERR_ARG;
  if (K != 128 || V != 128 || (gate_stride_t % 8) || !ix_aligned(gate, 16) || !ix_aligned(norm_weight, 16) ||
      !ix_aligned(o, 16) || (time_tile & 0xff) == 1 || (time_tile >> 8) != 0 || N * HV < 512)
    return IX_DECLINED;
  return ix_gdn_scan_impl(q, k, v, g, beta, o, IX_DT_BF16, q_pitch, k_pitch, v_pitch, state_pool, cu_seqlens,
                          state_indices, 0, N, H, HV, K, V, scale, time_tile, (const bf16_t*)gate, gate_stride_t,
                          (const bf16_t*)norm_weight, norm_eps, zero_centered, stream);
}

// ---------------------------------------------------------------------------------------------
// Preparation (gdn_ops.py:173-213 l2norm, :1197-1210 gating; fused form gdn_ops.py:513-558):
//   qn = io(x * (1 / sqrt(sum_k x_k^2 + 1e-6)))   sum: ix_tree8 over a lane's 8 squares, then the
//                                                 adjacent-pairwise tree over the K/8 lanes
//   g    = -exp(A_log[hv]) * softplus(a + dt_bias[hv])        fp32
//   beta = io(sigmoid(b))
template <int KS, typename TIO>
__global__ __launch_bounds__(256) void k_gdn_l2norm(const TIO* __restrict__ x, TIO* __restrict__ y, long rows,
                                                    int H, long x_pitch, float eps) {
  constexpr int K = KS * 8;
  constexpr int RPB = 256 / KS;
  const int sub = threadIdx.x % KS;
  const long row = (long)blockIdx.x * RPB + threadIdx.x / KS;
  const long rrow = row < rows ? row : rows - 1;
  float xv[8], sq[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    xv[i] = ix_ld(x + (rrow / H) * x_pitch + (rrow % H) * K + sub * 8 + i);
    sq[i] = xv[i] * xv[i];
  }
  const float s = ix_lane_tree<KS>(ix_tree8(sq));
  const float rn = ix_rsqrt_ieee(s + eps);
  if (row >= rows) return;
#pragma unroll
  for (int i = 0; i < 8; ++i) ix_st(y + row * K + sub * 8 + i, xv[i] * rn);
}

template <typename TIO>
__global__ __launch_bounds__(256) void k_gdn_gate(const TIO* __restrict__ a, long a_pitch,
                                                  const TIO* __restrict__ b, long b_pitch,
                                                  const float* __restrict__ A_log,
                                                  const float* __restrict__ dt_bias, float* __restrict__ g,
                                                  TIO* __restrict__ beta, long n, int HV, int exp_bf16) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const long t = i / HV;
  const int hv = (int)(i - t * HV);
  const float sp = ix_softplus(ix_ld(a + t * a_pitch + hv) + dt_bias[hv]);
  float ea = ix_exp(A_log[hv]);
  if (exp_bf16) ea = ix_bf2f(ix_f2bf(ea));  // a bf16 parameter's exp() is a bf16 value (the eager form's rounding)
  const float neg_ea = -ea;
  g[i] = neg_ea * sp;
  ix_st(beta + i, ix_sigmoid(ix_ld(b + t * b_pitch + hv)));
}

extern "C" int ix_gdn_l2norm(const void* x, long x_pitch, void* y, int io_dtype, long tokens, long H, long K,
                             float eps, void* stream) {
  if (!x || !y || tokens < 0 || H <= 0 || K <= 0 || x_pitch < H * K) return IX_ERR_ARG;
  const long rows = tokens * H;
  if (io_dtype != IX_DT_F32 && io_dtype != IX_DT_BF16) return IX_DECLINED;
  if (rows == 0) return IX_OK;
  hipStream_t st = (hipStream_t)stream;
#define IX_L2_CASE(KSV)                                                                                          \
  if (K == KSV * 8) {                                                                                            \
    const long grid = (rows + (256 / KSV) - 1) / (256 / KSV);                                                    \
    if (grid > 0x7fffffffL) return IX_DECLINED;                                                                  \
    if (io_dtype == IX_DT_BF16)                                                                                  \
      hipLaunchKernelGGL((k_gdn_l2norm<KSV, bf16_t>), dim3((unsigned)grid), dim3(256), 0, st, (const bf16_t*)x, \
                         (bf16_t*)y, rows, (int)H, x_pitch, eps);                                                \
    else                                                                                                         \
      hipLaunchKernelGGL((k_gdn_l2norm<KSV, float>), dim3((unsigned)grid), dim3(256), 0, st, (const float*)x,   \
                         (float*)y, rows, (int)H, x_pitch, eps);                                                 \
    return ix_launch_status();                                                                                   \
  }
  IX_L2_CASE(4)
  IX_L2_CASE(8)
  IX_L2_CASE(16)
  IX_L2_CASE(32)
#undef IX_L2_CASE
  return IX_DECLINED;
}

extern "C" int ix_gdn_gate(const void* a, long a_pitch, const void* b, long b_pitch, const float* A_log,
                           const float* dt_bias, float* g, void* beta, int io_dtype, long tokens, long HV,
                           int exp_dtype, void* stream) {
  if (!a || !b || !A_log || !dt_bias || !g || !beta || tokens < 0 || HV <= 0 || a_pitch < HV || b_pitch < HV)
    return IX_ERR_ARG;
  if (io_dtype != IX_DT_F32 && io_dtype != IX_DT_BF16) return IX_DECLINED;
  if (exp_dtype != IX_DT_F32 && exp_dtype != IX_DT_BF16) return IX_DECLINED;
  const int exp_bf16 = exp_dtype == IX_DT_BF16;
  const long n = tokens * HV;
  if (n == 0) return IX_OK;
  const long grid = (n + 255) / 256;
  if (grid > 0x7fffffffL) return IX_DECLINED;
  hipStream_t st = (hipStream_t)stream;
  if (io_dtype == IX_DT_BF16)
    hipLaunchKernelGGL((k_gdn_gate<bf16_t>), dim3((unsigned)grid), dim3(256), 0, st, (const bf16_t*)a, a_pitch,
                       (const bf16_t*)b, b_pitch, A_log, dt_bias, g, (bf16_t*)beta, n, (int)HV, exp_bf16);
  else
    hipLaunchKernelGGL((k_gdn_gate<float>), dim3((unsigned)grid), dim3(256), 0, st, (const float*)a, a_pitch,
                       (const float*)b, b_pitch, A_log, dt_bias, g, (float*)beta, n, (int)HV, exp_bf16);
  return ix_launch_status();
}

// ---------------------------------------------------------------------------------------------
// Open-chunk bookkeeping of the boundary (cpr) engine state (gdn_cpr_scatter.py:24-76; eager form
// gdn_cpr_state.py decode): lane n appends this step's prepared k, v, g, beta to the open-chunk buffers of its
// pool row at column pos[row] % C, then pos[row] += 1 (not for row 0, which absorbs padded lanes), and marks the
// row due for a boundary pass when its position has reached a multiple of C. One workgroup per lane; a live row
// appears at most once per step.
template <typename TIO>
__global__ __launch_bounds__(256) void k_gdn_cpr_scatter(const TIO* __restrict__ k, long k_pitch,
                                                         const TIO* __restrict__ v, long v_pitch,
                                                         const float* __restrict__ g, const TIO* __restrict__ beta,
                                                         const int* __restrict__ rows, int64_t* __restrict__ pos,
                                                         TIO* __restrict__ k_buf, TIO* __restrict__ v_buf,
                                                         float* __restrict__ g_buf, TIO* __restrict__ b_buf,
                                                         int* __restrict__ due, int HK, int HVV, int HV, int C) {
  const int n = blockIdx.x;
  const int row = rows[n];
  const int64_t p = pos[row];
  const int col = (int)(p % C);
  __syncthreads();  // every lane has read the position before lane 0 advances it
  const long slot = (long)row * C + col;
  for (int i = threadIdx.x; i < HK; i += 256) k_buf[slot * HK + i] = k[(long)n * k_pitch + i];
  for (int i = threadIdx.x; i < HVV; i += 256) v_buf[slot * HVV + i] = v[(long)n * v_pitch + i];
  for (int i = threadIdx.x; i < HV; i += 256) {
    g_buf[slot * HV + i] = g[(long)n * HV + i];
    b_buf[slot * HV + i] = beta[(long)n * HV + i];
  }
  if (threadIdx.x == 0 && row > 0) {
    pos[row] = p + 1;
    due[row] = ((p + 1) % C == 0) ? row : 0;
  }
}

extern "C" int ix_gdn_cpr_scatter(const void* k, long k_pitch, const void* v, long v_pitch, const float* g,
                                  const void* beta, const int* rows, int64_t* pos, void* k_buf, void* v_buf,
                                  float* g_buf, void* b_buf, int* due, int io_dtype, long N, long H, long K, long HV,
                                  long V, long C, void* stream) {
  if (!k || !v || !g || !beta || !rows || !pos || !k_buf || !v_buf || !g_buf || !b_buf || !due) return IX_ERR_ARG;
  if (N < 0 || H <= 0 || K <= 0 || HV <= 0 || V <= 0 || C <= 0 || k_pitch < H * K || v_pitch < HV * V)
    return IX_ERR_ARG;
  if (io_dtype != IX_DT_F32 && io_dtype != IX_DT_BF16) return IX_DECLINED;
  if (N == 0) return IX_OK;
  if (N > 0x7fffffffL) return IX_DECLINED;
  hipStream_t st = (hipStream_t)stream;
  if (io_dtype == IX_DT_BF16)
    hipLaunchKernelGGL(k_gdn_cpr_scatter<bf16_t>, dim3((unsigned)N), dim3(256), 0, st, (const bf16_t*)k, k_pitch,
                       (const bf16_t*)v, v_pitch, g, (const bf16_t*)beta, rows, pos, (bf16_t*)k_buf, (bf16_t*)v_buf,
                       g_buf, (bf16_t*)b_buf, due, (int)(H * K), (int)(HV * V), (int)HV, (int)C);
  else
    hipLaunchKernelGGL(k_gdn_cpr_scatter<float>, dim3((unsigned)N), dim3(256), 0, st, (const float*)k, k_pitch,
                       (const float*)v, v_pitch, g, (const float*)beta, rows, pos, (float*)k_buf, (float*)v_buf, g_buf,
                       (float*)b_buf, due, (int)(H * K), (int)(HV * V), (int)HV, (int)C);
  return ix_launch_status();
}

// The hand-off after a boundary pass (gdn_cpr_state.py:602-646): for every pool row marked due, the running state
// becomes the snapshot of the fp32 chain (rounded to the wire dtype and widened back), and the mark is cleared.
__global__ __launch_bounds__(256) void k_gdn_cpr_handoff(const float* __restrict__ entry, float* __restrict__ running,
                                                         int* __restrict__ due, long elems, int snap_bf16) {
  const int row = blockIdx.y;
  if (due[row] <= 0) return;
  const long i = ((long)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i < elems) {
    float4 x = *reinterpret_cast<const float4*>(entry + (long)row * elems + i);
    if (snap_bf16) { x.x = ix_rbf(x.x); x.y = ix_rbf(x.y); x.z = ix_rbf(x.z); x.w = ix_rbf(x.w); }
    *reinterpret_cast<float4*>(running + (long)row * elems + i) = x;
  }
}
__global__ __launch_bounds__(256) void k_gdn_cpr_clear_due(int* __restrict__ due, int rows) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < rows) due[i] = 0;
}

extern "C" int ix_gdn_cpr_handoff(const float* entry_state, float* running_state, int* due, long rows, long elems,
                                  int snapshot_dtype, void* stream) {
  if (!entry_state || !running_state || !due || rows < 0 || elems <= 0) return IX_ERR_ARG;
  if (snapshot_dtype != IX_DT_F32 && snapshot_dtype != IX_DT_BF16) return IX_DECLINED;
  if ((elems % 4) || !ix_aligned(entry_state, 16) || !ix_aligned(running_state, 16)) return IX_DECLINED;
  if (rows == 0) return IX_OK;
  const long gx = (elems / 4 + 255) / 256;
  if (rows > 65535 || gx > 0x7fffffffL) return IX_DECLINED;
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(k_gdn_cpr_handoff, dim3((unsigned)gx, (unsigned)rows), dim3(256), 0, st, entry_state,
                     running_state, due, elems, snapshot_dtype == IX_DT_BF16);
  // the marks are cleared by a second launch: every workgroup of the first reads its row's mark
  hipLaunchKernelGGL(k_gdn_cpr_clear_due, dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, st, due, (int)rows);
  return ix_launch_status();
}

// ---------------------------------------------------------------------------------------------
// Slot ids -> state-pool rows for a decode batch in one launch (gdn_cpr_rows.py:29-46, the fused form of
// gdn_recurrent_state.py:271-284): with a map, row = slot2row[clamp(slot, 0, map_n - 1)]; without one (the
// engine's block ids are the rows), row = slot if 0 <= slot < blocks else 0. Optionally the same launch stamps the
// rows' last-use clock (gdn_recurrent_state.py decode: clock += 1; last_used[rows] = clock). One workgroup, so
// every lane reads the clock before lane 0 advances it.
template <typename TS>
__global__ __launch_bounds__(256) void k_gdn_resolve_rows(const TS* __restrict__ slots, long n,
                                                          const int64_t* __restrict__ slot2row, long map_n,
                                                          long blocks, int64_t* __restrict__ rows64,
                                                          int* __restrict__ rows32, int64_t* __restrict__ last_used,
                                                          int64_t* __restrict__ clock) {
  const int64_t stamp = clock ? clock[0] + 1 : 0;
  for (long i = threadIdx.x; i < n; i += 256) {
    int64_t sl = (int64_t)slots[i];
    int64_t r;
    if (slot2row) {
      sl = sl < 0 ? 0 : (sl > map_n - 1 ? map_n - 1 : sl);
      r = slot2row[sl];
    } else {
      r = (sl >= 0 && sl < blocks) ? sl : 0;
    }
    if (rows64) rows64[i] = r;
    rows32[i] = (int)r;
    if (last_used) last_used[r] = stamp;
  }
  __syncthreads();
  if (clock && threadIdx.x == 0) clock[0] = stamp;
}

extern "C" int ix_gdn_resolve_rows(const void* slots, int slots_i64, long n, const int64_t* slot2row, long map_n,
                                   long blocks, int64_t* rows64, int* rows32, int64_t* last_used, int64_t* clock,
                                   void* stream) {
  if (n < 0 || (n > 0 && (!slots || !rows32))) return IX_ERR_ARG;
  if (slot2row ? map_n <= 0 : blocks <= 0) return IX_ERR_ARG;
  if ((last_used == nullptr) != (clock == nullptr)) return IX_ERR_ARG;
  if (n == 0 && !clock) return IX_OK;
  hipStream_t st = (hipStream_t)stream;
  if (slots_i64)
    hipLaunchKernelGGL(k_gdn_resolve_rows<int64_t>, dim3(1), dim3(256), 0, st, (const int64_t*)slots, n, slot2row,
                       map_n, blocks, rows64, rows32, last_used, clock);
  else
    hipLaunchKernelGGL(k_gdn_resolve_rows<int>, dim3(1), dim3(256), 0, st, (const int*)slots, n, slot2row, map_n,
                       blocks, rows64, rows32, last_used, clock);
  return ix_launch_status();
}

// ---------------------------------------------------------------------------------------------
// Causal depthwise conv of width W <= 8 over packed tokens (gdn_ops.py:74-170):
//   acc = 0; for i = 0..W-1: acc = acc + w[d,i] * xp[t+i]   (multiply rounded, add rounded)
//   acc = acc + bias[d]; acc = acc * sigmoid(acc); y = bf16(acc)
// xp = [W-1 previous inputs (oldest first), from the state pool row or zeros] ++ x. A decode
// step is the same kernel with one token per sequence. The final state (the last W-1 inputs)
// is written by a second kernel so an in-place pool row is never read and written in one launch.
__device__ __forceinline__ int ix_seq_of(const int* __restrict__ cu, int N, int t) {
  int lo = 0, hi = N;  // largest n with cu[n] <= t
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cu[mid] <= t) lo = mid; else hi = mid;
  }
  return lo;
}

__device__ __forceinline__ float ix_conv_xp(const bf16_t* __restrict__ x, long x_pitch,
                                            const bf16_t* __restrict__ pool, int srow, int t_begin, int rel, long D,
                                            int d, int W) {
  // rel: position relative to the sequence start; negative -> history slot W-1+rel
  if (rel >= 0) return ix_bf2f(x[(long)(t_begin + rel) * x_pitch + d]);
  if (srow <= 0) return 0.0f;
  return ix_bf2f(pool[((long)srow * D + d) * (W - 1) + (W - 1 + rel)]);
}

__global__ __launch_bounds__(256) void k_gdn_conv(const bf16_t* __restrict__ x, long x_pitch,
                                                  const bf16_t* __restrict__ w,
                                                  const bf16_t* __restrict__ bias, bf16_t* __restrict__ y,
                                                  const bf16_t* __restrict__ pool, const int* __restrict__ cu,
                                                  const int* __restrict__ rows_in, int N, long D, int W,
                                                  int silu, long total) {
  // Two grid dimensions: one dimension may not exceed 2^32 threads, and a packed prefill does.
  const long i = ((long)blockIdx.y * gridDim.x + blockIdx.x) * 256 + threadIdx.x;
  if (i >= total) return;
  const int t = (int)(i / D);
  const int d = (int)(i % D);
  const int n = ix_seq_of(cu, N, t);
  const int t_begin = cu[n];
  const int rel = t - t_begin;
  const int srow = rows_in ? rows_in[n] : 0;
  float acc = 0.0f;
  for (int j = 0; j < W; ++j) {
    const float xv = ix_conv_xp(x, x_pitch, pool, srow, t_begin, rel - (W - 1) + j, D, d, W);
    const float p = ix_bf2f(w[(long)d * W + j]) * xv;
    acc = acc + p;
  }
  if (bias) acc = acc + ix_bf2f(bias[d]);
  if (silu) acc = acc * ix_sigmoid(acc);
  y[i] = ix_f2bf(acc);
}

// Eight consecutive channels of four consecutive tokens per thread: 16-byte loads and stores, and inside a
// sequence each input row is loaded once for the four windows that cover it. Per channel the arithmetic is that
// of k_gdn_conv, statement for statement, so the two kernels agree bit for bit (a NaN keeps its payload here).
template <int W>
__device__ __forceinline__ void ix_conv8_finish(const float (&xv)[W][8], const float (&wv)[8][W], bool has_bias,
                                                const float (&bv)[8], int silu, bf16_t* __restrict__ yrow) {
  uint32_t out[4];
#pragma unroll
  for (int c = 0; c < 8; c += 2) {
    float r2[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      float acc = 0.0f;
#pragma unroll
      for (int j = 0; j < W; ++j) {
        const float p = wv[c + e][j] * xv[j][c + e];
        acc = acc + p;
      }
      if (has_bias) acc = acc + bv[c + e];
      if (silu) acc = acc * ix_sigmoid(acc);
      r2[e] = acc;
    }
    out[c >> 1] = ix_pack_bf2_hw(r2[0], r2[1]);
  }
  *reinterpret_cast<uint4*>(yrow) = make_uint4(out[0], out[1], out[2], out[3]);
}


// The l2norm of a q or k head (K = 128: sixteen lanes of eight channels) on the bf16 values the convolution just
// rounded -- k_gdn_l2norm<16>'s expression on what it would have read back: squares, ix_tree8, the adjacent-pairwise
// tree over the sixteen lanes, one IEEE rsqrt, bf16(x * r). Every lane of the sixteen must be here.
__device__ __forceinline__ void ix_l2norm8_of16(bf16_t* __restrict__ yrow, float eps) {
  float v8[8], sq[8];
  ix_unpack8(*reinterpret_cast<const uint4*>(yrow), v8);
#pragma unroll
  for (int i = 0; i < 8; ++i) sq[i] = v8[i] * v8[i];
  const float ssum = ix_lane_tree<16>(ix_tree8(sq));
  const float rn = ix_rsqrt_ieee(ssum + eps);
  if (ssum < __builtin_inff()) {
    // every value is finite and so is every product: the hardware pack-convert rounds them as ix_f2bf does
    *reinterpret_cast<uint4*>(yrow) =
        make_uint4(ix_pack_bf2_hw(v8[0] * rn, v8[1] * rn), ix_pack_bf2_hw(v8[2] * rn, v8[3] * rn),
                   ix_pack_bf2_hw(v8[4] * rn, v8[5] * rn), ix_pack_bf2_hw(v8[6] * rn, v8[7] * rn));
    return;
  }
  // an infinity or a NaN among the head's values: products can be NaN, which ix_f2bf canonicalises
  __attribute__((aligned(16))) bf16_t out[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) out[i] = ix_f2bf(v8[i] * rn);
  *reinterpret_cast<uint4*>(yrow) = *reinterpret_cast<const uint4*>(out);
}

// NORM: channels below qk_channels are q and k heads of 128 and leave normalised (ix_gdn_conv_l2norm); a head's sixteen
// threads are consecutive and share the token group, so they take the same path through the kernel.
template <int W, int TOK, bool NORM>
__global__ __launch_bounds__(256) void k_gdn_conv8(const bf16_t* __restrict__ x, long x_pitch,
                                                   const bf16_t* __restrict__ w, const bf16_t* __restrict__ bias,
                                                   bf16_t* __restrict__ y, const bf16_t* __restrict__ pool,
                                                   const int* __restrict__ cu, const int* __restrict__ rows_in,
                                                   int N, long D, int silu, int T, long total, long qk_channels,
                                                   float eps, unsigned run_blocks, unsigned run_groups) {
  const long D8 = D >> 3;
  long i;
  if (run_blocks) {
    // Consecutive token groups of one 2048-channel block on one XCD, one after the other: the W - 1 rows a group
    // shares with the group before it are then still in that XCD's L2 (dealt round-robin, neighbouring groups sit
    // on different XCDs and every shared row is fetched twice). The host chose this only for D8 % 256 == 0.
    unsigned pos;
    if (!ix_xcd_run_position(blockIdx.x, run_blocks, &pos)) return;
    i = (long)(pos % run_groups) * D8 + (long)(pos / run_groups) * 256 + threadIdx.x;
  } else {
    i = ((long)blockIdx.y * gridDim.x + blockIdx.x) * 256 + threadIdx.x;
  }
  if (i >= total) return;
  const int t0 = (int)(i / D8) * TOK;
  const int d = (int)(i % D8) * 8;
  float wv[8][W], bv[8];
  {
    // 8 channels x W taps are 8 W consecutive elements (the host checked the alignment): W 16-byte loads
    static_assert(W == 4, "the unpacking below assumes four taps");
    const uint4* wp = reinterpret_cast<const uint4*>(w + (long)d * W);
#pragma unroll
    for (int c2 = 0; c2 < 4; ++c2) {
      float t8[8];
      ix_unpack8(wp[c2], t8);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        wv[2 * c2][j] = t8[j];
        wv[2 * c2 + 1][j] = t8[4 + j];
      }
    }
    // the channels' biases once per thread, not once per output
    if (bias) {
      ix_unpack8(*reinterpret_cast<const uint4*>(bias + d), bv);
    } else {
#pragma unroll
      for (int c = 0; c < 8; ++c) bv[c] = 0.0f;
    }
  }
  const bool has_bias = bias != nullptr;
  const int n0 = ix_seq_of(cu, N, t0);
  const int b0 = cu[n0], e0 = cu[n0 + 1];
  if (t0 - (W - 1) >= b0 && t0 + TOK <= e0) {
    // all TOK windows lie inside one sequence: TOK + W - 1 rows serve TOK outputs
    // the rows stay packed (4 registers each) until a window needs them
    uint4 xr[TOK + W - 1];
#pragma unroll
    for (int r = 0; r < TOK + W - 1; ++r)
      xr[r] = *reinterpret_cast<const uint4*>(x + (long)(t0 - (W - 1) + r) * x_pitch + d);
#pragma unroll
    for (int q = 0; q < TOK; ++q) {
      float xv[W][8];
#pragma unroll
      for (int j = 0; j < W; ++j) ix_unpack8(xr[q + j], xv[j]);
      if constexpr (NORM) {
        __attribute__((aligned(16))) bf16_t yv[8];
        ix_conv8_finish<W>(xv, wv, has_bias, bv, silu, yv);
        if (d < qk_channels) ix_l2norm8_of16(yv, eps);
        *reinterpret_cast<uint4*>(y + (long)(t0 + q) * D + d) = *reinterpret_cast<const uint4*>(yv);
      } else {
        ix_conv8_finish<W>(xv, wv, has_bias, bv, silu, y + (long)(t0 + q) * D + d);
      }
    }
    return;
  }
  for (int q = 0; q < TOK; ++q) {
    const int t = t0 + q;
    if (t >= T) break;
    const int n = ix_seq_of(cu, N, t);
    const int t_begin = cu[n];
    const int rel = t - t_begin;
    const int srow = rows_in ? rows_in[n] : 0;
    float xv[W][8];
#pragma unroll
    for (int j = 0; j < W; ++j) {
      const int r = rel - (W - 1) + j;
      if (r >= 0) {
        ix_unpack8(*reinterpret_cast<const uint4*>(x + (long)(t_begin + r) * x_pitch + d), xv[j]);
      } else {
#pragma unroll
        for (int c = 0; c < 8; ++c)
          xv[j][c] = srow > 0 ? ix_bf2f(pool[((long)srow * D + d + c) * (W - 1) + (W - 1 + r)]) : 0.0f;
      }
    }
    if constexpr (NORM) {
      __attribute__((aligned(16))) bf16_t yv[8];
      ix_conv8_finish<W>(xv, wv, has_bias, bv, silu, yv);
      if (d < qk_channels) ix_l2norm8_of16(yv, eps);
      *reinterpret_cast<uint4*>(y + (long)t * D + d) = *reinterpret_cast<const uint4*>(yv);
    } else {
      ix_conv8_finish<W>(xv, wv, has_bias, bv, silu, y + (long)t * D + d);
    }
  }
}

__global__ __launch_bounds__(256) void k_gdn_conv_state(const bf16_t* __restrict__ x, long x_pitch,
                                                        bf16_t* __restrict__ pool,
                                                        const int* __restrict__ cu,
                                                        const int* __restrict__ rows_in,
                                                        const int* __restrict__ rows_out, int N, long D, int W) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long)N * D) return;
  const int n = (int)(i / D);
  const int d = (int)(i % D);
  const int orow = rows_out[n];
  if (orow <= 0) return;
  const int t_begin = cu[n], len = cu[n + 1] - t_begin;
  const int srow = rows_in ? rows_in[n] : 0;
  bf16_t tmp[8];
  for (int j = 0; j < W - 1; ++j) {
    // new history slot j holds the input at relative position len - (W-1) + j
    const float xv = ix_conv_xp(x, x_pitch, pool, srow, t_begin, len - (W - 1) + j, D, d, W);
    tmp[j] = ix_f2bf(xv);  // exact: the value is a bf16 already
  }
  for (int j = 0; j < W - 1; ++j) pool[((long)orow * D + d) * (W - 1) + j] = tmp[j];
}

static int ix_gdn_conv_impl(const void* x, long x_pitch, const void* weight, const void* bias, void* y,
                            void* conv_pool, const int* cu_seqlens, const int* state_rows_in,
                            const int* state_rows_out, long N, long total_tokens, long D, long W, int silu,
                            long qk_channels, float eps, void* stream) {
  if (!x || !weight || !y || !cu_seqlens || N < 0 || total_tokens < 0 || D <= 0 || x_pitch < D) return IX_ERR_ARG;
  if (W < 1 || W > 8) return IX_DECLINED;
  if ((state_rows_in || state_rows_out) && !conv_pool) return IX_ERR_ARG;
  if (total_tokens > 0x7fffffffL || N > 0x7fffffffL) return IX_DECLINED;
  hipStream_t st = (hipStream_t)stream;
  const long total = total_tokens * D;
  if (total > 0 && N > 0) {
    const bool vec8 = (W == 4) && (D % 8 == 0) && (x_pitch % 8 == 0) && ix_aligned(x, 16) && ix_aligned(y, 16) &&
                      ix_aligned(weight, 16) && (!bias || ix_aligned(bias, 16));
    // Outputs per thread: long sequences amortise the W - 1 rows of history over 16 outputs; short ones (a decode
    // step has one token per sequence) keep one output per thread so the launch stays wide. Every output is
    // computed by the same expression whichever is chosen.
    if (qk_channels > 0 && !vec8) return IX_DECLINED;  // the normalising form is the eight-channel kernel's
    const long avg_len = total_tokens / N;
    // The normalising form stops at 8: with 16 its registers leave two waves per SIMD and the launch takes a quarter
    // longer than the plain one; with 8 it takes the same time (1.17 ms for 163,840 tokens of 8192 channels).
    const int TOK = !vec8 ? 1 : avg_len >= 64 ? (qk_channels > 0 ? 8 : 16) : avg_len >= 8 ? 4 : 1;
    const long work = vec8 ? ((total_tokens + TOK - 1) / TOK) * (D / 8) : total;
    const long blocks = (work + 255) / 256;
    // the XCD-run order for long sequences whose channel count fills whole workgroups
    const bool runs = vec8 && TOK > 1 && (D / 8) % 256 == 0 && blocks < (1L << 30);
    const unsigned run_blocks = runs ? (unsigned)blocks : 0u;
    const unsigned run_groups = runs ? (unsigned)((total_tokens + TOK - 1) / TOK) : 1u;
    const long gx = runs ? (long)ix_xcd_run_grid(run_blocks) : blocks < (1L << 22) ? blocks : (1L << 22);
    const long gy = runs ? 1 : (blocks + gx - 1) / gx;
    if (gy > 65535) return IX_DECLINED;
#define IX_CONV8(TOK_, NORM_)                                                                                       \
  hipLaunchKernelGGL((k_gdn_conv8<4, TOK_, NORM_>), dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, st,             \
                     (const bf16_t*)x, x_pitch, (const bf16_t*)weight, (const bf16_t*)bias, (bf16_t*)y,             \
                     (const bf16_t*)conv_pool, cu_seqlens, state_rows_in, (int)N, D, silu, (int)total_tokens, work, \
                     qk_channels, eps, run_blocks, run_groups)
    if (vec8 && qk_channels > 0) {
      if (TOK == 8) IX_CONV8(8, true);
      else if (TOK == 4) IX_CONV8(4, true);
      else IX_CONV8(1, true);
    } else if (vec8) {
      if (TOK == 16) IX_CONV8(16, false);
      else if (TOK == 4) IX_CONV8(4, false);
      else IX_CONV8(1, false);
    }
#undef IX_CONV8
    else
      hipLaunchKernelGGL(k_gdn_conv, dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, st, (const bf16_t*)x, x_pitch,
                         (const bf16_t*)weight, (const bf16_t*)bias, (bf16_t*)y, (const bf16_t*)conv_pool, cu_seqlens,
                         state_rows_in, (int)N, D, (int)W, silu, total);
  }
  if (state_rows_out && N > 0 && W > 1) {
    const long grid = (N * D + 255) / 256;
    if (grid > 0x7fffffffL) return IX_DECLINED;
    hipLaunchKernelGGL(k_gdn_conv_state, dim3((unsigned)grid), dim3(256), 0, st, (const bf16_t*)x, x_pitch,
                       (bf16_t*)conv_pool, cu_seqlens, state_rows_in, state_rows_out, (int)N, D, (int)W);
  }
  return ix_launch_status();
}

extern "C" int ix_gdn_conv(const void* x, long x_pitch, const void* weight, const void* bias, void* y,
                           void* conv_pool, const int* cu_seqlens, const int* state_rows_in,
                           const int* state_rows_out, long N, long total_tokens, long D, long W, int silu,
                           void* stream) {
  return ix_gdn_conv_impl(x, x_pitch, weight, bias, y, conv_pool, cu_seqlens, state_rows_in, state_rows_out, N,
                          total_tokens, D, W, silu, 0, 0.0f, stream);
}

// ix_gdn_conv with the l2norm of the q and k heads folded into its epilogue: channels [0, qk_channels) of y are heads of
// K = 128 and leave normalised (the bits of ix_gdn_conv followed by ix_gdn_l2norm over those columns), the rest (v) as
// ix_gdn_conv leaves them. Serves the eight-channel form only: W = 4, D and x_pitch multiples of 8, 16-byte aligned
// operands, qk_channels a multiple of 128; bf16.
extern "C" int ix_gdn_conv_l2norm(const void* x, long x_pitch, const void* weight, const void* bias, void* y,
                                  void* conv_pool, const int* cu_seqlens, const int* state_rows_in,
                                  const int* state_rows_out, long N, long total_tokens, long D, long W, int silu,
                                  long qk_channels, long K, float eps, void* stream) {
  if (qk_channels <= 0 || qk_channels > D || K <= 0) return IX_ERR_ARG;
  if (K != 128 || (qk_channels % 128) || (D % 128) || W != 4) return IX_DECLINED;
  return ix_gdn_conv_impl(x, x_pitch, weight, bias, y, conv_pool, cu_seqlens, state_rows_in, state_rows_out, N,
                          total_tokens, D, W, silu, qk_channels, eps, stream);
}

// ---------------------------------------------------------------------------------------------
// Everything a decode step does in front of the scan, in ONE launch (one token per sequence): the width-4 conv on the
// row's stored window with the window slid in place, the l2norm of the q and k heads, the gating. It replaces four
// launches (k_gdn_conv8<4, 1>, k_gdn_conv_state, k_gdn_l2norm<16>, k_gdn_gate: 4 - 8 us each at batch 64, all of it
// launch latency) and computes every value by the same statements:
//   conv    ix_conv8_finish on [h0, h1, h2, x] -> eight packed bf16 (k_gdn_conv8's expression)
//   window  [h1, h2, x] back to the same pool row (k_gdn_conv_state's values; a thread owns its eight channels' window,
//           reads it before it writes it, and nobody else touches it: no second launch is needed when the row a
//           sequence reads is the row it writes)
//   l2norm  on the bf16 values the conv stored, ix_tree8 + ix_lane_tree<16> (k_gdn_l2norm<16>'s expression): a head of
//           128 channels is 16 consecutive threads
//   gate    k_gdn_gate's two expressions, by the first HV threads of the sequence's first workgroup
// Layout: thread = eight consecutive channels of one sequence; workgroup = 2048 channels; grid = (D / 2048, N).
// y [N, D] receives normalised q and k (channels < 2 H K) and the conv's v behind them. A row <= 0 (a padded lane)
// reads a zero window and writes none.
__global__ __launch_bounds__(256) void k_gdn_decode_prep(const bf16_t* __restrict__ x, long x_pitch,
                                                         const bf16_t* __restrict__ a, long a_pitch,
                                                         const bf16_t* __restrict__ b, long b_pitch,
                                                         const bf16_t* __restrict__ w, const bf16_t* __restrict__ bias,
                                                         const float* __restrict__ A_log,
                                                         const float* __restrict__ dt_bias, bf16_t* __restrict__ pool,
                                                         const int* __restrict__ rows, bf16_t* __restrict__ y,
                                                         float* __restrict__ g, bf16_t* __restrict__ beta, long D,
                                                         int qk_channels, int HV, int silu, float eps) {
  constexpr int W = 4;
  const int n = blockIdx.y;
  const int d = (blockIdx.x * 256 + threadIdx.x) * 8;
  const int row = rows[n];
  if (blockIdx.x == 0) {
    for (int hv = threadIdx.x; hv < HV; hv += 256) {
      const float sp = ix_softplus(ix_ld(a + (long)n * a_pitch + hv) + dt_bias[hv]);
      const float neg_ea = -ix_exp(A_log[hv]);
      g[(long)n * HV + hv] = neg_ea * sp;
      ix_st(beta + (long)n * HV + hv, ix_sigmoid(ix_ld(b + (long)n * b_pitch + hv)));
    }
  }
  // whole 16-lane groups leave together (D is a multiple of 128): the lane tree below stays inside live groups
  if (d >= D) return;
  float wv[8][W], bv[8];
  {
    const uint4* wp = reinterpret_cast<const uint4*>(w + (long)d * W);
#pragma unroll
    for (int c2 = 0; c2 < 4; ++c2) {
      float t8[8];
      ix_unpack8(wp[c2], t8);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        wv[2 * c2][j] = t8[j];
        wv[2 * c2 + 1][j] = t8[4 + j];
      }
    }
    if (bias) {
      ix_unpack8(*reinterpret_cast<const uint4*>(bias + d), bv);
    } else {
#pragma unroll
      for (int c = 0; c < 8; ++c) bv[c] = 0.0f;
    }
  }
  // the window of the thread's eight channels: 8 x 3 consecutive bf16 of the pool row
  bf16_t hist[8 * (W - 1)];
  bf16_t* hp = pool + ((long)(row > 0 ? row : 0) * D + d) * (W - 1);
  if (row > 0) {
    const uint4* h4 = reinterpret_cast<const uint4*>(hp);
#pragma unroll
    for (int i = 0; i < 3; ++i) reinterpret_cast<uint4*>(hist)[i] = h4[i];
  } else {
#pragma unroll
    for (int i = 0; i < 8 * (W - 1); ++i) hist[i] = 0;
  }
  const uint4 xin = *reinterpret_cast<const uint4*>(x + (long)n * x_pitch + d);
  float xv[W][8];
#pragma unroll
  for (int c = 0; c < 8; ++c) {
#pragma unroll
    for (int j = 0; j < W - 1; ++j) xv[j][c] = ix_bf2f(hist[c * (W - 1) + j]);
  }
  ix_unpack8(xin, xv[W - 1]);
  __attribute__((aligned(16))) bf16_t yv[8];
  ix_conv8_finish<W>(xv, wv, bias != nullptr, bv, silu, yv);
  if (row > 0) {
    // slide the window: slot j <- slot j + 1, last slot <- this step's input
    __attribute__((aligned(16))) bf16_t nh[8 * (W - 1)];
    const bf16_t* xb = reinterpret_cast<const bf16_t*>(&xin);
#pragma unroll
    for (int c = 0; c < 8; ++c) {
#pragma unroll
      for (int j = 0; j < W - 2; ++j) nh[c * (W - 1) + j] = hist[c * (W - 1) + j + 1];
      nh[c * (W - 1) + W - 2] = xb[c];
    }
    uint4* o4 = reinterpret_cast<uint4*>(hp);
#pragma unroll
    for (int i = 0; i < 3; ++i) o4[i] = reinterpret_cast<const uint4*>(nh)[i];
  }
  bf16_t* yo = y + (long)n * D + d;
  if (d < qk_channels) {
    float v8[8], sq[8];
    ix_unpack8(*reinterpret_cast<const uint4*>(yv), v8);
#pragma unroll
    for (int i = 0; i < 8; ++i) sq[i] = v8[i] * v8[i];
    const float ssum = ix_lane_tree<16>(ix_tree8(sq));
    const float rn = ix_rsqrt_ieee(ssum + eps);
    __attribute__((aligned(16))) bf16_t out[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = ix_f2bf(v8[i] * rn);
    *reinterpret_cast<uint4*>(yo) = *reinterpret_cast<const uint4*>(out);
  } else {
    *reinterpret_cast<uint4*>(yo) = *reinterpret_cast<const uint4*>(yv);
  }
}

extern "C" int ix_gdn_decode_prep(const void* x, long x_pitch, const void* a, long a_pitch, const void* b, long b_pitch,
                                  const void* conv_weight, const void* conv_bias, const float* A_log,
                                  const float* dt_bias, void* conv_pool, const int* rows, void* y, float* g, void* beta,
                                  long N, long H, long K, long HV, long V, long W, int silu, float eps, void* stream) {
  if (!x || !a || !b || !conv_weight || !A_log || !dt_bias || !conv_pool || !rows || !y || !g || !beta) return IX_ERR_ARG;
  if (N < 0 || H <= 0 || K <= 0 || HV <= 0 || V <= 0) return IX_ERR_ARG;
  const long D = 2 * H * K + HV * V;
  if (x_pitch < D || a_pitch < HV || b_pitch < HV) return IX_ERR_ARG;
  // one head = 16 threads of eight channels; 16-byte accesses everywhere
  if (W != 4 || K != 128 || (D % 128) || (x_pitch % 8) || N > 65535) return IX_DECLINED;
  if (!ix_aligned(x, 16) || !ix_aligned(y, 16) || !ix_aligned(conv_weight, 16) || !ix_aligned(conv_pool, 16) ||
      (conv_bias && !ix_aligned(conv_bias, 16)))
    return IX_DECLINED;
  if (N == 0) return IX_OK;
  const long gx = (D / 8 + 255) / 256;
  hipLaunchKernelGGL(k_gdn_decode_prep, dim3((unsigned)gx, (unsigned)N), dim3(256), 0, (hipStream_t)stream,
                     (const bf16_t*)x, x_pitch, (const bf16_t*)a, a_pitch, (const bf16_t*)b, b_pitch,
                     (const bf16_t*)conv_weight, (const bf16_t*)conv_bias, A_log, dt_bias, (bf16_t*)conv_pool, rows,
                     (bf16_t*)y, g, (bf16_t*)beta, D, (int)(2 * H * K), (int)HV, silu, eps);
  return ix_launch_status();
}
