// Mixture-of-experts FFN: router top-k, expert-major permutation and block map, grouped
// fc1 + SwiGLU + prob epilogue, grouped fc2, fixed-order combine.
//
// Per-token function (skyrl/backends/skyrl_train/isoexec/ops/moe/moe_router_o2_kernel.py:87-174,369-386,
// moe_batched_experts.py:496-503, moe_batch_invariant.py:276-320, moe_combine_kernel.py:36-76):
//   router : k winners by (score desc, expert index asc); NaN scores count as -inf
//            mode 0: p = softmax over the k winning logits            (top-k then softmax)
//            mode 1: softmax over all E, top-k on the probabilities, renormalise by their sum
//            both sums over the k winners: adjacent-pairwise tree in rank order
//   expert : inter = bf16(x W1^T); gate/up halves; s = bf16(gate / (1 + exp(-gate)));
//            h = bf16(s * up); a = bf16(h * prob); y = bf16(a W2^T)
//   combine: the token's k rows added in ascending expert order; bf16 adds (a round per add)
//            or one fp32 sum and a single round.
// Nothing a token sees depends on the other tokens of the batch: the permutation and the block
// map are integer-only and only decide which workgroup computes a row; the GEMM core's K order
// is fixed (ix_gemm_core.h).
#include "ix_gemm_core.h"
#include "ix_gemm_stream.h"
#include "../../include/isoexec_hip.h"

#define IX_MOE_KMAX 16
#define IX_MOE_EC 8  // experts per lane: E <= 512
#define IX_MOE_TILE_T 256
#define IX_MOE_EMAX 512

// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ bool ix_beats(float av, int ai, float bv, int bi, int sentinel) {
  // does candidate a beat candidate b?  sentinel index = "no candidate"
  if (ai == sentinel) return false;
  if (bi == sentinel) return true;
  return (av > bv) || (av == bv && ai < bi);
}

// One step of the wave-wide "best candidate" exchange at lane distance S (selection by ix_beats is associative
// and commutative, so the exchange network does not matter; distances below 16 use the row-local lane controls).
template <int S>
__device__ __forceinline__ void ix_best_step(float& bv, int& bi, int sentinel) {
  const float ov = ix_xor_lane<S>(bv);
  const int oi = __float_as_int(ix_xor_lane<S>(__int_as_float(bi)));
  if (ix_beats(ov, oi, bv, bi, sentinel)) { bv = ov; bi = oi; }
}

__device__ __forceinline__ float ix_tree_k(float (&t)[IX_MOE_KMAX], int k) {
#pragma unroll
  for (int s = 1; s < IX_MOE_KMAX; s <<= 1) {
    if (s < k) {
#pragma unroll
      for (int i = 0; i < IX_MOE_KMAX; i += 2 * s)
        if (i + s < k) t[i] = t[i] + t[i + s];
    }
  }
  return t[0];
}

// EC = experts held per lane (E <= 64 EC): the instantiation only sets how many slots a lane carries.
template <int EC>
__global__ __launch_bounds__(256) void k_moe_router(const float* __restrict__ logits, long ld, int T, int E, int k,
                                                    int mode, float scaling, int* __restrict__ topk_idx,
                                                    float* __restrict__ topk_prob, float* __restrict__ dense_probs,
                                                    uint8_t* __restrict__ dense_map) {
  const int lane = threadIdx.x & 63;
  const long t = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T) return;
  float s[EC];
  bool live[EC];
#pragma unroll
  for (int c = 0; c < EC; ++c) {
    const int e = lane + 64 * c;
    live[c] = e < E;
    float v = live[c] ? logits[t * ld + e] : IX_NEG_INF;
    if (v != v) v = IX_NEG_INF;
    s[c] = v;
  }
  if (mode == 1) {
    float m = IX_NEG_INF;
#pragma unroll
    for (int c = 0; c < EC; ++c) m = fmaxf(m, s[c]);
    m = ix_lane_max<64>(m);
    float z = 0.0f;
#pragma unroll
    for (int c = 0; c < EC; ++c) {
      s[c] = live[c] ? ix_exp(s[c] - m) : 0.0f;
      z = z + s[c];
    }
    z = ix_lane_tree<64>(z);
#pragma unroll
    for (int c = 0; c < EC; ++c) s[c] = s[c] / z;
  }
  float vals[IX_MOE_KMAX];
  int idxs[IX_MOE_KMAX];
#pragma unroll
  for (int j = 0; j < IX_MOE_KMAX; ++j) {
    vals[j] = 0.0f;
    idxs[j] = 0;
    if (j < k) {
      float bv = 0.0f;
      int bi = E;
#pragma unroll
      for (int c = 0; c < EC; ++c) {
        const int e = lane + 64 * c;
        if (live[c] && ix_beats(s[c], e, bv, bi, E)) { bv = s[c]; bi = e; }
      }
      ix_best_step<1>(bv, bi, E);
      ix_best_step<2>(bv, bi, E);
      ix_best_step<4>(bv, bi, E);
      ix_best_step<8>(bv, bi, E);
      ix_best_step<16>(bv, bi, E);
      ix_best_step<32>(bv, bi, E);
      bi = min(bi, E - 1);
      vals[j] = bv;
      idxs[j] = bi;
#pragma unroll
      for (int c = 0; c < EC; ++c)
        if (lane + 64 * c == bi) live[c] = false;
    }
  }
  float p[IX_MOE_KMAX], tmp[IX_MOE_KMAX];
  if (mode == 0) {
    const float m = vals[0];
#pragma unroll
    for (int j = 0; j < IX_MOE_KMAX; ++j) { p[j] = (j < k) ? ix_exp(vals[j] - m) : 0.0f; tmp[j] = p[j]; }
  } else {
#pragma unroll
    for (int j = 0; j < IX_MOE_KMAX; ++j) { p[j] = (j < k) ? vals[j] : 0.0f; tmp[j] = p[j]; }
  }
  const float den = ix_tree_k(tmp, k);
#pragma unroll
  for (int j = 0; j < IX_MOE_KMAX; ++j) {
    p[j] = p[j] / den;
    if (scaling != 0.0f) p[j] = p[j] * scaling;
  }
#pragma unroll
  for (int j = 0; j < IX_MOE_KMAX; ++j) {
    if (j < k && lane == j) {
      topk_idx[t * k + j] = idxs[j];
      topk_prob[t * k + j] = p[j];
    }
  }
  if (dense_probs || dense_map) {
#pragma unroll
    for (int c = 0; c < EC; ++c) {
      const int e = lane + 64 * c;
      if (e < E) {
        float dp = 0.0f;
        uint8_t dm = 0;
#pragma unroll
        for (int j = 0; j < IX_MOE_KMAX; ++j)
          if (j < k && idxs[j] == e) { dp = p[j]; dm = 1; }
        if (dense_probs) dense_probs[t * E + e] = dp;
        if (dense_map) dense_map[t * E + e] = dm;
      }
    }
  }
}

// E <= 128: a token takes 16 lanes (a row of the wave, so every exchange is a row-local lane control) and a wave
// routes 4 tokens. Lane i of the row holds experts 4i .. 4i+3 and 64+4i .. 64+4i+3. Same function as k_moe_router
// bit for bit: the winner under ix_beats does not depend on the exchange network, and the softmax denominator is
// built as there -- s[v] + s[v + 64] per v = e mod 64, then the adjacent-pairwise tree over v (two levels inside the
// lane, four across the row).
// Token t by the 16 lanes of one row of a wave (li = lane within the row). Called with whole rows only (every lane of
// a row has the same t), so the lane controls below stay inside live lanes.
__device__ __forceinline__ void ix_moe_route_row16(const float* __restrict__ logits, long ld, long t, int li, int E,
                                                   int k, int mode, float scaling, int* __restrict__ topk_idx,
                                                   float* __restrict__ topk_prob, float* __restrict__ dense_probs,
                                                   uint8_t* __restrict__ dense_map, int* __restrict__ lds_idx,
                                                   float* __restrict__ lds_prob) {
  float s[8];
  int eid[8];
  bool live[8];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int e0 = 64 * h + 4 * li;
    float4 v4 = make_float4(IX_NEG_INF, IX_NEG_INF, IX_NEG_INF, IX_NEG_INF);
    if (e0 + 4 <= E && (ld & 3) == 0 && (reinterpret_cast<uintptr_t>(logits) & 15) == 0) {
      v4 = *reinterpret_cast<const float4*>(logits + t * ld + e0);
    } else {
      if (e0 + 0 < E) v4.x = logits[t * ld + e0 + 0];
      if (e0 + 1 < E) v4.y = logits[t * ld + e0 + 1];
      if (e0 + 2 < E) v4.z = logits[t * ld + e0 + 2];
      if (e0 + 3 < E) v4.w = logits[t * ld + e0 + 3];
    }
    const float q[4] = {v4.x, v4.y, v4.z, v4.w};
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int e = e0 + c;
      eid[4 * h + c] = e;
      live[4 * h + c] = e < E;
      float v = live[4 * h + c] ? q[c] : IX_NEG_INF;
      if (v != v) v = IX_NEG_INF;
      s[4 * h + c] = v;
    }
  }
  if (mode == 1) {
    float m = IX_NEG_INF;
#pragma unroll
    for (int c = 0; c < 8; ++c) m = fmaxf(m, s[c]);
    m = ix_lane_max<16>(m);
    float zl[4];
#pragma unroll
    for (int c = 0; c < 8; ++c) s[c] = live[c] ? ix_exp(s[c] - m) : 0.0f;
#pragma unroll
    for (int c = 0; c < 4; ++c) zl[c] = s[c] + s[4 + c];
    float z = (zl[0] + zl[1]) + (zl[2] + zl[3]);
    z = ix_lane_tree<16>(z);
#pragma unroll
    for (int c = 0; c < 8; ++c) s[c] = s[c] / z;
  }
  float vals[IX_MOE_KMAX];
  int idxs[IX_MOE_KMAX];
#pragma unroll
  for (int j = 0; j < IX_MOE_KMAX; ++j) {
    vals[j] = 0.0f;
    idxs[j] = 0;
    if (j < k) {
      float bv = 0.0f;
      int bi = E;
#pragma unroll
      for (int c = 0; c < 8; ++c)
        if (live[c] && ix_beats(s[c], eid[c], bv, bi, E)) { bv = s[c]; bi = eid[c]; }
      ix_best_step<1>(bv, bi, E);
      ix_best_step<2>(bv, bi, E);
      ix_best_step<4>(bv, bi, E);
      ix_best_step<8>(bv, bi, E);
      bi = min(bi, E - 1);
      vals[j] = bv;
      idxs[j] = bi;
#pragma unroll
      for (int c = 0; c < 8; ++c)
        if (eid[c] == bi) live[c] = false;
    }
  }
  float p[IX_MOE_KMAX], tmp[IX_MOE_KMAX];
  if (mode == 0) {
    const float m = vals[0];
#pragma unroll
    for (int j = 0; j < IX_MOE_KMAX; ++j) { p[j] = (j < k) ? ix_exp(vals[j] - m) : 0.0f; tmp[j] = p[j]; }
  } else {
#pragma unroll
    for (int j = 0; j < IX_MOE_KMAX; ++j) { p[j] = (j < k) ? vals[j] : 0.0f; tmp[j] = p[j]; }
  }
  const float den = ix_tree_k(tmp, k);
#pragma unroll
  for (int j = 0; j < IX_MOE_KMAX; ++j) {
    p[j] = p[j] / den;
    if (scaling != 0.0f) p[j] = p[j] * scaling;
  }
#pragma unroll
  for (int j = 0; j < IX_MOE_KMAX; ++j) {
    if (j < k && li == j) {
      topk_idx[t * k + j] = idxs[j];
      topk_prob[t * k + j] = p[j];
      if (lds_idx) {  // a kernel that goes on to permute keeps the winners in LDS as well
        lds_idx[t * k + j] = idxs[j];
        lds_prob[t * k + j] = p[j];
      }
    }
  }
  if (dense_probs || dense_map) {
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const int e = eid[c];
      if (e < E) {
        float dp = 0.0f;
        uint8_t dm = 0;
#pragma unroll
        for (int j = 0; j < IX_MOE_KMAX; ++j)
          if (j < k && idxs[j] == e) { dp = p[j]; dm = 1; }
        if (dense_probs) dense_probs[t * E + e] = dp;
        if (dense_map) dense_map[t * E + e] = dm;
      }
    }
  }
}

__global__ __launch_bounds__(256) void k_moe_router_row16(const float* __restrict__ logits, long ld, int T, int E,
                                                          int k, int mode, float scaling, int* __restrict__ topk_idx,
                                                          float* __restrict__ topk_prob,
                                                          float* __restrict__ dense_probs,
                                                          uint8_t* __restrict__ dense_map) {
  const long t = (long)blockIdx.x * 16 + (threadIdx.x >> 4);
  if (t >= T) return;  // whole rows leave together
  ix_moe_route_row16(logits, ld, t, threadIdx.x & 15, E, k, mode, scaling, topk_idx, topk_prob, dense_probs, dense_map,
                     nullptr, nullptr);
}

extern "C" int ix_moe_router_topk(const float* logits, long ld, long T, long E, long k, int mode, float scaling,
                                  int* topk_idx, float* topk_prob, float* dense_probs, uint8_t* dense_map,
                                  void* stream) {
  if (!logits || !topk_idx || !topk_prob || T < 0 || E <= 0 || k <= 0 || ld < E) return IX_ERR_ARG;
  if (k > E || k > IX_MOE_KMAX || (k & (k - 1)) != 0) return IX_DECLINED;  // pow2 k: padding would re-associate
  if (E > 64 * IX_MOE_EC) return IX_DECLINED;
  if (mode != 0 && mode != 1) return IX_ERR_ARG;
  if (T == 0) return IX_OK;
  const long grid = (T + 3) / 4;
  if (grid > 0x7fffffffL) return IX_DECLINED;
#define IX_ROUTER(EC_)                                                                                            \
  hipLaunchKernelGGL(k_moe_router<EC_>, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, logits, ld,      \
                     (int)T, (int)E, (int)k, mode, scaling, topk_idx, topk_prob, dense_probs, dense_map)
  if (E <= 128) {
    const long grid16 = (T + 15) / 16;
    hipLaunchKernelGGL(k_moe_router_row16, dim3((unsigned)grid16), dim3(256), 0, (hipStream_t)stream, logits, ld,
                       (int)T, (int)E, (int)k, mode, scaling, topk_idx, topk_prob, dense_probs, dense_map);
  } else if (E <= 256) IX_ROUTER(4);
  else IX_ROUTER(IX_MOE_EC);
#undef IX_ROUTER
  return ix_launch_status();
}

// ---------------------------------------------------------------------------------------------
// Permutation (integer only). Token tiles of 256. Per tile and expert, a 256-bit membership mask
// is built in LDS with integer OR (order-free, so the mask is the same in any execution order);
// a row's position inside its expert's segment is then a popcount of the mask below the token,
// which makes every expert's rows token-ascending without any ordered loop or counter.
__device__ __forceinline__ void ix_moe_build_masks(const int* __restrict__ topk_idx, int t0, int nt, int E, int k,
                                                   uint32_t* s_mask /* [E][8] */, int* s_idx /* [256][k] */) {
  for (int i = threadIdx.x; i < E * 8; i += 256) s_mask[i] = 0u;
  for (int i = threadIdx.x; i < nt * k; i += 256) s_idx[i] = topk_idx[(long)t0 * k + i];
  __syncthreads();
  const int t = threadIdx.x;
  if (t < nt) {
    for (int j = 0; j < k; ++j) {
      const int e = s_idx[t * k + j];
      atomicOr(&s_mask[e * 8 + (t >> 5)], 1u << (t & 31));
    }
  }
  __syncthreads();
}

__global__ __launch_bounds__(256) void k_moe_tile_counts(const int* __restrict__ topk_idx, int T, int E, int k,
                                                         int* __restrict__ tile_counts) {
  __shared__ int s_idx[IX_MOE_TILE_T * IX_MOE_KMAX];
  __shared__ uint32_t s_mask[IX_MOE_EMAX * 8];
  const int tile = blockIdx.x;
  const int t0 = tile * IX_MOE_TILE_T;
  const int nt = min(IX_MOE_TILE_T, T - t0);
  ix_moe_build_masks(topk_idx, t0, nt, E, k, s_mask, s_idx);
  for (int e = threadIdx.x; e < E; e += 256) {
    int c = 0;
#pragma unroll
    for (int w = 0; w < 8; ++w) c += __popc(s_mask[e * 8 + w]);
    tile_counts[(long)tile * E + e] = c;
  }
}

// Per expert, the running sum of its counts over the token tiles (tile_base[t][e] = rows of expert e in tiles before t)
// and its total. One wave per expert: a lane owns a run of consecutive tiles, sums it, the lanes' sums are scanned across
// the wave, then the lane walks its run again writing the bases. Integer only.
__global__ __launch_bounds__(256) void k_moe_tile_prefix(const int* __restrict__ tile_counts, int ntiles, int E,
                                                         int* __restrict__ tile_base, int* __restrict__ counts) {
  const int e = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (e >= E) return;  // whole waves leave together
  const int lane = threadIdx.x & 63;
  const int per = (ntiles + 63) >> 6;
  const int t_lo = min(lane * per, ntiles), t_hi = min(t_lo + per, ntiles);
  int mine = 0;
  for (int t = t_lo; t < t_hi; ++t) mine += tile_counts[(long)t * E + e];
  int incl = mine;  // inclusive scan over the lanes
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int up = __shfl_up(incl, d, 64);
    if (lane >= d) incl += up;
  }
  int run = incl - mine;
  for (int t = t_lo; t < t_hi; ++t) {
    const int c = tile_counts[(long)t * E + e];
    tile_base[(long)t * E + e] = run;
    run += c;
  }
  if (lane == 63) counts[e] = incl;
}

// meta layout: [0] = number of m-tiles, then tile_expert[max_tiles], tile_row0[max_tiles],
// tile_nrows[max_tiles]. One workgroup, after k_moe_tile_prefix has left every expert's row count in `counts`: an
// exclusive scan over the experts in LDS, then every expert writes its own row tiles.
__global__ __launch_bounds__(256) void k_moe_offsets(int E, int BM, int max_tiles, const int* __restrict__ counts,
                                                     int* __restrict__ offsets, int* __restrict__ meta) {
  __shared__ int s_cnt[IX_MOE_EMAX], s_off[IX_MOE_EMAX + 1], s_toff[IX_MOE_EMAX + 1];
  const int tid = threadIdx.x;
  for (int e = tid; e < E; e += 256) s_cnt[e] = counts[e];
  __syncthreads();
  // exclusive scan over the experts (rows and row tiles): lane owns experts 2 tid and 2 tid + 1 (E <= 512)
  {
    __shared__ int s_rows[256], s_tiles[256];
    int c[2], tl[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int e = 2 * tid + h;
      c[h] = e < E ? s_cnt[e] : 0;
      tl[h] = (c[h] + BM - 1) / BM;
    }
    s_rows[tid] = c[0] + c[1];
    s_tiles[tid] = tl[0] + tl[1];
    __syncthreads();
    for (int d = 1; d < 256; d <<= 1) {
      const int a = tid >= d ? s_rows[tid - d] : 0;
      const int b = tid >= d ? s_tiles[tid - d] : 0;
      __syncthreads();
      s_rows[tid] += a;
      s_tiles[tid] += b;
      __syncthreads();
    }
    int row0 = s_rows[tid] - (c[0] + c[1]);
    int tile0 = s_tiles[tid] - (tl[0] + tl[1]);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int e = 2 * tid + h;
      if (e < E) { s_off[e] = row0; s_toff[e] = tile0; }
      row0 += c[h];
      tile0 += tl[h];
    }
    if (tid == 255) {
      s_off[E] = s_rows[255];
      s_toff[E] = s_tiles[255];
      offsets[E] = s_rows[255];
      meta[0] = min(s_tiles[255], max_tiles);
    }
  }
  __syncthreads();
  int* tile_expert = meta + 1;
  int* tile_row0 = tile_expert + max_tiles;
  int* tile_nrows = tile_row0 + max_tiles;
  for (int e = tid; e < E; e += 256) {
    const int c = s_cnt[e];
    offsets[e] = s_off[e];
    int nt = s_toff[e];
    for (int r0 = 0; r0 < c && nt < max_tiles; r0 += BM, ++nt) {
      tile_expert[nt] = e;
      tile_row0[nt] = s_off[e] + r0;
      tile_nrows[nt] = min(BM, c - r0);
    }
  }
}

__global__ __launch_bounds__(256) void k_moe_scatter(const int* __restrict__ topk_idx,
                                                     const float* __restrict__ topk_prob, int T, int E, int k,
                                                     const int* __restrict__ tile_base,
                                                     const int* __restrict__ offsets, int* __restrict__ sorted_token,
                                                     float* __restrict__ permuted_prob,
                                                     int* __restrict__ combine_rows) {
  __shared__ int s_idx[IX_MOE_TILE_T * IX_MOE_KMAX];
  __shared__ uint32_t s_mask[IX_MOE_EMAX * 8];
  const int tile = blockIdx.x;
  const int t0 = tile * IX_MOE_TILE_T;
  const int nt = min(IX_MOE_TILE_T, T - t0);
  ix_moe_build_masks(topk_idx, t0, nt, E, k, s_mask, s_idx);
  const int t = threadIdx.x;
  if (t >= nt) return;
  const long tg = t0 + t;
  for (int j = 0; j < k; ++j) {
    const int e = s_idx[t * k + j];
    int local = __popc(s_mask[e * 8 + (t >> 5)] & ((1u << (t & 31)) - 1u));
    for (int w = 0; w < (t >> 5); ++w) local += __popc(s_mask[e * 8 + w]);
    int rank = 0;
    for (int j2 = 0; j2 < k; ++j2) rank += (s_idx[t * k + j2] < e);
    const int pos = offsets[e] + tile_base[(long)tile * E + e] + local;
    sorted_token[pos] = (int)tg;
    permuted_prob[pos] = topk_prob[tg * k + j];
    combine_rows[tg * k + rank] = pos;
  }
}

// The three steps above in one launch for a batch of at most one token tile (a decode step): the membership masks
// stay in LDS, the expert offsets come from a workgroup-wide scan (two experts per lane), and every output is the
// integer the general path writes.
// Body of the one-tile permutation for the first 256 threads of a workgroup (`tid`; threads past 255 of a larger
// workgroup pass through and only meet the barriers). s_idx [T * k] holds the winners already when `idx_in_lds`; the
// routing weights come from `prob_src` (global or LDS). Every thread of the workgroup must call it.
__device__ __forceinline__ void ix_moe_permute_tile_body(const int* __restrict__ topk_idx, const float* prob_src, int T,
                                                         int E, int k, int BM, int max_tiles, int* __restrict__ counts,
                                                         int* __restrict__ offsets, int* __restrict__ sorted_token,
                                                         float* __restrict__ permuted_prob,
                                                         int* __restrict__ combine_rows, int* __restrict__ meta,
                                                         int* s_idx, uint32_t* s_mask, int* s_off, int* s_rows,
                                                         int* s_tiles, bool idx_in_lds) {
  const int tid = threadIdx.x;
  const bool worker = tid < 256;
  if (worker) {
    for (int i = tid; i < E * 8; i += 256) s_mask[i] = 0u;
    if (!idx_in_lds)
      for (int i = tid; i < T * k; i += 256) s_idx[i] = topk_idx[i];
  }
  __syncthreads();
  if (worker && tid < T) {
    for (int j = 0; j < k; ++j) {
      const int e = s_idx[tid * k + j];
      atomicOr(&s_mask[e * 8 + (tid >> 5)], 1u << (tid & 31));
    }
  }
  __syncthreads();
  // lane owns experts 2 tid and 2 tid + 1
  int c[2] = {0, 0}, tl[2] = {0, 0};
  if (worker) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int e = 2 * tid + h;
      if (e < E) {
#pragma unroll
        for (int w = 0; w < 8; ++w) c[h] += __popc(s_mask[e * 8 + w]);
      }
      tl[h] = (c[h] + BM - 1) / BM;
    }
    s_rows[tid] = c[0] + c[1];
    s_tiles[tid] = tl[0] + tl[1];
  }
  __syncthreads();
  for (int d = 1; d < 256; d <<= 1) {  // inclusive scan over the 256 lane sums
    const int a = (worker && tid >= d) ? s_rows[tid - d] : 0;
    const int b = (worker && tid >= d) ? s_tiles[tid - d] : 0;
    __syncthreads();
    if (worker) {
      s_rows[tid] += a;
      s_tiles[tid] += b;
    }
    __syncthreads();
  }
  if (worker) {
    int row0 = s_rows[tid] - (c[0] + c[1]);   // rows before expert 2 tid
    int tile0 = s_tiles[tid] - (tl[0] + tl[1]);
    int* tile_expert = meta + 1;
    int* tile_row0 = tile_expert + max_tiles;
    int* tile_nrows = tile_row0 + max_tiles;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int e = 2 * tid + h;
      if (e < E) {
        s_off[e] = row0;
        counts[e] = c[h];
        offsets[e] = row0;
        int nt = tile0;
        for (int r0 = 0; r0 < c[h] && nt < max_tiles; r0 += BM, ++nt) {
          tile_expert[nt] = e;
          tile_row0[nt] = row0 + r0;
          tile_nrows[nt] = min(BM, c[h] - r0);
        }
      }
      row0 += c[h];
      tile0 += tl[h];
    }
    if (tid == 255) {
      offsets[E] = s_rows[255];
      meta[0] = min(s_tiles[255], max_tiles);
    }
  }
  __syncthreads();
  if (!worker || tid >= T) return;
  for (int j = 0; j < k; ++j) {
    const int e = s_idx[tid * k + j];
    int local = __popc(s_mask[e * 8 + (tid >> 5)] & ((1u << (tid & 31)) - 1u));
    for (int w = 0; w < (tid >> 5); ++w) local += __popc(s_mask[e * 8 + w]);
    int rank = 0;
    for (int j2 = 0; j2 < k; ++j2) rank += (s_idx[tid * k + j2] < e);
    const int pos = s_off[e] + local;
    sorted_token[pos] = tid;
    permuted_prob[pos] = prob_src[(long)tid * k + j];
    combine_rows[(long)tid * k + rank] = pos;
  }
}

__global__ __launch_bounds__(256) void k_moe_permute_one_tile(const int* __restrict__ topk_idx,
                                                              const float* __restrict__ topk_prob, int T, int E,
                                                              int k, int BM, int max_tiles, int* __restrict__ counts,
                                                              int* __restrict__ offsets,
                                                              int* __restrict__ sorted_token,
                                                              float* __restrict__ permuted_prob,
                                                              int* __restrict__ combine_rows, int* __restrict__ meta) {
  __shared__ int s_idx[IX_MOE_TILE_T * IX_MOE_KMAX];
  __shared__ uint32_t s_mask[IX_MOE_EMAX * 8];
  __shared__ int s_off[IX_MOE_EMAX + 1];
  __shared__ int s_rows[256], s_tiles[256];
  ix_moe_permute_tile_body(topk_idx, topk_prob, T, E, k, BM, max_tiles, counts, offsets, sorted_token, permuted_prob,
                           combine_rows, meta, s_idx, s_mask, s_off, s_rows, s_tiles, false);
}

// Router and permutation of a batch of at most one token tile (a decode step) in ONE launch: a workgroup of 1024
// threads routes 64 tokens at a time (16 lanes each, ix_moe_route_row16: the function of k_moe_router_row16), keeps the
// winners in LDS, and goes straight on to the one-tile permutation above. Same integers and same weights as
// ix_moe_router_topk followed by ix_moe_permute; two launches and about ten microseconds of launch latency less.
__global__ __launch_bounds__(1024) void k_moe_route_one_tile(const float* __restrict__ logits, long ld, int T, int E,
                                                             int k, int mode, float scaling, int BM, int max_tiles,
                                                             int* __restrict__ topk_idx, float* __restrict__ topk_prob,
                                                             int* __restrict__ counts, int* __restrict__ offsets,
                                                             int* __restrict__ sorted_token,
                                                             float* __restrict__ permuted_prob,
                                                             int* __restrict__ combine_rows, int* __restrict__ meta) {
  __shared__ int s_idx[IX_MOE_TILE_T * IX_MOE_KMAX];
  __shared__ float s_prob[IX_MOE_TILE_T * IX_MOE_KMAX];
  __shared__ uint32_t s_mask[128 * 8];
  __shared__ int s_off[128 + 1];
  __shared__ int s_rows[256], s_tiles[256];
  for (int t0 = 0; t0 < T; t0 += 64) {
    const int t = t0 + (int)(threadIdx.x >> 4);
    if (t < T)
      ix_moe_route_row16(logits, ld, t, threadIdx.x & 15, E, k, mode, scaling, topk_idx, topk_prob, nullptr, nullptr,
                         s_idx, s_prob);
  }
  // (the body's first barrier publishes s_idx and s_prob)
  ix_moe_permute_tile_body(topk_idx, s_prob, T, E, k, BM, max_tiles, counts, offsets, sorted_token, permuted_prob,
                           combine_rows, meta, s_idx, s_mask, s_off, s_rows, s_tiles, true);
}

// Block map for rows that are ALREADY grouped by expert (the caller holds tokens_per_expert, e.g. a dispatcher's
// output): exclusive scan of the counts, then every expert writes its own row tiles. One workgroup, integer only.
// The counts live on the device, so the host cannot check them against the size of the row buffers: the kernel
// itself keeps every tile inside [0, rows) -- an expert's count is cut to what is left of `rows` after the experts
// before it (counts that add up to more than `rows` lose their tail instead of reaching past the buffers).
template <typename TI>
__global__ __launch_bounds__(256) void k_moe_block_map(const TI* __restrict__ counts_in, int E, int BM, int max_tiles,
                                                       int rows, int* __restrict__ offsets, int* __restrict__ meta) {
  __shared__ int s_rows[256], s_tiles[256];
  const int tid = threadIdx.x;
  int c[2], tl[2];  // lane owns experts 2 tid and 2 tid + 1 (E <= 512)
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int e = 2 * tid + h;
    const long want = e < E ? (long)counts_in[e] : 0;
    c[h] = (int)(want < 0 ? 0 : (want > rows ? rows : want));
  }
  s_rows[tid] = min(c[0] + c[1], rows);  // a partial sum never needs to exceed `rows`: no overflow for any counts
  __syncthreads();
  for (int d = 1; d < 256; d <<= 1) {
    const int a = tid >= d ? s_rows[tid - d] : 0;
    __syncthreads();
    s_rows[tid] = min(s_rows[tid] + a, rows);
    __syncthreads();
  }
  // Saturating adds are associative for non-negative terms: s_rows[tid] = min(rows, sum of the counts up to this lane).
  const int before = tid > 0 ? s_rows[tid - 1] : 0;
  c[0] = min(c[0], rows - before);
  c[1] = min(c[1], rows - before - c[0]);
#pragma unroll
  for (int h = 0; h < 2; ++h) tl[h] = (c[h] + BM - 1) / BM;
  s_tiles[tid] = tl[0] + tl[1];
  __syncthreads();
  for (int d = 1; d < 256; d <<= 1) {
    const int b = tid >= d ? s_tiles[tid - d] : 0;
    __syncthreads();
    s_tiles[tid] += b;
    __syncthreads();
  }
  int row0 = before;
  int tile0 = s_tiles[tid] - (tl[0] + tl[1]);
  int* tile_expert = meta + 1;
  int* tile_row0 = tile_expert + max_tiles;
  int* tile_nrows = tile_row0 + max_tiles;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int e = 2 * tid + h;
    if (e < E) {
      if (offsets) offsets[e] = row0;
      int nt = tile0;
      for (int r0 = 0; r0 < c[h] && nt < max_tiles; r0 += BM, ++nt) {
        tile_expert[nt] = e;
        tile_row0[nt] = row0 + r0;
        tile_nrows[nt] = min(BM, c[h] - r0);
      }
    }
    row0 += c[h];
    tile0 += tl[h];
  }
  if (tid == 255) {
    if (offsets) offsets[E] = s_rows[255];
    meta[0] = min(s_tiles[255], max_tiles);
  }
}

extern "C" int ix_moe_block_map(const void* counts, int counts_i64, long E, long BM, long rows, int* offsets,
                                int* tile_meta, long max_tiles, void* stream) {
  if (!counts || !tile_meta || E <= 0 || BM <= 0 || max_tiles <= 0 || rows < 0) return IX_ERR_ARG;
  if (E > IX_MOE_EMAX || rows > 0x3fffffffL) return IX_DECLINED;  // two clamped counts are added in an int
  hipStream_t st = (hipStream_t)stream;
  if (counts_i64)
    hipLaunchKernelGGL(k_moe_block_map<long>, dim3(1), dim3(256), 0, st, (const long*)counts, (int)E, (int)BM,
                       (int)max_tiles, (int)rows, offsets, tile_meta);
  else
    hipLaunchKernelGGL(k_moe_block_map<int>, dim3(1), dim3(256), 0, st, (const int*)counts, (int)E, (int)BM,
                       (int)max_tiles, (int)rows, offsets, tile_meta);
  return ix_launch_status();
}

extern "C" long ix_moe_max_tiles(long T, long k, long E, long BM) {
  if (T < 0 || k <= 0 || E <= 0 || BM <= 0) return 0;
  return (T * k + BM - 1) / BM + E;
}

extern "C" size_t ix_moe_permute_scratch_ints(long T, long E) {
  if (T < 0 || E <= 0) return 0;
  const long ntiles = (T + IX_MOE_TILE_T - 1) / IX_MOE_TILE_T;
  return (size_t)(2 * ntiles * E);
}

extern "C" int ix_moe_pick_bm(long T, long k, long E) {
  const long avg = (T * k) / (E > 0 ? E : 1);
  return avg >= 96 ? 256 : (avg >= 48 ? 128 : 32);
}

extern "C" int ix_moe_permute(const int* topk_idx, const float* topk_prob, long T, long E, long k, long BM,
                              int* counts, int* offsets, int* sorted_token, float* permuted_prob,
                              int* combine_rows, int* tile_meta, long max_tiles, int* scratch, void* stream) {
  if (!topk_idx || !topk_prob || !counts || !offsets || !sorted_token || !permuted_prob || !combine_rows ||
      !tile_meta || !scratch)
    return IX_ERR_ARG;
  if (T < 0 || E <= 0 || k <= 0 || k > IX_MOE_KMAX || BM <= 0) return IX_ERR_ARG;
  if (E > IX_MOE_EMAX) return IX_DECLINED;
  if (max_tiles < ix_moe_max_tiles(T, k, E, BM)) return IX_ERR_ARG;
  if (T * k > 0x7fffffffL) return IX_DECLINED;
  hipStream_t st = (hipStream_t)stream;
  const long ntiles = (T + IX_MOE_TILE_T - 1) / IX_MOE_TILE_T;
  if (ntiles == 1) {
    hipLaunchKernelGGL(k_moe_permute_one_tile, dim3(1), dim3(256), 0, st, topk_idx, topk_prob, (int)T, (int)E, (int)k,
                       (int)BM, (int)max_tiles, counts, offsets, sorted_token, permuted_prob, combine_rows, tile_meta);
    return ix_launch_status();
  }
  int* tile_counts = scratch;
  int* tile_base = scratch + ntiles * E;
  if (ntiles > 0)
    hipLaunchKernelGGL(k_moe_tile_counts, dim3((unsigned)ntiles), dim3(256), 0, st, topk_idx, (int)T, (int)E, (int)k,
                       tile_counts);
  hipLaunchKernelGGL(k_moe_tile_prefix, dim3((unsigned)((E + 3) / 4)), dim3(256), 0, st, tile_counts, (int)ntiles, (int)E,
                     tile_base, counts);
  hipLaunchKernelGGL(k_moe_offsets, dim3(1), dim3(256), 0, st, (int)E, (int)BM, (int)max_tiles, counts, offsets,
                     tile_meta);
  if (ntiles > 0)
    hipLaunchKernelGGL(k_moe_scatter, dim3((unsigned)ntiles), dim3(256), 0, st, topk_idx, topk_prob, (int)T, (int)E,
                       (int)k, tile_base, offsets, sorted_token, permuted_prob, combine_rows);
  return ix_launch_status();
}

// ix_moe_router_topk + ix_moe_permute for a batch of at most one token tile (T <= 256) and E <= 128, in one launch.
extern "C" int ix_moe_route_one_tile(const float* logits, long ld, long T, long E, long k, int mode, float scaling,
                                     long BM, int* topk_idx, float* topk_prob, int* counts, int* offsets,
                                     int* sorted_token, float* permuted_prob, int* combine_rows, int* tile_meta,
                                     long max_tiles, void* stream) {
  if (!logits || !topk_idx || !topk_prob || !counts || !offsets || !sorted_token || !permuted_prob || !combine_rows ||
      !tile_meta)
    return IX_ERR_ARG;
  if (T < 0 || E <= 0 || k <= 0 || BM <= 0 || ld < E) return IX_ERR_ARG;
  if (mode != 0 && mode != 1) return IX_ERR_ARG;
  if (k > E || k > IX_MOE_KMAX || (k & (k - 1)) != 0) return IX_DECLINED;  // as the router
  if (T > IX_MOE_TILE_T || E > 128) return IX_DECLINED;                    // one token tile, 16 lanes per token
  if (max_tiles < ix_moe_max_tiles(T, k, E, BM)) return IX_ERR_ARG;
  hipLaunchKernelGGL(k_moe_route_one_tile, dim3(1), dim3(1024), 0, (hipStream_t)stream, logits, ld, (int)T, (int)E, (int)k,
                     mode, scaling, (int)BM, (int)max_tiles, topk_idx, topk_prob, counts, offsets, sorted_token,
                     permuted_prob, combine_rows, tile_meta);
  return ix_launch_status();
}

// ---------------------------------------------------------------------------------------------
// The permutation for callers that cannot allocate (code under graph capture, serving loops, harnesses that forbid
// it): the two integer tables ix_moe_permute takes as `scratch` live in a file-scope device array instead. Every GPU
// the library runs on holds its own copy of the array, at its own address, until the process ends; the address is
// resolved once per device, with that device current, on the first call there. Kernels receive that address as an
// argument, exactly as they receive the caller's workspace in ix_moe_permute. Both tables are fully rewritten by
// every call before they are read (k_moe_tile_counts writes [ntiles, E], k_moe_tile_prefix writes the bases), so nothing
// has to start at zero; two calls that overlap on one GPU share the array and race.
#define IX_MOE_STATIC_SCRATCH_INTS (256 * 1024)  // 1 MiB: 2 * ceil(T / 256) * E ints, e.g. 262,144 tokens at E = 128
#define IX_MAX_DEVICES 64
static __device__ __align__(256) int ix_moe_static_scratch[IX_MOE_STATIC_SCRATCH_INTS];
static int* volatile ix_moe_static_scratch_ptr[IX_MAX_DEVICES];  // per device, 0 = not resolved yet

static int ix_moe_static_scratch_for_current_device(int** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= IX_MAX_DEVICES) return IX_ERR_LAUNCH;
  int* p = ix_moe_static_scratch_ptr[dev];
  if (!p) {
    // Two threads resolving at once store the same address: the lookup has no side effect on the array.
    void* sym = nullptr;
    if (hipGetSymbolAddress(&sym, HIP_SYMBOL(ix_moe_static_scratch)) != hipSuccess || !sym) return IX_ERR_LAUNCH;
    p = static_cast<int*>(sym);
    ix_moe_static_scratch_ptr[dev] = p;
  }
  *out = p;
  return IX_OK;
}

extern "C" size_t ix_moe_permute_static_max_ints(void) { return (size_t)IX_MOE_STATIC_SCRATCH_INTS; }

// Set-up call: resolves the array's address on the current device, so that a caller can take the one runtime lookup
// out of the region where it may make no such call (a stream capture). Launches nothing; may be called again.
extern "C" int ix_moe_permute_static_init(void) {
  int* scratch = nullptr;
  return ix_moe_static_scratch_for_current_device(&scratch);
}

extern "C" int ix_moe_permute_static(const int* topk_idx, const float* topk_prob, long T, long E, long k, long BM,
                                     int* counts, int* offsets, int* sorted_token, float* permuted_prob,
                                     int* combine_rows, int* tile_meta, long max_tiles, void* stream) {
  if (T < 0 || E <= 0) return IX_ERR_ARG;
  if (ix_moe_permute_scratch_ints(T, E) > (size_t)IX_MOE_STATIC_SCRATCH_INTS) return IX_ERR_SIZE;
  int* scratch = nullptr;
  const int rc = ix_moe_static_scratch_for_current_device(&scratch);
  if (rc != IX_OK) return rc;
  return ix_moe_permute(topk_idx, topk_prob, T, E, k, BM, counts, offsets, sorted_token, permuted_prob, combine_rows,
                        tile_meta, max_tiles, scratch, stream);
}

// ---------------------------------------------------------------------------------------------
// Grouped GEMMs over the block map. A workgroup past the device-side tile count exits at once,
// so the host never reads the routing back.
//
// Workgroup -> tile: hardware hands consecutive workgroup ids to the 8 XCDs round-robin and each XCD has its own
// L2, so the tile order (row tile major, column tile minor: an expert's tiles are adjacent) is cut into 8 equal
// runs, one per XCD. The ~32 tiles an XCD works on at a time then belong to one or two experts: an expert's
// weights and a row tile's activations go through one L2 once, instead of through all eight.
__device__ __forceinline__ bool ix_moe_tile_of_block(unsigned bid, int n_row_tiles, int nb_n, int* mt, int* nt) {
  const unsigned xcd = bid & 7u;
  const unsigned idx = bid >> 3;
  const unsigned tiles = (unsigned)n_row_tiles * (unsigned)nb_n;  // < 2^31: the launch checks the bound
  const unsigned q = tiles >> 3, r = tiles & 7u;
  const unsigned lo = q * xcd + ((r * xcd) >> 3), hi = q * (xcd + 1) + ((r * (xcd + 1)) >> 3);
  const unsigned l = lo + idx;
  if (l >= hi) return false;
  *mt = (int)(l / (unsigned)nb_n);
  *nt = (int)(l - (unsigned)*mt * (unsigned)nb_n);
  return true;
}

template <int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(WM* WN * 64) void k_moe_fc1_glu(const bf16_t* __restrict__ x, long ldx, int T,
                                                             const int* __restrict__ sorted_token,
                                                             const float* __restrict__ permuted_prob,
                                                             const bf16_t* __restrict__ W1,
                                                             const int* __restrict__ meta, int max_tiles,
                                                             bf16_t* __restrict__ inter, int Hd, int F, int nb_n) {
  using Cfg = IxGemmCfg<BM, BN, WM, WN>;
  static_assert(Cfg::NI % 2 == 0, "a wave must hold gate tiles and their up tiles");
  constexpr int NP = Cfg::NI / 2;  // (gate, up) pairs of 32 columns per wave
  extern __shared__ __align__(16) char ix_lds[];
  int mt, nt;
  if (!ix_moe_tile_of_block(blockIdx.x, meta[0], nb_n, &mt, &nt)) return;
  const int e = meta[1 + mt];
  const long row0 = meta[1 + max_tiles + mt];
  const int nrows = meta[1 + 2 * max_tiles + mt];
  const int n0h = nt * (BN / 2);

  // activations: gathered token rows of x; weights: the expert's [2F, Hd] fc1 matrix with the
  // tile's rows interleaved so that each wave holds NP gate tiles (ni < NP) and their up tiles (ni >= NP):
  // tile row r -> wave r / TN, block b = (r % TN) / 32, half b / NP, column n0h + 32 * NP * wave + 32 * (b % NP) + r % 32.
  const ix_rsrc_t x_rsrc = ix_make_rsrc(x, (uint32_t)(((long)(T - 1) * ldx + Hd) * 2));
  const ix_rsrc_t w_rsrc = ix_make_rsrc(W1 + (long)e * 2 * F * Hd, (uint32_t)((long)2 * F * Hd * 2));
  auto x_row = [&](int r) -> uint32_t {
    return (r < nrows) ? (uint32_t)((long)sorted_token[row0 + r] * ldx * 2) : IX_OOB;
  };
  auto w_row = [&](int r) -> uint32_t {
    const int b = (r % Cfg::TN) >> 5;
    const int col = n0h + (r / Cfg::TN) * (32 * NP) + (b % NP) * 32 + (r & 31);
    return (col < F) ? (uint32_t)(((long)(b / NP) * F + col) * Hd * 2) : IX_OOB;
  };

  ix_f32x16 acc[Cfg::MI][Cfg::NI];
  ix_acc_zero<Cfg>(acc);
  ix_gemm_mainloop<Cfg>(x_rsrc, x_row, w_rsrc, w_row, Hd, ix_lds, acc);

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave / WN, wn = wave % WN;
  // the wave's 32 columns all exist and rows are 16-byte aligned: two half-waves join their column blocks into
  // 16-byte stores (same values, same places)
  // the same for every wave of the workgroup (a barrier depends on it): the whole tile's columns exist
  const bool wide = n0h + BN / 2 <= F && (F % 8 == 0) && (reinterpret_cast<uintptr_t>(inter) % 16 == 0);
  // late zero-fills of the ring by other waves' past-the-end fetches must not land on the store buffers
  if (wide) __syncthreads();
  char* buf = ix_lds + wave * ix_store_block32_lds_bytes<2 * NP>();
  if constexpr (Cfg::MI * Cfg::NI == 16) asm volatile("s_nop 15\n\ts_nop 15");  // matrix pipeline drained before the
                                                                                  // accumulation registers are read by hand
  // bf16(gate), bf16(up) -> s = bf16(silu(gate)) -> h = bf16(s * up) -> bf16(h * prob), two columns at a time so that
  // each rounding is one hardware pack-convert for the pair (round to nearest even; a NaN stays a NaN).
  auto chain2 = [&](float g0, float g1, float u0, float u1, float prob) -> uint32_t {
    float gate0, gate1, up0, up1, s0, s1, h0, h1;
    ix_rbf2_hw(g0, g1, gate0, gate1);
    ix_rbf2_hw(u0, u1, up0, up1);
    ix_rbf2_hw(ix_silu_div(gate0), ix_silu_div(gate1), s0, s1);
    ix_rbf2_hw(s0 * up0, s1 * up1, h0, h1);
    return ix_pack_bf2_hw(h0 * prob, h1 * prob);
  };
  ix_static_for<0, Cfg::MI>([&](auto mic) {
    constexpr int mi = decltype(mic)::value;
    const int r = wm * Cfg::TM + mi * 32 + (lane & 31);
    const bool live = r < nrows;  // the same for the two lanes that share a row
    const long m = row0 + (live ? r : 0);
    const float prob = live ? permuted_prob[m] : 0.0f;
    constexpr bool AG = Cfg::MI * Cfg::NI == 16;
    if (wide) {
      uint4 pieces[2 * NP];
      ix_static_for<0, NP>([&](auto cbc) {
        constexpr int cb = decltype(cbc)::value;  // gate block cb, up block NP + cb
        float g16[16], u16[16];
        ix_acc_read16<AG>(acc[mi][cb], g16);
        ix_acc_read16<AG>(acc[mi][NP + cb], u16);
        auto G = [&](int i) { return g16[i]; };
        auto U = [&](int i) { return u16[i]; };
#pragma unroll
        for (int p = 0; p < 2; ++p) {
          uint2 pk[2];
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const int q = 2 * p + h;
            pk[h].x = chain2(G(q * 4), G(q * 4 + 1), U(q * 4), U(q * 4 + 1), prob);
            pk[h].y = chain2(G(q * 4 + 2), G(q * 4 + 3), U(q * 4 + 2), U(q * 4 + 3), prob);
          }
          pieces[cb * 2 + p] = ix_join_halves(pk[0], pk[1]);
        }
      });
      const int first = wm * Cfg::TM + mi * 32;  // whole rows of the wave's 32 NP columns per store instruction
      ix_store_block32_via_lds<2 * NP>(buf, pieces, inter + (row0 + first) * F + n0h + wn * (32 * NP), F,
                                       min(32, nrows - first));
      return;
    }
    if (!live) return;
    ix_static_for<0, NP>([&](auto cbc) {
      constexpr int cb = decltype(cbc)::value;
      const int c0 = n0h + wn * (32 * NP) + cb * 32;
      auto G = [&](int i) { return ix_acc_read<AG>(acc[mi][cb], i); };
      auto U = [&](int i) { return ix_acc_read<AG>(acc[mi][NP + cb], i); };
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int col = c0 + ix_acc_row(q * 4, lane);
        const int valid = min(4, F - col);
        if (valid <= 0) continue;
        const uint32_t lo = chain2(G(q * 4), G(q * 4 + 1), U(q * 4), U(q * 4 + 1), prob);
        const uint32_t hi = chain2(G(q * 4 + 2), G(q * 4 + 3), U(q * 4 + 2), U(q * 4 + 3), prob);
        bf16_t* dst = inter + m * F + col;
        if (valid >= 4) {
          *reinterpret_cast<uint2*>(dst) = make_uint2(lo, hi);  // col % 4 == 0, F % 8 == 0, inter 16-byte aligned
        } else {
          if (valid > 0) dst[0] = (bf16_t)(lo & 0xffffu);
          if (valid > 1) dst[1] = (bf16_t)(lo >> 16);
          if (valid > 2) dst[2] = (bf16_t)(hi & 0xffffu);
        }
      }
    });
  });
}

template <int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(WM* WN * 64) void k_moe_fc2(const bf16_t* __restrict__ inter,
                                                         const bf16_t* __restrict__ W2,
                                                         const int* __restrict__ meta, int max_tiles,
                                                         bf16_t* __restrict__ out, int Hd, int F, int nb_n) {
  using Cfg = IxGemmCfg<BM, BN, WM, WN>;
  extern __shared__ __align__(16) char ix_lds[];
  int mt, nt;
  if (!ix_moe_tile_of_block(blockIdx.x, meta[0], nb_n, &mt, &nt)) return;
  const int e = meta[1 + mt];
  const long row0 = meta[1 + max_tiles + mt];
  const int nrows = meta[1 + 2 * max_tiles + mt];
  const long n0 = (long)nt * BN;
  const int n_valid = (int)min((long)BN, (long)Hd - n0);

  const ix_rsrc_t x_rsrc = ix_make_rsrc(inter + row0 * F, (uint32_t)((long)nrows * F * 2));
  const ix_rsrc_t w_rsrc = ix_make_rsrc(W2 + ((long)e * Hd + n0) * F, (uint32_t)((long)n_valid * F * 2));
  auto x_row = [&](int r) -> uint32_t { return (r < nrows) ? (uint32_t)(r * F * 2) : IX_OOB; };
  auto w_row = [&](int r) -> uint32_t { return (r < n_valid) ? (uint32_t)(r * F * 2) : IX_OOB; };

  ix_f32x16 acc[Cfg::MI][Cfg::NI];
  ix_acc_zero<Cfg>(acc);
  ix_gemm_mainloop<Cfg>(x_rsrc, x_row, w_rsrc, w_row, F, ix_lds, acc);

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const bool wide = n_valid == BN && (Hd % 8 == 0) && (reinterpret_cast<uintptr_t>(out) % 16 == 0);
  constexpr bool AG = Cfg::MI * Cfg::NI == 16;
  if constexpr (AG) asm volatile("s_nop 15\n\ts_nop 15");
  // late zero-fills of the ring by other waves' past-the-end fetches must not land on the store buffers
  if (wide) __syncthreads();
  constexpr int NPIECE = Cfg::NI * 2;
  char* buf = ix_lds + wave * ix_store_block32_lds_bytes<NPIECE>();
  ix_static_for<0, Cfg::MI>([&](auto mic) {
    constexpr int mi = decltype(mic)::value;
    const int r = wm * Cfg::TM + mi * 32 + (lane & 31);
    const bool live = r < nrows;  // the same for the two lanes that share a row
    const long m = row0 + r;
    if (wide) {
      uint4 pieces[NPIECE];
      ix_static_for<0, Cfg::NI>([&](auto nic) {
        constexpr int ni = decltype(nic)::value;
        float a16[16];
        ix_acc_read16<AG>(acc[mi][ni], a16);
#pragma unroll
        for (int p = 0; p < 2; ++p) {
          uint2 pk[2];
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const int q = 2 * p + h;
            pk[h].x = ix_pack_bf2_hw(a16[q * 4], a16[q * 4 + 1]);
            pk[h].y = ix_pack_bf2_hw(a16[q * 4 + 2], a16[q * 4 + 3]);
          }
          pieces[ni * 2 + p] = ix_join_halves(pk[0], pk[1]);
        }
      });
      const int first = wm * Cfg::TM + mi * 32;  // whole rows of the wave's TN columns per store instruction
      ix_store_block32_via_lds<NPIECE>(buf, pieces, out + (row0 + first) * Hd + n0 + wn * Cfg::TN, Hd,
                                       min(32, nrows - first));
      return;
    }
    if (!live) return;
    ix_static_for<0, Cfg::NI>([&](auto nic) {
      constexpr int ni = decltype(nic)::value;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const long n = n0 + wn * Cfg::TN + ni * 32 + ix_acc_row(q * 4, lane);
        const int valid = (int)min(4L, (long)Hd - n);
        if (valid <= 0) continue;
        ix_store4_bf16(out + m * Hd + n, valid, true, acc[mi][ni][q * 4], acc[mi][ni][q * 4 + 1],
                       acc[mi][ni][q * 4 + 2], acc[mi][ni][q * 4 + 3]);
      }
    });
  });
}

// ---- streaming form of the second expert GEMM (pipeline F): the four-wave 256 x 256 tile, Hd a multiple of 256, F a
// multiple of 64 with at least IX_STREAM_MIN_KT k-tiles. A workgroup takes every (gridDim.x / 8)-th tile of its XCD's run
// of the (row tile, column tile) order of ix_moe_tile_of_block.
struct IxMoeFc2Seq {
  const bf16_t* inter;
  const bf16_t* W2;
  bf16_t* out;
  const int* meta;
  int max_tiles, Hd, nb_n, K;  // K = F
  long lda, ldw, ldc, parts_ld;  // F, F, Hd, unused
  __device__ __forceinline__ bool locate(unsigned xcd, unsigned idx, IxStreamTile& t) const {
    int mt, nt;
    if (!ix_moe_tile_of_block(xcd + 8u * idx, meta[0], nb_n, &mt, &nt)) return false;
    const long e = meta[1 + mt], row0 = meta[1 + max_tiles + mt];
    t.x = inter + row0 * K;
    t.w = W2 + (e * Hd + (long)nt * 256) * K;
    t.c = out + row0 * Hd + (long)nt * 256;
    t.part = nullptr;
    t.mv = meta[1 + 2 * max_tiles + mt];
    t.nv = 256;
    return true;
  }
};

__global__ __launch_bounds__(256) void k_moe_fc2_stream(const bf16_t* __restrict__ inter, const bf16_t* __restrict__ W2,
                                                        const int* __restrict__ meta, int max_tiles,
                                                        bf16_t* __restrict__ out, int Hd, int F, int nb_n) {
  using Cfg = IxGemmCfg<256, 256, 2, 2>;
  extern __shared__ __align__(16) char ix_lds[];
  IxPlainStreamJob<Cfg, IxMoeFc2Seq, false> job;
  job.seq.inter = inter;
  job.seq.W2 = W2;
  job.seq.out = out;
  job.seq.meta = meta;
  job.seq.max_tiles = max_tiles;
  job.seq.Hd = Hd;
  job.seq.nb_n = nb_n;
  job.seq.K = F;
  job.seq.lda = F;
  job.seq.ldw = F;
  job.seq.ldc = Hd;
  job.seq.parts_ld = 0;
  ix_gemm_stream4<Cfg>(job, F / IX_BK, ix_lds);
}

// ---- streaming form of the first expert GEMM (pipeline F) ------------------------------------------------------------
// The four-wave 256 x 256 tile (128 gate + 128 up columns -> 128 output columns), F a multiple of 128, Hd a multiple of
// 64 with at least NSK + 3 k-tiles. What the one-tile kernel does after its main loop -- the SwiGLU chain of 128 outputs
// per lane, two transcendentals each -- rides here on the NEXT tile's matrix instructions: when the accumulators move
// out they are kept as bf16 pairs (the chain's first rounding: gate and up, 128 registers) and each pair's chain is cut
// into eight steps of two to five instructions, one per matrix instruction of the next tile's first eight k-tiles; then,
// in four more k-tiles, the quad transposes and the stores of the plain job. (NOW > 0 sends the first NOW of the wave's four
// 32-token blocks through the chain at once instead: fewer registers, less hidden.) Same operations in the same order on
// every element as chain2() of the one-tile kernel.
// Column layout: row rho = 8 g + 4 h + i of gate block cb and of up block 2 + cb is output column 32 h + 16 cb + 4 g + i
// of the wave's 64, so a lane ends up with 32 consecutive columns of its token. The permutation is applied where the
// weight rows are fetched (the tile's LDS rows are in matrix-instruction order).
// Token ids and routing weights: every thread loads its own (eight rows' ids, four tokens' weights; the index clamped to
// the last permuted row) with loads the compiler does not count (ix_load4_uncounted), issued in the third-last k-tile
// -- ids of the NEXT tile, weights of the current one -- and taken into use in the second-last: the closing wait of the
// k-tile in between has retired them. A load the compiler knows about would make it wait for the whole operand stream
// at the first use; scalar loads cost their full latency one after the other (3.6 us per tile, measured).
// Scalar registers are short here (six pointers, five descriptors, the ring's bookkeeping): the walk over the weight
// rows is one running vector register, not eight scalar offsets, which the compiler would multiply by the k-tiles of
// the unrolled loop, spill, and reload right in front of the loads that use them.
struct IxMoeFc1StreamJob {
  const bf16_t* x;
  long ldx;
  int T;
  int rows;  // permuted rows in all (T * k)
  const int* sorted_token;
  const float* permuted_prob;
  const bf16_t* W1;
  const int* meta;
  int max_tiles;
  bf16_t* inter;
  int Hd, F, nb_n;
  unsigned xcd, idx, stride;
  static constexpr int NOW = 0;                    // 32-token blocks chained while the accumulators move out (0: all deferred)
  static constexpr int NCH = 2 * (4 - NOW);        // k-tiles of deferred chains
  static constexpr int NSK = NCH + 4;              // + one k-tile of transposes and stores per 32-token block

  ix_rsrc_t nx_xr, nx_wr;
  bool has_next;
  int nx_row0, c_row0, nx_nrows, nx_n0h, c_nrows, c_n0h;
  static constexpr int DMA_IDLE = 0;  // no reloaded scalar operand in front of a load (checked in every build)
  uint32_t xvo[8];  // this thread's eight activation chunks (gathered token rows)
  uint32_t wv;      // its next weight chunk: the ring asks for chunks 0, 1, .. 7, 0, .. and w_voff() steps it on
  int w_st16, w_stA, w_stB, w_stC;  // the four steps of that walk (bytes)
  float prob[4];    // routing weights of this lane's four tokens: set for the current tile in its second-last k-tile, read
                    // when its accumulators move out and by its deferred chains during the next tile
  ix_rsrc_t p_ir;   // pending tile: descriptor of its part of inter
  uint32_t p_voff;
  uint32_t pg[4][2][8], pu[4][2][8];  // pending gate / up values of the deferred blocks, two bf16 per register
  uint32_t res[4][2][8];              // chain results, accumulator layout
  uint32_t ta[4][4], tb[4][4];
  float g0, g1, a0, a1;               // a chain in flight

  __device__ __forceinline__ void locate() {
    int mt = 0, nt = 0;
    has_next = ix_moe_tile_of_block(xcd + 8u * idx, meta[0], nb_n, &mt, &nt);
    if (!has_next) {  // no tile: no rows, and a weight descriptor without bytes (its fetches touch no memory)
      nx_row0 = nx_nrows = nx_n0h = 0;
      nx_wr = ix_make_rsrc(W1, 0u);
      return;
    }
    const long e = meta[1 + mt];
    nx_row0 = meta[1 + max_tiles + mt];
    nx_nrows = meta[1 + 2 * max_tiles + mt];
    nx_n0h = nt * 128;
    // weights: the expert's gate rows n0h .. n0h + 127 and, F rows further on, its up rows
    nx_wr = ix_make_rsrc(W1 + (e * 2 * F + nx_n0h) * Hd, (uint32_t)(((long)F + 128) * Hd * 2));
  }
  __device__ __forceinline__ uint32_t kb() const {
    return (uint32_t)(((threadIdx.x & 7) ^ ix_swz8(threadIdx.x >> 3)) * 16);  // rows 32 apart share the swizzle
  }
  // Loads for the tile after the current one (token ids of this thread's eight rows: tile row r0 + 32 j of chunk j,
  // r0 = thread / 8) and for the current one (routing weights of this lane's four tokens). In flight until take_gathers().
  uint32_t g_tok[8], g_prob[4];
  __device__ __forceinline__ void issue_gathers() {
    const int r0 = threadIdx.x >> 3, last = rows - 1;
    const int trow = (int)(threadIdx.x >> 7) * 128 + (int)(threadIdx.x & 31);  // token of accumulator block row 0
    ix_static_for<0, 8>([&](auto jc) {
      constexpr int j = decltype(jc)::value;
      g_tok[j] = ix_load4_uncounted(sorted_token, (uint32_t)min(nx_row0 + r0 + 32 * j, last) * 4u);
    });
    ix_static_for<0, 4>([&](auto mc) {
      constexpr int mi = decltype(mc)::value;
      g_prob[mi] = ix_load4_uncounted(permuted_prob, (uint32_t)min(c_row0 + trow + 32 * mi, last) * 4u);
    });
  }
  __device__ __forceinline__ void take_gathers() {
    const int r0 = threadIdx.x >> 3;
    ix_static_for<0, 8>([&](auto jc) {
      constexpr int j = decltype(jc)::value;
      const uint32_t tok = ix_landed(g_tok[j]);
      // a row the tile does not have (a missing next tile has none) gets an offset outside the descriptor
      xvo[j] = (r0 + 32 * j < nx_nrows) ? tok * (uint32_t)(ldx * 2) + kb() : IX_OOB;
    });
    // rows past the tile's last got some row's weight: their products are dropped by the store's range check
    ix_static_for<0, 4>([&](auto mc) { prob[decltype(mc)::value] = __uint_as_float(ix_landed(g_prob[decltype(mc)::value])); });
  }
  __device__ __forceinline__ bool open_first() {
    xcd = blockIdx.x & 7u;
    idx = blockIdx.x >> 3;
    stride = gridDim.x >> 3;
    nx_xr = ix_make_rsrc(x, (uint32_t)(((long)(T - 1) * ldx + Hd) * 2));  // the same for every tile
    locate();
    p_ir = ix_make_rsrc(nullptr, 0u);  // the empty pending tile
    p_voff = IX_OOB;
#pragma unroll
    for (int i = 0; i < 64; ++i) pg[i >> 4][(i >> 3) & 1][i & 7] = pu[i >> 4][(i >> 3) & 1][i & 7] = res[i >> 4][(i >> 3) & 1][i & 7] = 0u;
#pragma unroll
    for (int i = 0; i < 4; ++i) prob[i] = 0.0f;
    g0 = g1 = a0 = a1 = 0.0f;
    return has_next;
  }
  __device__ __forceinline__ void open_next() {  // start of the third-last k-tile
    idx += stride;
    locate();
    issue_gathers();
  }
  __device__ __forceinline__ void first_voffs() {
    {  // the first tile's rows: nothing is in flight yet, ordinary loads
      const int r0 = threadIdx.x >> 3;
      uint32_t tok[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) tok[j] = (uint32_t)sorted_token[min(nx_row0 + r0 + 32 * j, rows - 1)];
#pragma unroll
      for (int j = 0; j < 8; ++j) xvo[j] = (r0 + 32 * j < nx_nrows) ? tok[j] * (uint32_t)(ldx * 2) + kb() : IX_OOB;
    }
    // Weight tile row r0 + 32 j (chunk j of thread row r0) = wave column j / 4, block j % 4 (gate 0, gate 1, up 0, up 1),
    // matrix-instruction row r0: weight row [up: F] + 64 (j / 4) + 16 (j % 2) + lane_col(r0) of the descriptor.
    // In rows, chunk 0..7 = 0, 16, F, F + 16, 64, 80, F + 64, F + 80 (+ lane_col); the walk's steps are the differences.
    const int r0 = threadIdx.x >> 3;
    const int lane_col = 32 * ((r0 >> 2) & 1) + 4 * (r0 >> 3) + (r0 & 3);
    wv = (uint32_t)((long)lane_col * Hd * 2) + kb();
    const int row_bytes = Hd * 2;
    w_st16 = __builtin_amdgcn_readfirstlane(16 * row_bytes);
    w_stA = __builtin_amdgcn_readfirstlane((F - 16) * row_bytes);
    w_stB = __builtin_amdgcn_readfirstlane((48 - F) * row_bytes);
    w_stC = __builtin_amdgcn_readfirstlane(-(F + 80) * row_bytes);
  }
  template <int J>
  __device__ __forceinline__ uint32_t x_voff() const { return xvo[J]; }
  // The step is added by an instruction the compiler cannot hoist, or it would keep every sum of every k-tile in a
  // register of its own.
  template <int J>
  __device__ __forceinline__ uint32_t w_voff() {
    const uint32_t v = wv;
    asm volatile("v_add_u32 %0, %1, %0" : "+v"(wv) : "s"(J == 7 ? w_stC : (J == 3 ? w_stB : ((J & 1) ? w_stA : w_st16))));
    return v;
  }
  // second-last k-tile, after the current tile's last fetch through xvo: the loads of the k-tile before have retired
  __device__ __forceinline__ void turn_offsets() { take_gathers(); }
  __device__ __forceinline__ void advance() {
    c_row0 = nx_row0;
    c_nrows = nx_nrows;
    c_n0h = nx_n0h;
  }
  // bf16(gate), bf16(up) -> s = bf16(silu(gate)) -> h = bf16(s * up) -> bf16(h * prob), two columns at a time
  static __device__ __forceinline__ uint32_t chain2(float g0_, float g1_, float u0_, float u1_, float p) {
    float gate0, gate1, up0, up1, s0, s1, h0, h1;
    ix_rbf2_hw(g0_, g1_, gate0, gate1);
    ix_rbf2_hw(u0_, u1_, up0, up1);
    ix_rbf2_hw(ix_silu_div(gate0), ix_silu_div(gate1), s0, s1);
    ix_rbf2_hw(s0 * up0, s1 * up1, h0, h1);
    return ix_pack_bf2_hw(h0 * p, h1 * p);
  }
  template <typename Acc>
  __device__ __forceinline__ void drain(Acc& acc) {
    ix_static_for<0, 8>([&](auto bc) {
      constexpr int mi = decltype(bc)::value >> 1, cb = decltype(bc)::value & 1;
      float g16[16], u16[16];
      ix_acc_read16<true>(acc[mi][cb], g16);
      ix_acc_read16<true>(acc[mi][2 + cb], u16);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if constexpr (mi < NOW) {
          res[mi][cb][i] = chain2(g16[2 * i], g16[2 * i + 1], u16[2 * i], u16[2 * i + 1], prob[mi]);
        } else {
          pg[mi][cb][i] = ix_pack_bf2_hw(g16[2 * i], g16[2 * i + 1]);
          pu[mi][cb][i] = ix_pack_bf2_hw(u16[2 * i], u16[2 * i + 1]);
        }
      }
      if constexpr (mi < NOW) {
        ix_pin8(res[mi][cb]);
      } else {
        ix_pin8(pg[mi][cb]);
        ix_pin8(pu[mi][cb]);
      }
    });
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // after the quad transposes a lane holds piece (lane % 4) of the four tokens of its quad
    const int r = (wave >> 1) * 128 + (lane & 28), c = (wave & 1) * 64 + 32 * (lane >> 5) + 8 * (lane & 3);
    p_ir = ix_make_rsrc(inter + (long)c_row0 * F + c_n0h, (uint32_t)(((long)(c_nrows - 1) * F + 128) * 2));
    p_voff = (uint32_t)(((long)r * F + c) * 2);
  }
  static constexpr int stores_after_p1(int s) { return s >= NCH ? 4 : 0; }
  static __device__ __forceinline__ int w_frag_row(int ni, int rho) { return ni * 32 + rho; }
  // k-tile s < NCH: the eight chains of (mi = NOW + s / 2, cb = s % 2), chain c in slots 8 c .. 8 c + 7.
  // k-tile s = NCH + mi: the 32 tokens mi: exchange stage 1 in slots 0..15, stage 2 in 16..31, stores 32..35.
  template <int I>
  __device__ __forceinline__ void micro() {
    constexpr int s = I / 64, q = I % 64;
    if constexpr (s < NCH) {
      constexpr int mi = NOW + (s >> 1), cb = s & 1, c = q >> 3, st = q & 7;
      if constexpr (st == 0) {
        g0 = __uint_as_float(pg[mi][cb][c] << 16);
        g1 = __uint_as_float(pg[mi][cb][c] & 0xffff0000u);
        a0 = (-g0) * IX_LOG2E;
        a1 = (-g1) * IX_LOG2E;
      } else if constexpr (st == 1) {
        a0 = ix_exp2(a0);
      } else if constexpr (st == 2) {
        a1 = ix_exp2(a1);
      } else if constexpr (st == 3) {
        a0 = 1.0f + a0;
        a1 = 1.0f + a1;
        a0 = __builtin_amdgcn_rcpf(a0);
      } else if constexpr (st == 4) {
        a1 = __builtin_amdgcn_rcpf(a1);
        a0 = g0 * a0;
      } else if constexpr (st == 5) {
        a1 = g1 * a1;
        ix_rbf2_hw(a0, a1, a0, a1);
      } else if constexpr (st == 6) {
        const float u0 = __uint_as_float(pu[mi][cb][c] << 16), u1 = __uint_as_float(pu[mi][cb][c] & 0xffff0000u);
        ix_rbf2_hw(a0 * u0, a1 * u1, a0, a1);
      } else {
        res[mi][cb][c] = ix_pack_bf2_hw(a0 * prob[mi], a1 * prob[mi]);
      }
    } else {
      constexpr int mi = s - NCH;
      if constexpr (q < 16) {
        // piece pi, dword d of the lane's 64 bytes: res[mi][pi / 2][4 (pi % 2) + d]; stage 1 pairs pieces (0, 1), (2, 3)
        constexpr int d = q >> 2, t = q & 3, a = t & 2;
        ta[t][d] = ix_quad_exchange<1, (t & 1) != 0>(res[mi][a >> 1][d], res[mi][a >> 1][4 + d]);
      } else if constexpr (q < 32) {
        constexpr int o = q - 16, d = o >> 2, t = o & 3, a = t & 1;
        tb[t][d] = ix_quad_exchange<2, (t & 2) != 0>(ta[a][d], ta[a + 2][d]);
      } else if constexpr (q < 36) {
        constexpr int t = q - 32;  // token t of the quad
        ix_buffer_store16<IX_STREAM_STORE_NT_FC1>(make_uint4(tb[t][0], tb[t][1], tb[t][2], tb[t][3]), p_ir,
                          p_voff == IX_OOB ? IX_OOB : p_voff + (uint32_t)((long)(mi * 32 + t) * F * 2));
      }
    }
  }
};

__global__ __launch_bounds__(256) void k_moe_fc1_glu_stream(const bf16_t* __restrict__ x, long ldx, int T, int rows,
                                                            const int* __restrict__ sorted_token,
                                                            const float* __restrict__ permuted_prob,
                                                            const bf16_t* __restrict__ W1, const int* __restrict__ meta,
                                                            int max_tiles, bf16_t* __restrict__ inter, int Hd, int F,
                                                            int nb_n) {
  using Cfg = IxGemmCfg<256, 256, 2, 2>;
  extern __shared__ __align__(16) char ix_lds[];
  IxMoeFc1StreamJob job;
  job.x = x;
  job.ldx = ldx;
  job.T = T;
  job.rows = rows;
  job.sorted_token = sorted_token;
  job.permuted_prob = permuted_prob;
  job.W1 = W1;
  job.meta = meta;
  job.max_tiles = max_tiles;
  job.inter = inter;
  job.Hd = Hd;
  job.F = F;
  job.nb_n = nb_n;
  ix_gemm_stream4<Cfg>(job, Hd / IX_BK, ix_lds);
}

template <int BM, int BN, int WM, int WN>
static int ix_moe_experts_launch(const bf16_t* x, long ldx, int T, long rows, const int* sorted_token,
                                 const float* permuted_prob,
                                 const bf16_t* W1, const bf16_t* W2, const int* meta, long max_tiles,
                                 bf16_t* inter, bf16_t* out, int Hd, int F, hipStream_t st) {
  using Cfg = IxGemmCfg<BM, BN, WM, WN>;
  auto k1 = k_moe_fc1_glu<BM, BN, WM, WN>;
  auto k2 = k_moe_fc2<BM, BN, WM, WN>;
  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)k1, hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES) !=
            hipSuccess ||
        hipFuncSetAttribute((const void*)k2, hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES) !=
            hipSuccess)
      return IX_ERR_LAUNCH;
    attr_set = true;
  }
  const long nb1 = (F + BN / 2 - 1) / (BN / 2);
  const long nb2 = (Hd + BN - 1) / BN;
  if (max_tiles * nb1 > 0x7fffffffL || max_tiles * nb2 > 0x7fffffffL) return IX_DECLINED;
  // 8 XCD runs of the tile order; the longest run sets the count
  bool fc1_streamed = false;
  if constexpr (BM == 256 && BN == 256 && WM == 2 && WN == 2) {
    // worth it from two tiles per workgroup up (max_tiles bounds the row tiles from above by at most one per expert)
    // (32-bit byte offsets into the permutation's arrays and into an expert's weight rows)
    if (Hd % IX_BK == 0 && Hd / IX_BK >= IxMoeFc1StreamJob::NSK + 3 && F % 128 == 0 && rows > 0 && rows < 0x20000000L &&
        ((long)F + 128) * Hd * 2 < 0x40000000L && max_tiles * nb1 >= 2 * IX_STREAM_WORKGROUPS) {
      static bool attr1_set = false;
      if (!attr1_set) {
        if (hipFuncSetAttribute((const void*)k_moe_fc1_glu_stream, hipFuncAttributeMaxDynamicSharedMemorySize,
                                Cfg::LDS_BYTES) != hipSuccess)
          return IX_ERR_LAUNCH;
        attr1_set = true;
      }
      hipLaunchKernelGGL(k_moe_fc1_glu_stream, dim3(IX_STREAM_WORKGROUPS), dim3(256), Cfg::LDS_BYTES, st, x, ldx, T,
                         (int)rows, sorted_token, permuted_prob, W1, meta, (int)max_tiles, inter, Hd, F, (int)nb1);
      fc1_streamed = true;
    }
  }
  if (!fc1_streamed)
    hipLaunchKernelGGL(k1, dim3((unsigned)(8 * ((max_tiles * nb1 + 7) / 8))), dim3(Cfg::NT), Cfg::LDS_BYTES, st, x, ldx, T,
                       sorted_token, permuted_prob, W1, meta, (int)max_tiles, inter, Hd, F, (int)nb1);
  if constexpr (BM == 256 && BN == 256 && WM == 2 && WN == 2) {
    // worth it from two tiles per workgroup up (max_tiles bounds the row tiles from above by at most one per expert)
    if (F % IX_BK == 0 && F / IX_BK >= IX_STREAM_MIN_KT && Hd % 256 == 0 && (long)Hd * 512 < 0x40000000L &&
        max_tiles * nb2 >= 2 * IX_STREAM_WORKGROUPS) {
      static bool attr2_set = false;
      if (!attr2_set) {
        if (hipFuncSetAttribute((const void*)k_moe_fc2_stream, hipFuncAttributeMaxDynamicSharedMemorySize,
                                Cfg::LDS_BYTES) != hipSuccess)
          return IX_ERR_LAUNCH;
        attr2_set = true;
      }
      hipLaunchKernelGGL(k_moe_fc2_stream, dim3(IX_STREAM_WORKGROUPS), dim3(256), Cfg::LDS_BYTES, st, inter, W2, meta,
                         (int)max_tiles, out, Hd, F, (int)nb2);
      return ix_launch_status();
    }
  }
  hipLaunchKernelGGL(k2, dim3((unsigned)(8 * ((max_tiles * nb2 + 7) / 8))), dim3(Cfg::NT), Cfg::LDS_BYTES, st, inter, W2, meta,
                     (int)max_tiles, out, Hd, F, (int)nb2);
  return ix_launch_status();
}

extern "C" int ix_moe_experts_tile(const void* x, long ldx, const int* sorted_token, const float* permuted_prob,
                                   const void* W1, const void* W2, const int* tile_meta, long max_tiles, long BM,
                                   long BN, void* inter, void* expert_out, long T, long rows, long Hd, long F,
                                   void* stream) {
  if (!x || !sorted_token || !permuted_prob || !W1 || !W2 || !tile_meta || !inter || !expert_out)
    return IX_ERR_ARG;
  if (T < 0 || rows < 0 || Hd <= 0 || F <= 0 || max_tiles < 0 || ldx < Hd) return IX_ERR_ARG;
  // 32-bit buffer offsets: the activation matrix, one expert's weights and one row tile must fit
  if (T * ldx * 2 >= 0x40000000L || 2 * F * Hd * 2 >= 0x40000000L || 256 * F * 2 >= 0x40000000L) return IX_DECLINED;
  if ((Hd % 8) || (F % 8) || (ldx % 8) || !ix_aligned(x, 16) || !ix_aligned(W1, 16) || !ix_aligned(W2, 16) ||
      !ix_aligned(inter, 16) || !ix_aligned(expert_out, 8))
    return IX_DECLINED;
  if (rows == 0 || max_tiles == 0) return IX_OK;
  hipStream_t st = (hipStream_t)stream;
  const bf16_t *xx = (const bf16_t*)x, *w1 = (const bf16_t*)W1, *w2 = (const bf16_t*)W2;
  bf16_t *it = (bf16_t*)inter, *eo = (bf16_t*)expert_out;
  if (BN != 256 && !(BN == 128 && BM == 128)) return IX_ERR_ARG;
  if (BN == 128)
    return ix_moe_experts_launch<128, 128, 2, 2>(xx, ldx, (int)T, rows, sorted_token, permuted_prob, w1, w2, tile_meta,
                                                 max_tiles, it, eo, (int)Hd, (int)F, st);
  switch (BM) {
    case 32:
      return ix_moe_experts_launch<32, 256, 1, 4>(xx, ldx, (int)T, rows, sorted_token, permuted_prob, w1, w2, tile_meta,
                                                  max_tiles, it, eo, (int)Hd, (int)F, st);
    case 128:
      return ix_moe_experts_launch<128, 256, 2, 4>(xx, ldx, (int)T, rows, sorted_token, permuted_prob, w1, w2, tile_meta,
                                                   max_tiles, it, eo, (int)Hd, (int)F, st);
    case 256:
      return ix_moe_experts_launch<256, 256, 2, 2>(xx, ldx, (int)T, rows, sorted_token, permuted_prob, w1, w2, tile_meta,
                                                   max_tiles, it, eo, (int)Hd, (int)F, st);
    default: return IX_ERR_ARG;
  }
}

extern "C" int ix_moe_experts(const void* x, long ldx, const int* sorted_token, const float* permuted_prob,
                              const void* W1, const void* W2, const int* tile_meta, long max_tiles, long BM,
                              void* inter, void* expert_out, long T, long rows, long Hd, long F, void* stream) {
  return ix_moe_experts_tile(x, ldx, sorted_token, permuted_prob, W1, W2, tile_meta, max_tiles, BM, 256, inter,
                             expert_out, T, rows, Hd, F, stream);
}

// ---------------------------------------------------------------------------------------------
// The grouped GEMMs of a decode step: weights streamed through registers.
//
// At decode sizes an expert has a handful of rows, the matrix pipes idle and the step is the time memory needs to
// deliver every touched expert's weights once. The ring kernels above stage weights in LDS, so a CU never has more
// than its 160 KiB in flight (one workgroup, ~100 KiB of weight bytes): about 5.1 TB/s. Here no LDS is used at all:
//   * weights are stored FRAGMENT-PACKED (ix_moe_pack_decode): per (expert, column tile, wave, k-tile) the 8 KiB a wave's
//     eight matrix instructions of that k-tile take as their A operands, in (block, step, lane) order, so that a load
//     instruction is 1 KiB of contiguous memory and a wave walks one contiguous stream;
//   * a lane keeps the fragments of the next D k-tiles in registers (D x 8 loads of 16 bytes in flight per lane, two
//     workgroups per CU: up to 256 KiB of weight bytes in flight per CU);
//   * activations (at most 32 token rows per tile, typically four live ones) come straight from memory as B operands,
//     a lane loading the 16 bytes of its own token, as far ahead as the weights; a dead token's lanes load a live row
//     and multiply zeros instead. No barrier, no shared state: the four waves of a workgroup only share the tile.
// Arithmetic is that of every other tile shape: v_mfma_f32_32x32x16_bf16, weights the A operand, K in tiles of 64, step
// s consuming k = 8 s .. 8 s + 7 (lane group 0) and 32 + 8 s .. (lane group 1), one fp32 accumulator per element, the
// epilogues of k_moe_fc1_glu / k_moe_fc2 statement for statement.
// Packed layouts (16-byte chunk index; r = lane % 32, g = lane / 32; chunk = W[row][64 kt + 32 g + 8 s .. + 7]):
//   W1f [E][F / 128][wave 4][Hd / 64][b 2][s 4][lane 64]   row = b F + 128 nt + 32 wave + r      (b: gate, up)
//   W2f [E][Hd / 256][wave 4][F / 64][b 2][s 4][lane 64]   row = 256 nt + 64 wave + 32 b + r
#define IX_DEC_D 4  // k-tiles of weight fragments a lane holds ahead of the matrix instructions

__global__ __launch_bounds__(256) void k_moe_pack_frag(const bf16_t* __restrict__ W, bf16_t* __restrict__ Wf,
                                                       int rows_per_expert, int K, int nb, int is_fc1, long chunks) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= chunks) return;
  const int KT = K / 64;
  const int lane = (int)(i & 63), st = (int)((i >> 6) & 3), b = (int)((i >> 8) & 1);
  long rest = i >> 9;
  const int kt = (int)(rest % KT);
  rest /= KT;
  const int w = (int)(rest & 3);
  rest >>= 2;
  const int nt = (int)(rest % nb);
  const long e = rest / nb;
  const int r = lane & 31, g = lane >> 5;
  const int row = is_fc1 ? b * (rows_per_expert / 2) + 128 * nt + 32 * w + r : 256 * nt + 64 * w + 32 * b + r;
  const uint4 v = *reinterpret_cast<const uint4*>(W + (e * rows_per_expert + row) * (long)K + 64 * kt + 32 * g + 8 * st);
  *reinterpret_cast<uint4*>(Wf + i * 8) = v;
}

template <int D>
struct IxDecStream {
  const uint4* wp;   // this lane's first chunk of the wave's stream: k-tile kt, chunk c at wp[kt * 512 + c * 64]
  const bf16_t* xp;  // this lane's token row + 32 g (a dead token's lanes point at a live row and discard what they load)
  bool live;
  uint4 wreg[D][8];
  uint4 xreg[D][4];
  __device__ __forceinline__ void load_w(uint4 (&dst)[8], int kt) {
#pragma unroll
    for (int c = 0; c < 8; ++c) dst[c] = wp[(long)kt * 512 + c * 64];
  }
  __device__ __forceinline__ void load_x(uint4 (&dst)[4], int kt) {
#pragma unroll
    for (int st = 0; st < 4; ++st) dst[st] = *reinterpret_cast<const uint4*>(xp + 64 * kt + 8 * st);
  }
  template <int d>
  __device__ __forceinline__ void multiply(const uint4 (&xc)[4], ix_f32x16& a0, ix_f32x16& a1) {
#pragma unroll
    for (int st = 0; st < 4; ++st) {
      uint4 xv = xc[st];
      if (!live) xv = make_uint4(0u, 0u, 0u, 0u);  // a select, not a branch
      const ix_bf16x8 xf = *reinterpret_cast<const ix_bf16x8*>(&xv);
      a0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const ix_bf16x8*>(&wreg[d][st]), xf, a0, 0, 0, 0);
      a1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const ix_bf16x8*>(&wreg[d][4 + st]), xf, a1, 0, 0, 0);
    }
  }
  // The whole product of a wave: two 32 x 32 blocks (weight chunks 0..3 -> a0, 4..7 -> a1) over KT_ k-tiles. KT_ is a
  // compile-time constant and the walk is straight-line code: with a loop (or any branch) the compiler's wait
  // bookkeeping falls back to "wait for every load" at the join, which would drain the D k-tiles in flight at every
  // step; in straight-line code it waits for exactly the loads a matrix instruction reads.
  template <int KT_>
  __device__ __forceinline__ void run(ix_f32x16& a0, ix_f32x16& a1) {
    static_assert(KT_ >= D, "the ring is filled before the first multiply");
    // sched_barrier(0): the compiler's scheduler may not move a load across it -- left alone it sinks every load down
    // to its first use (fewest live registers), which is a ring of depth zero. Loads retire in order, so the
    // activation fragments of a k-tile are requested together with its weight fragments, D k-tiles ahead: a wait for
    // k-tile kt then leaves the (D - 1) x 12 younger loads in flight.
    ix_static_for<0, D>([&](auto dc) {
      load_x(xreg[decltype(dc)::value], decltype(dc)::value);
      load_w(wreg[decltype(dc)::value], decltype(dc)::value);
    });
    __builtin_amdgcn_sched_barrier(0);
    ix_static_for<0, KT_>([&](auto kc) {
      constexpr int kt = decltype(kc)::value, d = kt % D;
      multiply<d>(xreg[d], a0, a1);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (kt + D < KT_) {
        load_x(xreg[d], kt + D);
        load_w(wreg[d], kt + D);
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  }
};

template <int D, int KT>
__global__ __launch_bounds__(256, 2) void k_moe_fc1_dec(const bf16_t* __restrict__ x, long ldx,
                                                        const int* __restrict__ sorted_token,
                                                        const float* __restrict__ permuted_prob,
                                                        const bf16_t* __restrict__ W1f, const int* __restrict__ meta,
                                                        int max_tiles, bf16_t* __restrict__ inter, int Hd, int F,
                                                        int nb_n) {
  int mt, nt;
  if (!ix_moe_tile_of_block(blockIdx.x, meta[0], nb_n, &mt, &nt)) return;
  const long e = meta[1 + mt];
  const long row0 = meta[1 + max_tiles + mt];
  const int nrows = meta[1 + 2 * max_tiles + mt];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int r = lane & 31, g = lane >> 5;
  const bool live = r < nrows;
  IxDecStream<D> st;
  st.wp = reinterpret_cast<const uint4*>(W1f) + (((e * nb_n + nt) * 4 + w) * (long)KT) * 512 + lane;
  st.live = live;
  st.xp = x + (long)sorted_token[row0 + (live ? r : 0)] * ldx + 32 * g;  // a tile has at least one row
  ix_f32x16 ag, au;
#pragma unroll
  for (int i = 0; i < 16; ++i) ag[i] = au[i] = 0.0f;
  st.template run<KT>(ag, au);
  if (!live) return;
  const long m = row0 + r;
  const float prob = permuted_prob[m];
  const int c0 = nt * 128 + w * 32;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int col = c0 + ix_acc_row(q * 4, lane);
    const uint32_t lo = IxMoeFc1StreamJob::chain2(ag[q * 4], ag[q * 4 + 1], au[q * 4], au[q * 4 + 1], prob);
    const uint32_t hi = IxMoeFc1StreamJob::chain2(ag[q * 4 + 2], ag[q * 4 + 3], au[q * 4 + 2], au[q * 4 + 3], prob);
    *reinterpret_cast<uint2*>(inter + m * F + col) = make_uint2(lo, hi);  // col % 4 == 0, F % 8 == 0, inter 16-byte aligned
  }
}

template <int D, int KT>
__global__ __launch_bounds__(256, 2) void k_moe_fc2_dec(const bf16_t* __restrict__ inter, const bf16_t* __restrict__ W2f,
                                                        const int* __restrict__ meta, int max_tiles,
                                                        bf16_t* __restrict__ out, int Hd, int F, int nb_n) {
  int mt, nt;
  if (!ix_moe_tile_of_block(blockIdx.x, meta[0], nb_n, &mt, &nt)) return;
  const long e = meta[1 + mt];
  const long row0 = meta[1 + max_tiles + mt];
  const int nrows = meta[1 + 2 * max_tiles + mt];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int r = lane & 31, g = lane >> 5;
  const bool live = r < nrows;
  IxDecStream<D> st;
  st.wp = reinterpret_cast<const uint4*>(W2f) + (((e * nb_n + nt) * 4 + w) * (long)KT) * 512 + lane;
  st.live = live;
  st.xp = inter + (row0 + (live ? r : 0)) * (long)F + 32 * g;  // a tile has at least one row
  ix_f32x16 a0, a1;
#pragma unroll
  for (int i = 0; i < 16; ++i) a0[i] = a1[i] = 0.0f;
  st.template run<KT>(a0, a1);
  if (!live) return;
  const long m = row0 + r;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const long n = (long)nt * 256 + w * 64 + ix_acc_row(q * 4, lane);
    ix_store4_bf16(out + m * Hd + n, 4, true, a0[q * 4], a0[q * 4 + 1], a0[q * 4 + 2], a0[q * 4 + 3]);
    ix_store4_bf16(out + m * Hd + n + 32, 4, true, a1[q * 4], a1[q * 4 + 1], a1[q * 4 + 2], a1[q * 4 + 3]);
  }
}

// The k-tile counts the straight-line kernels are instantiated for (K = 64 KT).
#define IX_DEC_KTS(M) M(8) M(12) M(16) M(24) M(32) M(48) M(64)
static bool ix_moe_decode_kt_served(long kt) {
#define IX_DEC_IS(KT_) if (kt == KT_) return true;
  IX_DEC_KTS(IX_DEC_IS)
#undef IX_DEC_IS
  return false;
}
static bool ix_moe_decode_serves(long Hd, long F) {
  return Hd % 256 == 0 && F % 128 == 0 && ix_moe_decode_kt_served(Hd / 64) && ix_moe_decode_kt_served(F / 64);
}

// Fragment-packed copies of both expert matrices for the decode kernels (each the size of its source).
extern "C" int ix_moe_pack_decode(const void* W1, const void* W2, void* W1f, void* W2f, long E, long Hd, long F,
                                  void* stream) {
  if (!W1 || !W2 || !W1f || !W2f || E <= 0 || Hd <= 0 || F <= 0) return IX_ERR_ARG;
  if (!ix_moe_decode_serves(Hd, F) || !ix_aligned(W1, 16) || !ix_aligned(W2, 16) || !ix_aligned(W1f, 16) ||
      !ix_aligned(W2f, 16))
    return IX_DECLINED;
  const long c1 = E * 2 * F * Hd / 8, c2 = E * Hd * F / 8;
  if ((c1 + 255) / 256 > 0x7fffffffL) return IX_DECLINED;
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(k_moe_pack_frag, dim3((unsigned)((c1 + 255) / 256)), dim3(256), 0, st, (const bf16_t*)W1, (bf16_t*)W1f,
                     (int)(2 * F), (int)Hd, (int)(F / 128), 1, c1);
  hipLaunchKernelGGL(k_moe_pack_frag, dim3((unsigned)((c2 + 255) / 256)), dim3(256), 0, st, (const bf16_t*)W2, (bf16_t*)W2f,
                     (int)Hd, (int)F, (int)(Hd / 256), 0, c2);
  return ix_launch_status();
}

// ix_moe_experts for a block map of 32-row tiles (BM = 32), reading the fragment-packed matrices.
extern "C" int ix_moe_experts_decode(const void* x, long ldx, const int* sorted_token, const float* permuted_prob,
                                     const void* W1f, const void* W2f, const int* tile_meta, long max_tiles, void* inter,
                                     void* expert_out, long T, long rows, long Hd, long F, void* stream) {
  if (!x || !sorted_token || !permuted_prob || !W1f || !W2f || !tile_meta || !inter || !expert_out) return IX_ERR_ARG;
  if (T < 0 || rows < 0 || Hd <= 0 || F <= 0 || max_tiles < 0 || ldx < Hd) return IX_ERR_ARG;
  if (!ix_moe_decode_serves(Hd, F) || (ldx % 8) || !ix_aligned(x, 16) || !ix_aligned(W1f, 16) || !ix_aligned(W2f, 16) ||
      !ix_aligned(inter, 16) || !ix_aligned(expert_out, 16))
    return IX_DECLINED;
  if (rows == 0 || max_tiles == 0) return IX_OK;
  const long nb1 = F / 128, nb2 = Hd / 256;
  if (max_tiles * nb1 > 0x7fffffffL || max_tiles * nb2 > 0x7fffffffL) return IX_DECLINED;
  hipStream_t st = (hipStream_t)stream;
#define IX_DEC_FC1(KT_)                                                                                               \
  if (Hd / 64 == KT_)                                                                                                 \
    hipLaunchKernelGGL((k_moe_fc1_dec<IX_DEC_D, KT_>), dim3((unsigned)(8 * ((max_tiles * nb1 + 7) / 8))), dim3(256), 0, st, \
                       (const bf16_t*)x, ldx, sorted_token, permuted_prob, (const bf16_t*)W1f, tile_meta, (int)max_tiles, \
                       (bf16_t*)inter, (int)Hd, (int)F, (int)nb1);
#define IX_DEC_FC2(KT_)                                                                                               \
  if (F / 64 == KT_)                                                                                                  \
    hipLaunchKernelGGL((k_moe_fc2_dec<IX_DEC_D, KT_>), dim3((unsigned)(8 * ((max_tiles * nb2 + 7) / 8))), dim3(256), 0, st, \
                       (const bf16_t*)inter, (const bf16_t*)W2f, tile_meta, (int)max_tiles, (bf16_t*)expert_out, (int)Hd, \
                       (int)F, (int)nb2);
  IX_DEC_KTS(IX_DEC_FC1)
  IX_DEC_KTS(IX_DEC_FC2)
#undef IX_DEC_FC1
#undef IX_DEC_FC2
  return ix_launch_status();
}

// ---------------------------------------------------------------------------------------------
// KC > 0: k known at compile time -- the k row numbers and the k rows are requested before the first add, so a thread has
// k loads in flight instead of one (the sum is the same left-to-right sum). KC = 0: any k.
template <int KC>
__global__ __launch_bounds__(256) void k_moe_combine(const bf16_t* __restrict__ expert_out,
                                                     const int* __restrict__ combine_rows,
                                                     bf16_t* __restrict__ out, long T, int Hd, int k, int fp32_acc,
                                                     int vec) {
  const int groups = (Hd + 7) / 8;
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= T * groups) return;
  const long t = i / groups;
  const int c0 = (int)(i % groups) * 8;
  float acc[8];
  if constexpr (KC > 0) {
    long row[KC];
    float xv[KC][8];
#pragma unroll
    for (int r = 0; r < KC; ++r) row[r] = combine_rows[t * KC + r];
#pragma unroll
    for (int r = 0; r < KC; ++r) ix_load8(expert_out + row[r] * Hd + c0, Hd - c0, vec != 0, 0.0f, xv[r]);
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = xv[0][j];
#pragma unroll
    for (int r = 1; r < KC; ++r) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float sum = acc[j] + xv[r][j];
        acc[j] = fp32_acc ? sum : ix_rbf(sum);
      }
    }
  } else {
    for (int r = 0; r < k; ++r) {
      const long row = combine_rows[t * k + r];
      float xv[8];
      ix_load8(expert_out + row * Hd + c0, Hd - c0, vec != 0, 0.0f, xv);
      if (r == 0) {
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] = xv[j];
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float sum = acc[j] + xv[j];
          acc[j] = fp32_acc ? sum : ix_rbf(sum);
        }
      }
    }
  }
  ix_store8_bf16(out + t * Hd + c0, Hd - c0, vec != 0, acc);
}

extern "C" int ix_moe_combine(const void* expert_out, const int* combine_rows, void* out, long T, long Hd, long k,
                              int fp32_acc, void* stream) {
  if (!expert_out || !combine_rows || !out || T < 0 || Hd <= 0 || k <= 0) return IX_ERR_ARG;
  if (T == 0) return IX_OK;
  const long groups = (Hd + 7) / 8;
  const long grid = (T * groups + 255) / 256;
  if (grid > 0x7fffffffL) return IX_DECLINED;
  const int vec = (Hd % 8 == 0) && ix_aligned(expert_out, 16) && ix_aligned(out, 16);
#define IX_COMBINE(KC_)                                                                                        \
  hipLaunchKernelGGL(k_moe_combine<KC_>, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream,             \
                     (const bf16_t*)expert_out, combine_rows, (bf16_t*)out, T, (int)Hd, (int)k, fp32_acc, vec)
  switch (k) {
    case 2: IX_COMBINE(2); break;
    case 4: IX_COMBINE(4); break;
    case 8: IX_COMBINE(8); break;
    default: IX_COMBINE(0); break;
  }
#undef IX_COMBINE
  return ix_launch_status();
}

// ---------------------------------------------------------------------------------------------
// The combine with a weight per expert row and any of the eager form's dtypes (moe_batch_invariant.py:276-320 after
// :366-369 `permuted_tokens * permuted_probs.unsqueeze(-1)`): value_r = x[row_r] * w[row_r], summed left to right
// over a token's k rows. The arithmetic dtype is torch's promotion of (token dtype, weight dtype): in bf16 the
// product and every partial sum are rounded to bf16, in fp32 nothing is rounded before the store.
template <typename TIN>
__global__ __launch_bounds__(256) void k_moe_combine_weighted(const TIN* __restrict__ expert_out,
                                                              const float* __restrict__ row_weight,
                                                              const int* __restrict__ combine_rows, void* __restrict__ out,
                                                              long T, int Hd, int k, int arith_bf16, int out_bf16,
                                                              int vec) {
  const int groups = (Hd + 7) / 8;
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= T * groups) return;
  const long t = i / groups;
  const int c0 = (int)(i % groups) * 8;
  float acc[8];
  for (int r = 0; r < k; ++r) {
    const long row = combine_rows[t * k + r];
    float xv[8];
    ix_load8(expert_out + row * Hd + c0, Hd - c0, vec != 0, 0.0f, xv);
    if (row_weight) {
      const float w = row_weight[row];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float prod = xv[j] * w;
        xv[j] = arith_bf16 ? ix_rbf(prod) : prod;
      }
    }
    if (r == 0) {
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] = xv[j];
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float sum = acc[j] + xv[j];
        acc[j] = arith_bf16 ? ix_rbf(sum) : sum;
      }
    }
  }
  if (out_bf16) {
    ix_store8_bf16((bf16_t*)out + t * Hd + c0, Hd - c0, vec != 0, acc);
  } else {
    float* o = (float*)out + t * Hd + c0;
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (c0 + j < Hd) o[j] = acc[j];
  }
}

extern "C" int ix_moe_combine_weighted(const void* expert_out, int in_dtype, const float* row_weight, int arith_dtype,
                                       const int* combine_rows, void* out, int out_dtype, long T, long Hd, long k,
                                       void* stream) {
  if (!expert_out || !combine_rows || !out || T < 0 || Hd <= 0 || k <= 0) return IX_ERR_ARG;
  const auto known = [](int d) { return d == IX_DT_F32 || d == IX_DT_BF16; };
  if (!known(in_dtype) || !known(arith_dtype) || !known(out_dtype)) return IX_DECLINED;
  if (in_dtype == IX_DT_F32 && arith_dtype == IX_DT_BF16) return IX_ERR_ARG;  // promotion never narrows
  if (T == 0) return IX_OK;
  const long groups = (Hd + 7) / 8;
  const long grid = (T * groups + 255) / 256;
  if (grid > 0x7fffffffL) return IX_DECLINED;
  const int vec = (Hd % 8 == 0) && ix_aligned(expert_out, 16) && ix_aligned(out, 16);
  const int ab = arith_dtype == IX_DT_BF16, ob = out_dtype == IX_DT_BF16;
  if (in_dtype == IX_DT_BF16)
    hipLaunchKernelGGL(k_moe_combine_weighted<bf16_t>, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream,
                       (const bf16_t*)expert_out, row_weight, combine_rows, out, T, (int)Hd, (int)k, ab, ob, vec);
  else
    hipLaunchKernelGGL(k_moe_combine_weighted<float>, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream,
                       (const float*)expert_out, row_weight, combine_rows, out, T, (int)Hd, (int)k, ab, ob, vec);
  return ix_launch_status();
}
