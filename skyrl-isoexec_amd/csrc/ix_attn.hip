// Causal grouped-query attention over packed sequences with ONE walk of the keys per query, and
// rotary position embedding.
//
// The canonical function, per (query token at absolute position p, query head h):
//   keys 0..p of the query's own sequence are walked in blocks of 32, block b = keys [32b, 32b+32);
//   with c = scale * log2(e) (one fp32 product), per block:
//               s_j  = q . k_j                           bf16 MFMA, fp32 accumulate, d in 8 steps of 16
//               s_j  = -inf for j > p
//               m'   = max(m, max_j s_j)                 running maximum of the UNSCALED scores (scale > 0)
//               a    = exp2((m - m') * c)                exactly 1 when the maximum did not move
//               p_j  = exp2(fma(s_j, c, -(m' * c)))      one fused multiply-add per score
//               l    = l * a + (lo + hi)                 lo/hi: the two halves' sums, see ix_attn_block
//               O    = O * a + sum_j bf16(p_j) * v_j     bf16 MFMA, fp32 accumulate, keys in 2 steps of 16
//   out = bf16(O * (1 / l)), one IEEE reciprocal per query.
// Nothing in that chain depends on which other queries share the launch: a workgroup holds the
// queries of 32/GROUP * 4 consecutive tokens for the GROUP query heads of one key/value head, every
// MFMA row or column belongs to one query, and a block that lies wholly beyond a query's position is
// an exact no-op for it (a = 1, p_j = 0), so whether a wave computes or skips it gives the same bits.
// A one-token decode step and a full-sequence pass therefore agree bit for bit.
#include "ix_common.h"
#include "../../include/isoexec_hip.h"

typedef __attribute__((ext_vector_type(8))) __bf16 ix_bf16x8;
typedef __attribute__((ext_vector_type(16))) float ix_f32x16;

#define IX_ATTN_D 128
#define IX_ATTN_BN 32
#define IX_ATTN_KP (IX_ATTN_D * 2 + 16)  // bytes per key row of the K tile
// Bytes per key row of the V tile. 80 dwords: the four key rows that one transpose read of 32 lanes touches
// (16 dwords each) then fall on four disjoint quarters of the 64 banks.
#define IX_ATTN_VP (IX_ATTN_D * 2 + 64)

typedef __attribute__((ext_vector_type(4))) short ix_s16x4;

// A workgroup of NT threads stages a block of 32 keys x 128 d of K and of V: 512 16-byte chunks each, CPT per
// thread. Chunk c = j * NT + tid holds d (c % 16) * 8 .. +8 of key c / 16; both tiles keep the key-major layout
// of memory, so a chunk is one 16-byte store.
// Named members, not arrays: the stages must live in registers whatever the unroller decides.
struct IxAttnStage {
  uint4 k0, v0, k1, v1;
};

template <int NT>
__device__ __forceinline__ void ix_attn_fetch1(uint4& kk, uint4& vv, int j, const bf16_t* __restrict__ kbase,
                                               const bf16_t* __restrict__ vbase, long kv_pitch, int kb, int key_limit) {
  const int c = j * NT + threadIdx.x;
  const int key = kb * IX_ATTN_BN + (c >> 4);
  const int dch = (c & 15) * 8;
  kk = vv = make_uint4(0, 0, 0, 0);  // beyond the last key any query of this workgroup needs: zeros, nothing read
  if (key <= key_limit) {
    kk = *reinterpret_cast<const uint4*>(kbase + (long)key * kv_pitch + dch);
    vv = *reinterpret_cast<const uint4*>(vbase + (long)key * kv_pitch + dch);
  }
}

template <int CPT>
__device__ __forceinline__ void ix_attn_fetch(IxAttnStage& st, const bf16_t* __restrict__ kbase,
                                              const bf16_t* __restrict__ vbase, long kv_pitch, int kb, int key_limit) {
  ix_attn_fetch1<512 / CPT>(st.k0, st.v0, 0, kbase, vbase, kv_pitch, kb, key_limit);
  if (CPT > 1) ix_attn_fetch1<512 / CPT>(st.k1, st.v1, 1, kbase, vbase, kv_pitch, kb, key_limit);
}

template <int NT>
__device__ __forceinline__ void ix_attn_commit1(const uint4& kk, const uint4& vv, int j, char* ldsK, char* ldsV) {
  const int c = j * NT + threadIdx.x;
  const int key = c >> 4;
  const int dch = (c & 15) * 8;
  *reinterpret_cast<uint4*>(ldsK + key * IX_ATTN_KP + dch * 2) = kk;
  *reinterpret_cast<uint4*>(ldsV + key * IX_ATTN_VP + dch * 2) = vv;
}

template <int CPT>
__device__ __forceinline__ void ix_attn_commit(const IxAttnStage& st, char* ldsK, char* ldsV) {
  ix_attn_commit1<512 / CPT>(st.k0, st.v0, 0, ldsK, ldsV);
  if (CPT > 1) ix_attn_commit1<512 / CPT>(st.k1, st.v1, 1, ldsK, ldsV);
}

// One block of 32 keys for the 32 queries of a wave. Lane (qc = lane % 32, hf = lane / 32) holds
// query qc; of the block's keys it holds, in register i, key (i/4)*8 + hf*4 + i%4.
__device__ __forceinline__ void ix_attn_block(const char* ldsK, const char* ldsV, const ix_bf16x8 (&qf)[8],
                                              ix_f32x16 (&O)[4], float& m, float& l, int kb, int qpos, int min_qpos,
                                              float c) {
  const int lane = threadIdx.x & 63;
  const int qc = lane & 31, hf = lane >> 5;
  ix_f32x16 sacc;
#pragma unroll
  for (int i = 0; i < 16; ++i) sacc[i] = 0.0f;
#pragma unroll
  for (int s = 0; s < 8; ++s) {
    const ix_bf16x8 kf = *reinterpret_cast<const ix_bf16x8*>(ldsK + qc * IX_ATTN_KP + (16 * s + hf * 8) * 2);
    sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[s], sacc, 0, 0, 0);
  }
  // A block that ends at or before the wave's smallest position needs no mask (wave-uniform test).
  const bool need_mask = kb * IX_ATTN_BN + IX_ATTN_BN - 1 > min_qpos;
  if (need_mask) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int key = kb * IX_ATTN_BN + (i >> 2) * 8 + hf * 4 + (i & 3);
      sacc[i] = key <= qpos ? sacc[i] : IX_NEG_INF;
    }
  }
  float bm = sacc[0];
#pragma unroll
  for (int i = 1; i < 16; ++i) bm = fmaxf(bm, sacc[i]);
  bm = fmaxf(bm, __shfl_xor(bm, 32, IX_WAVE));
  const float m_new = fmaxf(m, bm);
  const float alpha = ix_exp2((m - m_new) * c);
  const float mc = -(m_new * c);
  float p[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) p[i] = ix_exp2(__builtin_fmaf(sacc[i], c, mc));
  const float pa[8] = {p[0], p[1], p[2], p[3], p[4], p[5], p[6], p[7]};
  const float pb[8] = {p[8], p[9], p[10], p[11], p[12], p[13], p[14], p[15]};
  const float mine = ix_tree8(pa) + ix_tree8(pb);
  const float other = __shfl_xor(mine, 32, IX_WAVE);
  const float tot = hf ? other + mine : mine + other;  // (half 0) + (half 1) on both lanes
  l = l * alpha + tot;
  m = m_new;
  // x * 1.0f is x: when no query of the wave moved its maximum, the rescale is skipped for all of them.
  const bool rescale = __any(alpha != 1.0f);
  ix_bf16x8 pf[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) w[j] = ix_pack_bf2_hw(p[8 * s + 2 * j], p[8 * s + 2 * j + 1]);
    pf[s] = *reinterpret_cast<const ix_bf16x8*>(w);
  }
  // this lane's address inside the 4 key x 16 d patch its group of 16 lanes transposes
  const char* vsrc = ldsV + (hf * 4 + ((lane & 15) >> 2)) * IX_ATTN_VP + (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;
#pragma unroll
  for (int dt = 0; dt < 4; ++dt) {
    if (rescale) {
#pragma unroll
      for (int i = 0; i < 16; ++i) O[dt][i] = O[dt][i] * alpha;
    }
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      // The lane needs V[key][d = 32 dt + qc] for keys 16 s + hf * 4 + 0..3 and those 8 further on. A transpose
      // read works in groups of 16 lanes: lane i of a group receives, as element e, element i % 4 of the 8 bytes
      // that lane 4 e + i / 4 of the group addressed. With lane j addressing key j / 4, d 4 * (j % 4) .. +4 of the
      // group's 4 key x 16 d patch, lane i ends up with keys 0..3 at d = i.
      typedef __attribute__((address_space(3))) ix_s16x4 lds_s16x4;
      const char* src = vsrc + (16 * s) * IX_ATTN_VP + 64 * dt;
      const ix_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(src));
      const ix_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(src + 8 * IX_ATTN_VP));
      const ix_s16x4 w[2] = {lo, hi};
      const ix_bf16x8 vf = *reinterpret_cast<const ix_bf16x8*>(w);
      O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[s], O[dt], 0, 0, 0);
    }
  }
}

// NW waves per workgroup (4 or 8): NW * 32 / GROUP consecutive tokens share each staged key block, so a larger
// workgroup pulls fewer key/value bytes per query; which queries share a workgroup never reaches the arithmetic.
template <int GROUP, int NW>
__global__ __launch_bounds__(NW * 64) void k_attn_varlen(const bf16_t* __restrict__ q, long q_pitch,
                                                     const bf16_t* __restrict__ k, const bf16_t* __restrict__ v,
                                                     long kv_pitch, bf16_t* __restrict__ o,
                                                     const int* __restrict__ cu_q, const long* __restrict__ kv_start,
                                                     const int* __restrict__ q_pos0, int HQ, float scale) {
  constexpr int TOK_W = 32 / GROUP;   // tokens per wave
  constexpr int TOK_WG = NW * TOK_W;  // tokens per workgroup
  constexpr int CPT = 512 / (NW * 64);
  // two LDS copies of the key/value block: block kb+1 is written while block kb is still being read
  __shared__ __attribute__((aligned(16))) char ldsK[2][IX_ATTN_BN * IX_ATTN_KP];
  __shared__ __attribute__((aligned(16))) char ldsV[2][IX_ATTN_BN * IX_ATTN_VP];
  const int n = blockIdx.y, g = blockIdx.z;
  const int qb = cu_q[n];
  const int len = cu_q[n + 1] - qb;
  const int t0 = ((int)gridDim.x - 1 - (int)blockIdx.x) * TOK_WG;  // long tiles first
  if (t0 >= len) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int qc = lane & 31, hf = lane >> 5;
  const int rel = t0 + wave * TOK_W + qc / GROUP;
  const int h = g * GROUP + qc % GROUP;
  const bool live = rel < len;
  const int p0 = q_pos0 ? q_pos0[n] : 0;
  bf16_t* orow = o + ((long)(qb + rel) * HQ + h) * IX_ATTN_D;
  if (p0 < 0) {  // null lane: defined output, nothing read
    if (live) {
      for (int dt = 0; dt < 4; ++dt)
        for (int i = 0; i < 16; ++i) orow[32 * dt + (i >> 2) * 8 + hf * 4 + (i & 3)] = 0;
    }
    return;
  }
  // A padding column carries a zero query and no causal limit: finite scores, result discarded.
  const int qpos = live ? p0 + rel : 0x7fffffff;
  ix_bf16x8 qf[8];
  {
    const bf16_t* qrow = q + (long)(qb + (live ? rel : 0)) * q_pitch + (long)h * IX_ATTN_D;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      uint4 w = make_uint4(0, 0, 0, 0);
      if (live) w = *reinterpret_cast<const uint4*>(qrow + 16 * s + hf * 8);
      qf[s] = *reinterpret_cast<const ix_bf16x8*>(&w);
    }
  }
  const int last_tok = min(len, t0 + TOK_WG) - 1;
  const int key_limit = p0 + last_tok;                       // last key any query here may see
  const int nblocks = key_limit / IX_ATTN_BN + 1;
  const int wave_last = min(len - 1, t0 + wave * TOK_W + TOK_W - 1);
  const int wave_blocks = wave_last >= t0 + wave * TOK_W ? (p0 + wave_last) / IX_ATTN_BN + 1 : 0;
  // smallest position among the wave's live queries (its first token); padding columns have no limit
  const int wave_min_qpos = p0 + t0 + wave * TOK_W;
  const long kv0 = kv_start[n];
  const bf16_t* kbase = k + kv0 * kv_pitch + (long)g * IX_ATTN_D;
  const bf16_t* vbase = v + kv0 * kv_pitch + (long)g * IX_ATTN_D;

  ix_f32x16 O[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) O[dt][i] = 0.0f;
  float m = IX_NEG_INF, l = 0.0f;
  const float c = scale * IX_LOG2E;

  // Two register stages: while block kb is multiplied, block kb+1 sits in LDS and blocks kb+2 and kb+3 are
  // in flight from memory. One barrier per block.
  IxAttnStage sa, sb;
  ix_attn_fetch<CPT>(sa, kbase, vbase, kv_pitch, 0, key_limit);
  if (nblocks > 1) ix_attn_fetch<CPT>(sb, kbase, vbase, kv_pitch, 1, key_limit);
  ix_attn_commit<CPT>(sa, ldsK[0], ldsV[0]);
  if (nblocks > 2) ix_attn_fetch<CPT>(sa, kbase, vbase, kv_pitch, 2, key_limit);
  __syncthreads();
  for (int kb = 0; kb < nblocks; kb += 2) {
    // even block: compute from copy 0; publish block kb+1 (stage b) into copy 1; refill stage b with kb+3
    if (kb < wave_blocks) ix_attn_block(ldsK[0], ldsV[0], qf, O, m, l, kb, qpos, wave_min_qpos, c);
    if (kb + 1 < nblocks) ix_attn_commit<CPT>(sb, ldsK[1], ldsV[1]);
    if (kb + 3 < nblocks) ix_attn_fetch<CPT>(sb, kbase, vbase, kv_pitch, kb + 3, key_limit);
    __syncthreads();
    if (kb + 1 >= nblocks) break;
    // odd block: compute from copy 1; publish block kb+2 (stage a) into copy 0; refill stage a with kb+4
    if (kb + 1 < wave_blocks) ix_attn_block(ldsK[1], ldsV[1], qf, O, m, l, kb + 1, qpos, wave_min_qpos, c);
    if (kb + 2 < nblocks) ix_attn_commit<CPT>(sa, ldsK[0], ldsV[0]);
    if (kb + 4 < nblocks) ix_attn_fetch<CPT>(sa, kbase, vbase, kv_pitch, kb + 4, key_limit);
    __syncthreads();
  }
  if (live) {
    const float inv = 1.0f / l;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) {
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int d = 32 * dt + i4 * 8 + hf * 4;
        uint2 w;
        w.x = ix_pack_bf2_hw(O[dt][4 * i4 + 0] * inv, O[dt][4 * i4 + 1] * inv);
        w.y = ix_pack_bf2_hw(O[dt][4 * i4 + 2] * inv, O[dt][4 * i4 + 3] * inv);
        *reinterpret_cast<uint2*>(orow + d) = w;
      }
    }
  }
}

extern "C" int ix_attn_varlen(const void* q, long q_pitch, const void* k, const void* v, long kv_pitch, void* o,
                              const int* cu_q, const long* kv_start, const int* q_pos0, long N, long max_q_len,
                              long HQ, long HKV, long D, float scale, void* stream) {
  if (!q || !k || !v || !o || !cu_q || !kv_start) return IX_ERR_ARG;
  if (N < 0 || max_q_len < 0 || HQ <= 0 || HKV <= 0 || HQ % HKV != 0) return IX_ERR_ARG;
  if (!(scale > 0.0f) || scale > 3.0e38f) return IX_ERR_ARG;  // the running maximum is kept unscaled
  if (D != IX_ATTN_D) return IX_DECLINED;
  if (q_pitch % 8 != 0 || kv_pitch % 8 != 0 || !ix_aligned(q, 16) || !ix_aligned(k, 16) || !ix_aligned(v, 16) ||
      !ix_aligned(o, 8))
    return IX_DECLINED;
  if (N == 0 || max_q_len == 0) return IX_OK;
  if (N > 65535 || HKV > 65535) return IX_DECLINED;
  const int group = (int)(HQ / HKV);
  hipStream_t st = (hipStream_t)stream;
#define IX_ATTN_LAUNCH_NW(G, NWV)                                                                               \
  {                                                                                                             \
    const long tok_wg = NWV * (32 / G);                                                                         \
    const long tiles = (max_q_len + tok_wg - 1) / tok_wg;                                                       \
    if (tiles > 0x7fffffffL) return IX_DECLINED;                                                                \
    hipLaunchKernelGGL((k_attn_varlen<G, NWV>), dim3((unsigned)tiles, (unsigned)N, (unsigned)HKV),              \
                       dim3(NWV * 64), 0, st, (const bf16_t*)q, q_pitch, (const bf16_t*)k, (const bf16_t*)v,    \
                       kv_pitch, (bf16_t*)o, cu_q, kv_start, q_pos0, (int)HQ, scale);                           \
  }
#define IX_ATTN_LAUNCH(G)                                                                                       \
  case G:                                                                                                       \
    if (big) IX_ATTN_LAUNCH_NW(G, 8) else IX_ATTN_LAUNCH_NW(G, 4)                                               \
    break;
  // long query runs (prefill) use eight waves per workgroup, short ones (decode, small chunks) four
  const bool big = max_q_len >= 8 * (32 / group);
  switch (group) {
    IX_ATTN_LAUNCH(1)
    IX_ATTN_LAUNCH(2)
    IX_ATTN_LAUNCH(4)
    IX_ATTN_LAUNCH(8)
    IX_ATTN_LAUNCH(16)
    IX_ATTN_LAUNCH(32)
    default:
      return IX_DECLINED;
  }
#undef IX_ATTN_LAUNCH_NW
#undef IX_ATTN_LAUNCH
  return ix_launch_status();
}

// ---- rotary position embedding -------------------------------------------------------------------
// x [tokens, heads, D] (token pitch x_pitch), rotated in place over its first R lanes:
//   y[d]       = bf16( bf16(x[d]       * cos[d])       + bf16((-x[d + R/2]) * sin[d]) )        d <  R/2
//   y[d + R/2] = bf16( bf16(x[d + R/2] * cos[d + R/2]) + bf16(  x[d]        * sin[d + R/2]) )
// Three bf16 rounds per output, each product and the sum computed in fp32. cos/sin: [positions, R]
// bf16 tables; pos[t] picks the row.
__global__ __launch_bounds__(256) void k_rope(bf16_t* __restrict__ x, long x_pitch, const bf16_t* __restrict__ cs,
                                              const bf16_t* __restrict__ sn, const int* __restrict__ pos, long total,
                                              int heads, int D, int R) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int half = R >> 1;
  const int d = (int)(i % half);
  const long th = i / half;
  const int hd = (int)(th % heads);
  const long t = th / heads;
  bf16_t* row = x + t * x_pitch + (long)hd * D;
  const long tab = (long)pos[t] * R;
  const float a = ix_bf2f(row[d]), b = ix_bf2f(row[d + half]);
  const float c0 = ix_bf2f(cs[tab + d]), c1 = ix_bf2f(cs[tab + d + half]);
  const float s0 = ix_bf2f(sn[tab + d]), s1 = ix_bf2f(sn[tab + d + half]);
  const float lo = ix_rbf(a * c0) + ix_rbf((b * -1.0f) * s0);
  const float hi = ix_rbf(b * c1) + ix_rbf(a * s1);
  row[d] = ix_f2bf(lo);
  row[d + half] = ix_f2bf(hi);
}

extern "C" int ix_rope_inplace(void* x, long x_pitch, const void* cos_table, const void* sin_table,
                               const int* positions, long tokens, long heads, long D, long R, void* stream) {
  if (!x || !cos_table || !sin_table || !positions || tokens < 0 || heads <= 0 || D <= 0) return IX_ERR_ARG;
  if (R <= 0 || R % 2 != 0 || R > D) return IX_ERR_ARG;
  const long total = tokens * heads * (R / 2);
  if (total == 0) return IX_OK;
  const long grid = (total + 255) / 256;
  if (grid > (1L << 24)) return IX_DECLINED;
  hipLaunchKernelGGL(k_rope, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, (bf16_t*)x, x_pitch,
                     (const bf16_t*)cos_table, (const bf16_t*)sin_table, positions, total, (int)heads, (int)D, (int)R);
  return ix_launch_status();
}
