// Causal grouped-query attention over packed sequences with ONE walk of the keys per query, and
// rotary position embedding.
//
// The canonical function, per (query token at absolute position p, query head h):
//   keys 0..p of the query's own sequence are walked in blocks of 32, block b = keys [32b, 32b+32);
//   with c = scale * log2(e) (one fp32 product), per block:
//               s_j  = q . k_j                           bf16 MFMA, fp32 accumulate, d in 8 steps of 16
//               s_j  = -inf for j > p
//               b    = max_j s_j                         the block's maximum, UNSCALED (scale > 0)
//               m'   = b if (b - m) * c > 8 else m       the reference point moves only when the maximum has
//                                                        grown by more than 2^8; m starts at -inf
//               a    = exp2((m - m') * c)                exactly 1 when the reference did not move
//               p_j  = exp2(fma(s_j, c, -(m' * c)))      one fused multiply-add per score; p_j <= 2^8 (1 + eps)
//               l_h  = l_h * a + sum of p_j over the 16 keys of half h (h = (j / 4) % 2), as two 8-trees
//               O    = O * a + sum_j bf16(p_j) * v_j     bf16 MFMA, fp32 accumulate, keys in 2 steps of 16
//   out = bf16(O * (1 / (l_0 + l_1))), one IEEE reciprocal per query.
// Nothing in that chain depends on which other queries share the launch: a workgroup holds the
// queries of 32/GROUP * 4 consecutive tokens for the GROUP query heads of one key/value head, every
// MFMA row or column belongs to one query, and a block that lies wholly beyond a query's position is
// an exact no-op for it (b = -inf, a = 1, p_j = 0), so whether a wave computes or skips it gives the same bits.
// A one-token decode step and a full-sequence pass therefore agree bit for bit.
#include "ix_gemm_core.h"
#include "../../include/isoexec_hip.h"

#define IX_ATTN_D 128
#define IX_ATTN_BN 32
#define IX_ATTN_ROW (IX_ATTN_D * 2)                 // bytes per key row of a tile
#define IX_ATTN_TILE (IX_ATTN_BN * IX_ATTN_ROW)     // one K or V tile of a block: 8 KiB
#define IX_ATTN_STAGE (2 * IX_ATTN_TILE)            // K tile, then V tile
#ifndef IX_ATTN_STAGES
#define IX_ATTN_STAGES 4  // ring depth: 64 KiB of LDS per workgroup
#endif

typedef __attribute__((ext_vector_type(4))) short ix_s16x4;
typedef __attribute__((address_space(3))) ix_s16x4 ix_lds_s16x4;

// Key/value blocks go memory -> LDS directly (16 bytes per lane, no registers) into a ring of S stages. Both
// tiles keep memory's key-major layout, 256 bytes per key, with the 16-byte chunks of a row permuted:
//   K: chunk c of key r sits at slot c ^ (r & 15)         a fragment read takes one chunk of 32 consecutive keys
//   V: chunk c of key r sits at slot c ^ ((r & 3) << 2)   a transpose read takes 4 chunks of 4 consecutive keys
// so that either read spreads over all LDS banks. A lane's LDS destination is fixed by its position in the
// wave (destination = base + 16 * lane), so the permutation is applied to the memory address it fetches.
template <int NT>
struct IxAttnFetch {
  static constexpr int CPT = 512 / NT;  // chunks per thread per tile
  uint32_t voff_k[CPT], voff_v[CPT];    // byte offsets inside a block: key row * pitch + chunk * 16
  uint32_t lds0;                        // LDS address of this wave's first destination in stage 0
  __device__ __forceinline__ void init(const char* lds, uint32_t pitch_bytes) {
    const int wave = threadIdx.x >> 6;
#pragma unroll
    for (int j = 0; j < CPT; ++j) {
      const int q = j * NT + threadIdx.x;
      const int row = q >> 4, slot = q & 15;
      voff_k[j] = (uint32_t)row * pitch_bytes + (uint32_t)((slot ^ (row & 15)) << 4);
      voff_v[j] = (uint32_t)row * pitch_bytes + (uint32_t)((slot ^ ((row & 3) << 2)) << 4);
    }
    lds0 = __builtin_amdgcn_readfirstlane(ix_lds_addr(lds) + wave * 1024);
  }
  // Block kb of the sequence into ring stage `stage`. Keys beyond key_limit lie outside the buffer range and
  // arrive as zeros; a block wholly beyond it is all zeros and touches no memory.
  __device__ __forceinline__ void issue(const bf16_t* kbase, const bf16_t* vbase, long kv_pitch, int kb, int stage,
                                        int key_limit) const {
    const int rows = min(IX_ATTN_BN, key_limit + 1 - kb * IX_ATTN_BN);
    const uint32_t bytes = rows > 0 ? (uint32_t)(rows - 1) * (uint32_t)(kv_pitch * 2) + IX_ATTN_ROW : 0u;
    const long first = rows > 0 ? (long)kb * IX_ATTN_BN * kv_pitch : 0;
    const ix_rsrc_t rk = ix_make_rsrc(kbase + first, bytes);
    const ix_rsrc_t rv = ix_make_rsrc(vbase + first, bytes);
    const uint32_t dst = __builtin_amdgcn_readfirstlane(lds0 + stage * IX_ATTN_STAGE);
#pragma unroll
    for (int j = 0; j < CPT; ++j) {
      ix_dma16(rk, dst + j * NT * 16, voff_k[j], 0);
      ix_dma16(rv, dst + IX_ATTN_TILE + j * NT * 16, voff_v[j], 0);
    }
  }
};

// Lane (qc = lane % 32, hf = lane / 32) holds query qc. Of a block's 32 scores it holds, in register i, the
// one of key (i/4)*8 + hf*4 + i%4.
struct IxAttnLane {
  uint32_t k_addr;  // LDS byte offset in a K tile of key row qc, chunk hf (step s: XOR with s << 5)
  uint32_t v_addr;  // LDS byte offset in a V tile of this lane's 8 bytes of the first transpose patch
  __device__ __forceinline__ void init() {
    const int lane = threadIdx.x & 63;
    const int qc = lane & 31, hf = lane >> 5;
    k_addr = qc * IX_ATTN_ROW + ((hf ^ (qc & 15)) << 4);
    // A transpose read works in groups of 16 lanes: lane i of a group receives, as element e, element i % 4 of
    // the 8 bytes that lane 4 e + i / 4 addressed. With lane j addressing key j / 4, d 4 (j % 4) .. +4 of the
    // group's 4 key x 16 d patch, lane i ends up with keys 0..3 at d = i. The group (lane / 16) % 2 takes the
    // d half, hf the key quad.
    const int rl = (lane >> 2) & 3;                             // key within the quad
    const int cl = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);   // 16-byte chunk within the 64 bytes of a d tile
    v_addr = (hf * 4 + rl) * IX_ATTN_ROW + (((rl << 2) | cl) << 4) + 8 * (lane & 1);
  }
};

// The K fragments of one block: kf[s] holds d 16 s + hf * 8 .. +8 of key qc.
__device__ __forceinline__ void ix_attn_keys(const char* tileK, const IxAttnLane& ln, ix_bf16x8 (&kf)[8]) {
#pragma unroll
  for (int s = 0; s < 8; ++s) kf[s] = *reinterpret_cast<const ix_bf16x8*>(tileK + (ln.k_addr ^ (s << 5)));
}

// S^T = K Q^T for one block: 8 steps of 16 along d.
__device__ __forceinline__ void ix_attn_scores(const ix_bf16x8 (&kf)[8], const ix_bf16x8 (&qf)[8], ix_f32x16& sacc) {
#pragma unroll
  for (int i = 0; i < 16; ++i) sacc[i] = 0.0f;
#pragma unroll
  for (int s = 0; s < 8; ++s) sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[s], qf[s], sacc, 0, 0, 0);
}

// The V^T fragments of one block: vf[dt][s] holds, for d = 32 dt + qc, keys 16 s + hf * 4 + 0..3 and those 8
// further on -- the same key slots the probabilities of this lane sit in.
__device__ __forceinline__ void ix_attn_values(const char* tileV, const IxAttnLane& ln, ix_bf16x8 (&vf)[4][2]) {
#pragma unroll
  for (int dt = 0; dt < 4; ++dt) {
    const char* src = tileV + (ln.v_addr ^ (dt << 6));
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const ix_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((ix_lds_s16x4*)(src + (16 * s) * IX_ATTN_ROW));
      const ix_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((ix_lds_s16x4*)(src + (16 * s + 8) * IX_ATTN_ROW));
      const ix_s16x4 w[2] = {lo, hi};
      vf[dt][s] = *reinterpret_cast<const ix_bf16x8*>(w);
    }
  }
}

// max(x of this lane, x of the lane 32 away) without a trip through LDS.
__device__ __forceinline__ float ix_attn_max_halves(float x) {
  const uint32_t u = __float_as_uint(x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// One step of the skewed loop. The softmax arithmetic of block kb needs only registers (its scores were
// computed a step earlier), so it runs while the fragments of V (block kb) and of K (block kb + 1, from the
// next ring stage) travel from LDS; then O^T += V^T P^T and the scores of block kb + 1. Past the wave's last
// block those scores are computed from whatever the stage holds and never used.
// MASK: the block reaches beyond the position of some query of the wave.
// l is this HALF's share of the denominator: the 16 key slots the lane holds; the halves meet at the end.
#define IX_ATTN_LAZY 8.0f
template <bool MASK>
__device__ __forceinline__ void ix_attn_step(const char* stage, const char* stage_next, const IxAttnLane& ln,
                                             const ix_bf16x8 (&qf)[8], ix_f32x16& sacc, ix_f32x16 (&O)[4], float& m,
                                             float& l, int kb, int qpos, float c) {
  const int hf = (threadIdx.x & 63) >> 5;
  ix_bf16x8 vf[4][2];
  ix_attn_values(stage + IX_ATTN_TILE, ln, vf);
  ix_bf16x8 kf[8];
  ix_attn_keys(stage_next, ln, kf);
  if (MASK) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int key = kb * IX_ATTN_BN + (i >> 2) * 8 + hf * 4 + (i & 3);
      sacc[i] = key <= qpos ? sacc[i] : IX_NEG_INF;
    }
  }
  float bm = sacc[0];
#pragma unroll
  for (int i = 1; i < 16; ++i) bm = fmaxf(bm, sacc[i]);
  bm = ix_attn_max_halves(bm);
  const float m_new = (bm - m) * c > IX_ATTN_LAZY ? bm : m;
  const float alpha = ix_exp2((m - m_new) * c);
  const float mc = -(m_new * c);
  float p[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) p[i] = ix_exp2(__builtin_fmaf(sacc[i], c, mc));
  const float pa[8] = {p[0], p[1], p[2], p[3], p[4], p[5], p[6], p[7]};
  const float pb[8] = {p[8], p[9], p[10], p[11], p[12], p[13], p[14], p[15]};
  l = l * alpha + (ix_tree8(pa) + ix_tree8(pb));
  m = m_new;
  ix_bf16x8 pf[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) w[j] = ix_pack_bf2_hw(p[8 * s + 2 * j], p[8 * s + 2 * j + 1]);
    pf[s] = *reinterpret_cast<const ix_bf16x8*>(w);
  }
  // x * 1.0f is x: when no query of the wave moved its reference, the rescale is skipped for all of them.
  if (__any(alpha != 1.0f)) {
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) O[dt][i] = O[dt][i] * alpha;
  }
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[dt][s], pf[s], O[dt], 0, 0, 0);
  ix_attn_scores(kf, qf, sacc);
}

// NW waves per workgroup: NW * 32 / GROUP consecutive tokens share each staged key block; which queries share a
// workgroup never reaches the arithmetic. Two workgroups per CU (register limit below).
// Inside a wave the loop is skewed by one block: while block kb goes through its softmax, the scores of block
// kb + 1 are already in the matrix pipeline.
template <int GROUP, int NW, int S>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void k_attn_varlen(const bf16_t* __restrict__ q, long q_pitch,
                                                     const bf16_t* __restrict__ k, const bf16_t* __restrict__ v,
                                                     long kv_pitch, bf16_t* __restrict__ o,
                                                     const int* __restrict__ cu_q, const long* __restrict__ kv_start,
                                                     const int* __restrict__ q_pos0, int HQ, float scale,
                                                     int n_seq, int n_kvh, int tiles) {
  constexpr int TOK_W = 32 / GROUP;   // tokens per wave
  constexpr int TOK_WG = NW * TOK_W;  // tokens per workgroup
  constexpr int NT = NW * 64;
  constexpr int CPT = 512 / NT;
  static_assert(S >= 3, "the ring holds the block being read, the next one and at least one in flight");
  extern __shared__ __align__(16) char ix_attn_lds[];
  // Workgroup -> (query tile, sequence, key/value head). Hardware deals consecutive workgroup ids to the 8 XCDs
  // round-robin and each XCD has its own L2, so all query tiles of one (sequence, head) pair go to one XCD: its
  // keys and values are fetched from memory by one L2 and then shared by the pair's tiles.
  // The grid is 8 * ceil(pairs / 8) * tiles workgroups: XCD x takes the pairs x, x + 8, ...
  const int pairs = n_seq * n_kvh;
  const int xcd = (int)(blockIdx.x & 7);
  const int idx = (int)(blockIdx.x >> 3);
  const int slot = idx / tiles, tile = idx - slot * tiles;
  const int pair = slot * 8 + xcd;
  if (pair >= pairs) return;
  const int n = pair % n_seq, g = pair / n_seq;
  const int qb = cu_q[n];
  const int len = cu_q[n + 1] - qb;
  const int t0 = (tiles - 1 - tile) * TOK_WG;  // long tiles first
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
  // A block that ends at or before the smallest position among the wave's live queries (its first token; padding
  // columns have no limit) needs no mask: blocks below first_masked.
  const int first_masked = (p0 + t0 + wave * TOK_W + 1) / IX_ATTN_BN;
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

  IxAttnFetch<NT> fetch;
  fetch.init(ix_attn_lds, (uint32_t)(kv_pitch * 2));
  IxAttnLane ln;
  ln.init();
  // The q loads above are the only vector-memory operations the compiler counts; they have been consumed
  // (converted into qf) before the first wait below is trusted to speak of the ring alone.
  __builtin_amdgcn_s_waitcnt(IX_VMCNT(0));
#pragma unroll
  for (int b = 0; b < S - 1; ++b) fetch.issue(kbase, vbase, kv_pitch, b, b, key_limit);
  __builtin_amdgcn_s_waitcnt(IX_VMCNT((S - 2) * 2 * CPT));  // block 0 has landed
  __syncthreads();
  ix_f32x16 sacc;
  if (wave_blocks > 0) {
    ix_bf16x8 kf[8];
    ix_attn_keys(ix_attn_lds, ln, kf);
    ix_attn_scores(kf, qf, sacc);
  }
  int st = 0;  // ring stage of block kb
  for (int kb = 0; kb < nblocks; ++kb) {
    // Blocks 0 .. kb+S-2 have been issued; all but the newest S-3 of them, so blocks up to kb+1, have landed for
    // this thread after the wait and for every thread after the barrier. The barrier also says that every wave
    // is done with block kb-1, whose stage the next fetch overwrites.
    __builtin_amdgcn_s_waitcnt(IX_VMCNT((S - 3) * 2 * CPT));
    __syncthreads();
    const int st_free = st == 0 ? S - 1 : st - 1;
    const int st_next = st == S - 1 ? 0 : st + 1;
    fetch.issue(kbase, vbase, kv_pitch, kb + S - 1, st_free, key_limit);
    if (kb < wave_blocks) {
      const char* cur = ix_attn_lds + st * IX_ATTN_STAGE;
      const char* nxt = ix_attn_lds + st_next * IX_ATTN_STAGE;
      if (kb < first_masked)
        ix_attn_step<false>(cur, nxt, ln, qf, sacc, O, m, l, kb, qpos, c);
      else
        ix_attn_step<true>(cur, nxt, ln, qf, sacc, O, m, l, kb, qpos, c);
    }
    st = st_next;
  }
  __builtin_amdgcn_s_waitcnt(IX_VMCNT(0));  // nothing may still be on its way into LDS when the wave ends
  // the denominator: (half 0's share) + (half 1's share), in that order on both lanes
  const float l_other = __shfl_xor(l, 32, IX_WAVE);
  l = hf ? l_other + l : l + l_other;
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

template <int GROUP, int NW, int S>
static int ix_attn_launch(const void* q, long q_pitch, const void* k, const void* v, long kv_pitch, void* o,
                          const int* cu_q, const long* kv_start, const int* q_pos0, long N, long max_q_len, long HQ,
                          long HKV, float scale, hipStream_t st) {
  constexpr int LDS = S * IX_ATTN_STAGE;
  auto kern = k_attn_varlen<GROUP, NW, S>;
  static bool attr_set = false;  // per instantiation
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS) != hipSuccess)
      return IX_ERR_LAUNCH;
    attr_set = true;
  }
  const long tok_wg = NW * (32 / GROUP);
  const long tiles = (max_q_len + tok_wg - 1) / tok_wg;
  if (tiles > 0x7fffffffL) return IX_DECLINED;
  const long grid = 8 * ((N * HKV + 7) / 8) * tiles;
  if (grid > 0x7fffffffL) return IX_DECLINED;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NW * 64), LDS, st, (const bf16_t*)q, q_pitch,
                     (const bf16_t*)k, (const bf16_t*)v, kv_pitch, (bf16_t*)o, cu_q, kv_start, q_pos0, (int)HQ, scale,
                     (int)N, (int)HKV, (int)tiles);
  return ix_launch_status();
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
  if (kv_pitch >= (1L << 26)) return IX_DECLINED;  // a block's byte range must fit the 32-bit buffer size
  const int group = (int)(HQ / HKV);
  hipStream_t st = (hipStream_t)stream;
  // Four waves per workgroup and at most 256 registers per wave: two workgroups share a CU, each behind its own
  // barrier, so one's matrix work meets the other's softmax arithmetic (measured: an eight-wave workgroup, whose
  // two waves per SIMD stand behind the same barrier, is 4 % slower on long prefills although it stages half as
  // many key/value bytes per query; and a decode step runs 20-40 % faster with two workgroups per CU).
#define IX_ATTN_LAUNCH(G)                                                                                          \
  case G:                                                                                                          \
    return ix_attn_launch<G, 4, IX_ATTN_STAGES>(q, q_pitch, k, v, kv_pitch, o, cu_q, kv_start, q_pos0, N, max_q_len, \
                                                HQ, HKV, scale, st);
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
#undef IX_ATTN_LAUNCH
}

// ---- rotary position embedding -------------------------------------------------------------------
// x [tokens, heads, D] (token pitch x_pitch), rotated in place over its first R lanes:
//   y[d]       = bf16( bf16(x[d]       * cos[d])       + bf16((-x[d + R/2]) * sin[d]) )        d <  R/2
//   y[d + R/2] = bf16( bf16(x[d + R/2] * cos[d + R/2]) + bf16(  x[d]        * sin[d + R/2]) )
// Three bf16 rounds per output, each product and the sum computed in fp32. cos/sin: [positions, R]
// bf16 tables; pos[t] picks the row.
__global__ __launch_bounds__(256) void k_rope(bf16_t* __restrict__ x, long x_pitch, const bf16_t* __restrict__ cs,
                                              const bf16_t* __restrict__ sn, const int* __restrict__ pos, long total,
                                              int heads, int D, int R, int table_rows) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int half = R >> 1;
  const int d = (int)(i % half);
  const long th = i / half;
  const int hd = (int)(th % heads);
  const long t = th / heads;
  bf16_t* row = x + t * x_pitch + (long)hd * D;
  const int p = pos[t];
  if (p < 0 || p >= table_rows) {
    // a position the tables do not hold: no read past them, and a result nobody can mistake for a rotation
    row[d] = (bf16_t)0x7fc0;
    row[d + half] = (bf16_t)0x7fc0;
    return;
  }
  const long tab = (long)p * R;
  const float a = ix_bf2f(row[d]), b = ix_bf2f(row[d + half]);
  const float c0 = ix_bf2f(cs[tab + d]), c1 = ix_bf2f(cs[tab + d + half]);
  const float s0 = ix_bf2f(sn[tab + d]), s1 = ix_bf2f(sn[tab + d + half]);
  const float lo = ix_rbf(a * c0) + ix_rbf((b * -1.0f) * s0);
  const float hi = ix_rbf(b * c1) + ix_rbf(a * s1);
  row[d] = ix_f2bf(lo);
  row[d + half] = ix_f2bf(hi);
}

// The same rotation, eight pairs per thread: 16-byte accesses (two of x, four of the tables, two stores) instead of
// 2-byte ones, 32-bit index arithmetic. Every output is the expression of k_rope above, so which kernel runs cannot
// move a bit. Needs R / 2, D and the pitch to be multiples of 8 and 16-byte aligned operands.
__global__ __launch_bounds__(256) void k_rope8(bf16_t* __restrict__ x, long x_pitch, const bf16_t* __restrict__ cs,
                                               const bf16_t* __restrict__ sn, const int* __restrict__ pos,
                                               unsigned total, int heads, int D, int R, int table_rows) {
  const unsigned i = blockIdx.x * 256u + threadIdx.x;
  if (i >= total) return;
  const unsigned chunks = (unsigned)R >> 4;  // 8-pair chunks per head
  const unsigned c = i % chunks;
  const unsigned th = i / chunks;
  const unsigned hd = th % (unsigned)heads;
  const unsigned t = th / (unsigned)heads;
  const int half = R >> 1;
  bf16_t* row = x + (long)t * x_pitch + (long)hd * D + c * 8;
  const int p = pos[t];
  uint4 lo4, hi4;
  if (p < 0 || p >= table_rows) {
    lo4 = hi4 = make_uint4(0x7fc07fc0u, 0x7fc07fc0u, 0x7fc07fc0u, 0x7fc07fc0u);
  } else {
    const bf16_t* ct = cs + (long)p * R + c * 8;
    const bf16_t* st = sn + (long)p * R + c * 8;
    const uint4 a4 = *reinterpret_cast<const uint4*>(row), b4 = *reinterpret_cast<const uint4*>(row + half);
    const uint4 c0 = *reinterpret_cast<const uint4*>(ct), c1 = *reinterpret_cast<const uint4*>(ct + half);
    const uint4 s0 = *reinterpret_cast<const uint4*>(st), s1 = *reinterpret_cast<const uint4*>(st + half);
    const uint32_t* aw = &a4.x; const uint32_t* bw = &b4.x;
    const uint32_t* c0w = &c0.x; const uint32_t* c1w = &c1.x; const uint32_t* s0w = &s0.x; const uint32_t* s1w = &s1.x;
    uint32_t* low = &lo4.x; uint32_t* hiw = &hi4.x;
    // The products are rounded by the hardware pack-convert, two at a time (ix_rbf2_hw: k_rope's ix_rbf on everything but
    // a NaN, whose payload it keeps); a NaN stays a NaN through the add whatever its payload, and the sums are stored
    // with their NaNs made canonical (ix_pack_bf2_canon_hw), so the stored bits are k_rope's.
    auto lo16 = [](uint32_t u) { return __uint_as_float(u << 16); };
    auto hi16 = [](uint32_t u) { return __uint_as_float(u & 0xffff0000u); };
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float a0 = lo16(aw[w]), a1 = hi16(aw[w]), b0 = lo16(bw[w]), b1 = hi16(bw[w]);
      float t0, t1, u0, u1;
      ix_rbf2_hw(a0 * lo16(c0w[w]), a1 * hi16(c0w[w]), t0, t1);
      ix_rbf2_hw((b0 * -1.0f) * lo16(s0w[w]), (b1 * -1.0f) * hi16(s0w[w]), u0, u1);
      low[w] = ix_pack_bf2_canon_hw(t0 + u0, t1 + u1);
      ix_rbf2_hw(b0 * lo16(c1w[w]), b1 * hi16(c1w[w]), t0, t1);
      ix_rbf2_hw(a0 * lo16(s1w[w]), a1 * hi16(s1w[w]), u0, u1);
      hiw[w] = ix_pack_bf2_canon_hw(t0 + u0, t1 + u1);
    }
  }
  *reinterpret_cast<uint4*>(row) = lo4;
  *reinterpret_cast<uint4*>(row + half) = hi4;
}

extern "C" int ix_rope_inplace(void* x, long x_pitch, const void* cos_table, const void* sin_table, long table_rows,
                               const int* positions, long tokens, long heads, long D, long R, void* stream) {
  if (!x || !cos_table || !sin_table || !positions || tokens < 0 || heads <= 0 || D <= 0) return IX_ERR_ARG;
  if (table_rows <= 0 || table_rows > 0x7fffffffL) return IX_ERR_ARG;
  if (R <= 0 || R % 2 != 0 || R > D) return IX_ERR_ARG;
  const long total = tokens * heads * (R / 2);
  if (total == 0) return IX_OK;
  if (R % 16 == 0 && D % 8 == 0 && x_pitch % 8 == 0 && ix_aligned(x, 16) && ix_aligned(cos_table, 16) &&
      ix_aligned(sin_table, 16) && total / 8 < 0x7fffffffL) {
    const unsigned total8 = (unsigned)(total / 8);
    hipLaunchKernelGGL(k_rope8, dim3((total8 + 255u) / 256u), dim3(256), 0, (hipStream_t)stream, (bf16_t*)x, x_pitch,
                       (const bf16_t*)cos_table, (const bf16_t*)sin_table, positions, total8, (int)heads, (int)D, (int)R,
                       (int)table_rows);
    return ix_launch_status();
  }
  const long grid = (total + 255) / 256;
  if (grid > (1L << 24)) return IX_DECLINED;
  hipLaunchKernelGGL(k_rope, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, (bf16_t*)x, x_pitch,
                     (const bf16_t*)cos_table, (const bf16_t*)sin_table, positions, total, (int)heads, (int)D, (int)R,
                     (int)table_rows);
  return ix_launch_status();
}
