// Row-count-invariant log-softmax + target gather over a fixed-leaf exp-sum tree.
//
// Function computed per row (the expression tree of the reference's leaf_sum_exp /
// finalize_rows / full_row_logprobs, skyrl/backends/skyrl_train/isoexec/ops/logprobs/rowinv.py:136-245):
//   m      = max_j x[j]                                   (exact, order-free)
//   leaf_g = Kahan-fp32 sum over blocks b of  blocksum(g, b)      g = 0..G-1, L = V/G columns each
//   S      = balanced pairwise fold of the G leaves               (combine_order(G))
//   logp   = (x[target] - m) - log(S)        lse = m + log(S)
// blocksum(g, b) covers BLOCK = 4096 consecutive columns of leaf g (the last block masked):
//   column sums col[p] = sum over the 8 chunks c of term[c*512 + p], left to right, p = 0..511,
//   then the adjacent-pairwise tree over the 512 columns,
//   term[i] = exp2((x[i] - m) * log2(e)) for live columns and 0 for masked ones.
// Every quantity above depends only on (V, G) and the row's own values, never on the number
// of rows or on which launch shape ran, so a row's bits are the same at any row count.
//
// Two launch shapes evaluate that same function:
//   * rows >= IX_LP_SPLIT_BELOW : one 512-thread workgroup per row, one launch;
//   * fewer rows                : row split over many workgroups (partial max, block sums,
//                                 finalize) so a single decode row still fills the chip.
#include "ix_common.h"
#include "../../include/isoexec_hip.h"

#define IX_LP_BLOCK 4096
#define IX_LP_MAX_UNITS 4096  // G * ceil(L / BLOCK) a workgroup can hold in LDS
#define IX_LP_MAX_G 64
#define IX_LP_SPLIT_BELOW 192
#define IX_LP_SEG 8192  // columns per partial-max / full-row-write workgroup in the split shape

// Eight consecutive elements as they lie in memory (a 16-byte-aligned group of bf16, a 32-byte-aligned group of
// fp32): loading and widening are separate steps so that several loads can be in flight before the first is used.
template <typename T>
struct IxRaw8;
template <>
struct IxRaw8<bf16_t> {
  uint4 v;
  __device__ __forceinline__ void load(const bf16_t* __restrict__ p) { v = *reinterpret_cast<const uint4*>(p); }
  __device__ __forceinline__ void widen(float (&o)[8]) const { ix_unpack8(v, o); }
};
template <>
struct IxRaw8<float> {
  float4 a, b;
  __device__ __forceinline__ void load(const float* __restrict__ p) {
    a = *reinterpret_cast<const float4*>(p);
    b = *reinterpret_cast<const float4*>(p + 4);
  }
  __device__ __forceinline__ void widen(float (&o)[8]) const {
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
  }
};

// One wave sums one block. `blk` points at the block's first column, n_valid <= 4096 columns
// exist. Returns the block sum in every lane.
// `row_max()` yields the row maximum; it is called after the block's loads are issued, so a maximum that is itself
// read from memory does not put its latency in front of theirs.
template <typename T, typename MaxFn>
__device__ __forceinline__ float ix_block_expsum_with(const T* __restrict__ blk, int n_valid, const MaxFn& row_max,
                                                      bool vec, int lane) {
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (vec) {
    // vec implies that the leaf length is a multiple of 8, so a group of 8 columns is whole or absent. All eight
    // groups are requested before the first is used: a lane has eight independent loads in flight instead of one
    // (a load, its wait and its sum per group is bound by memory latency). An absent group reads the block's first
    // columns instead (no branch between the loads) and adds +0.0. The sums are the ones below: slot i adds its
    // groups in ascending c.
    IxRaw8<T> raw[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const int off = c * 512 + lane * 8;
      raw[c].load(blk + ((n_valid - off >= 8) ? off : 0));
    }
    __builtin_amdgcn_sched_barrier(0);  // the loads are issued back to back; widening waits with the sums
    const float m = row_max();
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const bool whole = n_valid - (c * 512 + lane * 8) >= 8;
      float x[8];
      raw[c].widen(x);
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = acc[i] + (whole ? ix_exp_fast(x[i] - m) : 0.0f);
    }
    return ix_lane_tree<64>(ix_tree8(acc));
  }
  const float m = row_max();
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    const int off = c * 512 + lane * 8;
    const int valid = n_valid - off;
    if (valid > 0) {  // a fully masked group adds +0.0 to every slot: a no-op on the bits
      float x[8];
      ix_load8(blk + off, valid, vec, 0.0f, x);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float t = (i < valid) ? ix_exp_fast(x[i] - m) : 0.0f;
        acc[i] = acc[i] + t;
      }
    }
  }
  return ix_lane_tree<64>(ix_tree8(acc));
}

template <typename T>
__device__ __forceinline__ float ix_block_expsum(const T* __restrict__ blk, int n_valid, float m, bool vec,
                                                 int lane) {
  return ix_block_expsum_with(blk, n_valid, [m]() { return m; }, vec, lane);
}

__device__ __forceinline__ float ix_kahan_blocks(const float* __restrict__ bsum, int nb) {
  float acc = 0.0f, comp = 0.0f;
  for (int b = 0; b < nb; ++b) {
    const float y = bsum[b] - comp;
    const float t = acc + y;
    comp = (t - acc) - y;
    acc = t;
  }
  return acc;
}

// In-place balanced fold; leaf[0] ends as the root. Stride doubling == combine_order(G) of
// skyrl/backends/skyrl_train/isoexec/ops/collectives/pik/plan.py:104-119.
__device__ __forceinline__ float ix_fold_leaves(float* leaf, int G) {
  for (int s = 1; s < G; s <<= 1)
    for (int i = 0; i + s < G; i += 2 * s) leaf[i] = leaf[i] + leaf[i + s];
  return leaf[0];
}

template <typename T>
__device__ __forceinline__ void ix_lp_emit(const T* __restrict__ xr, int V, float m, float log_s,
                                           const int64_t* __restrict__ target, long row, float* out_lp,
                                           float* out_lse) {
  if (out_lp) {
    const int64_t t = target[row];
    const bool valid = (t >= 0) && (t < (int64_t)V);
    float sampled = 0.0f;
    if (valid) {
      float o[8];
      ix_load8(xr + t, 1, false, 0.0f, o);
      sampled = o[0];
    }
    out_lp[row] = valid ? (sampled - m) - log_s : 0.0f;
  }
  if (out_lse) out_lse[row] = m + log_s;
}

// ---------------------------------------------------------------------------------------------
// Shape 1: one workgroup (8 waves) per row.
template <typename T>
__global__ __launch_bounds__(512) void k_lp_row(const T* __restrict__ x, long row_stride, int V, int G,
                                                const int64_t* __restrict__ target, float* __restrict__ out_lp,
                                                float* __restrict__ out_lse, float* __restrict__ out_full,
                                                long full_stride, int vec) {
  __shared__ float s_wmax[8];
  __shared__ float s_bsum[IX_LP_MAX_UNITS];
  __shared__ float s_leaf[IX_LP_MAX_G];
  __shared__ float s_fin[2];
  const long row = blockIdx.x;
  const T* xr = x + row * row_stride;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int L = V / G;
  const int NB = (L + IX_LP_BLOCK - 1) / IX_LP_BLOCK;

  float m = IX_NEG_INF;
  for (long off = (long)tid * 8; off < V; off += 512 * 8) {
    float o[8];
    ix_load8(xr + off, V - off, vec != 0, IX_NEG_INF, o);
    m = fmaxf(m, ix_tree8_max(o));
  }
  m = ix_lane_max<64>(m);
  if (lane == 0) s_wmax[wave] = m;
  __syncthreads();
  m = s_wmax[0];
#pragma unroll
  for (int w = 1; w < 8; ++w) m = fmaxf(m, s_wmax[w]);

  const int units = G * NB;
  for (int u = wave; u < units; u += 8) {
    const int g = u / NB, b = u - g * NB;
    const long base = (long)g * L + (long)b * IX_LP_BLOCK;
    const int nv = min(IX_LP_BLOCK, L - b * IX_LP_BLOCK);
    const float bs = ix_block_expsum(xr + base, nv, m, vec != 0, lane);
    if (lane == 0) s_bsum[u] = bs;
  }
  __syncthreads();
  if (tid < G) s_leaf[tid] = ix_kahan_blocks(s_bsum + tid * NB, NB);
  __syncthreads();
  if (tid == 0) {
    const float S = ix_fold_leaves(s_leaf, G);
    const float log_s = ix_log(S);
    s_fin[0] = m;
    s_fin[1] = log_s;
    ix_lp_emit(xr, V, m, log_s, target, row, out_lp, out_lse);
  }
  if (out_full) {
    __syncthreads();
    const float mm = s_fin[0], ls = s_fin[1];
    float* orow = out_full + row * full_stride;
    for (long off = (long)tid * 8; off < V; off += 512 * 8) {
      float o[8];
      ix_load8(xr + off, V - off, vec != 0, 0.0f, o);
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (off + i < V) orow[off + i] = (o[i] - mm) - ls;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Shape 2: the row split over many workgroups. Workspace layout (floats):
//   pmax [rows, P]  P = ceil(V / IX_LP_SEG)
//   bsum [rows, U]  U = G * NB
//   fin  [rows, 2]  (m, log S)
template <typename T>
__global__ __launch_bounds__(256) void k_lp_partmax(const T* __restrict__ x, long row_stride, int V, int P,
                                                    float* __restrict__ pmax, int vec) {
  __shared__ float s_w[4];
  const long row = blockIdx.x / P;  // parts fastest: consecutive workgroups read consecutive memory
  const int p = blockIdx.x % P;
  const T* xr = x + row * row_stride;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const long lo = (long)p * IX_LP_SEG;
  const long hi = min((long)V, lo + IX_LP_SEG);
  float m = IX_NEG_INF;
  for (long off = lo + (long)tid * 8; off < hi; off += 256 * 8) {
    float o[8];
    ix_load8(xr + off, hi - off, vec != 0, IX_NEG_INF, o);
    m = fmaxf(m, ix_tree8_max(o));
  }
  m = ix_lane_max<64>(m);
  if (lane == 0) s_w[wave] = m;
  __syncthreads();
  if (tid == 0) pmax[row * P + p] = fmaxf(fmaxf(s_w[0], s_w[1]), fmaxf(s_w[2], s_w[3]));
}

__device__ __forceinline__ float ix_row_max_from_parts(const float* __restrict__ pm, int P, int lane) {
  float m = IX_NEG_INF;
  for (int i = lane; i < P; i += 64) m = fmaxf(m, pm[i]);
  return ix_lane_max<64>(m);
}

// Work order: (row, group of 4 units) with the units fastest, i.e. memory order, walked in 8 XCD runs
// (ix_xcd_run_position). On 4096 x 151936 bf16: rows fastest 0.234 ms, memory order 0.219 ms, XCD runs 0.210 ms.
template <typename T>
__global__ __launch_bounds__(256) void k_lp_blocksums(const T* __restrict__ x, long row_stride, int V, int G,
                                                      int P, const float* __restrict__ pmax,
                                                      float* __restrict__ bsum, int vec, int ny,
                                                      unsigned total) {
  unsigned l;
  if (!ix_xcd_run_position(blockIdx.x, total, &l)) return;
  const long row = l / ny;
  const int by = l % ny;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int L = V / G;
  const int NB = (L + IX_LP_BLOCK - 1) / IX_LP_BLOCK;
  const int units = G * NB;
  const int u = by * 4 + wave;
  if (u >= units) return;
  const int g = u / NB, b = u - g * NB;
  const long base = (long)g * L + (long)b * IX_LP_BLOCK;
  const int nv = min(IX_LP_BLOCK, L - b * IX_LP_BLOCK);
  const float bs = ix_block_expsum_with(
      x + row * row_stride + base, nv, [&]() { return ix_row_max_from_parts(pmax + row * P, P, lane); }, vec != 0, lane);
  if (lane == 0) bsum[row * units + u] = bs;
}

template <typename T>
__global__ __launch_bounds__(64) void k_lp_finalize(const T* __restrict__ x, long row_stride, int V, int G, int P,
                                                    const float* __restrict__ pmax,
                                                    const float* __restrict__ bsum, float* __restrict__ fin,
                                                    const int64_t* __restrict__ target,
                                                    float* __restrict__ out_lp, float* __restrict__ out_lse) {
  __shared__ float s_leaf[IX_LP_MAX_G];
  const long row = blockIdx.x;
  const int lane = threadIdx.x;
  const int L = V / G;
  const int NB = (L + IX_LP_BLOCK - 1) / IX_LP_BLOCK;
  const float m = ix_row_max_from_parts(pmax + row * P, P, lane);
  if (lane < G) s_leaf[lane] = ix_kahan_blocks(bsum + row * (long)(G * NB) + lane * NB, NB);
  __syncthreads();
  if (lane == 0) {
    const float S = ix_fold_leaves(s_leaf, G);
    const float log_s = ix_log(S);
    fin[row * 2 + 0] = m;
    fin[row * 2 + 1] = log_s;
    ix_lp_emit(x + row * row_stride, V, m, log_s, target, row, out_lp, out_lse);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void k_lp_fullwrite(const T* __restrict__ x, long row_stride, int V,
                                                      const float* __restrict__ fin, float* __restrict__ out_full,
                                                      long full_stride, int vec, int PW) {
  const long row = blockIdx.x / PW;  // segments fastest
  const T* xr = x + row * row_stride;
  float* orow = out_full + row * full_stride;
  const float mm = fin[row * 2], ls = fin[row * 2 + 1];
  const long lo = (long)(blockIdx.x % PW) * IX_LP_SEG;
  const long hi = min((long)V, lo + IX_LP_SEG);
  for (long off = lo + (long)threadIdx.x * 8; off < hi; off += 256 * 8) {
    float o[8];
    ix_load8(xr + off, hi - off, vec != 0, 0.0f, o);
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (off + i < hi) orow[off + i] = (o[i] - mm) - ls;
  }
}

// rowmax[row] = max over P parts (exact; any order). One wave per row.
__global__ __launch_bounds__(256) void k_lp_reduce_parts(const float* __restrict__ parts, long parts_ld, int P,
                                                         long rows, float* __restrict__ rowmax) {
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const float m = ix_row_max_from_parts(parts + row * parts_ld, P, threadIdx.x & 63);
  if ((threadIdx.x & 63) == 0) rowmax[row] = m;
}

extern "C" int ix_rowmax_reduce(const float* parts, long parts_ld, long P, long rows, float* rowmax, void* stream) {
  if (!parts || !rowmax || rows < 0 || P <= 0 || parts_ld < P || P > 0x7fffffffL) return IX_ERR_ARG;
  if (rows == 0) return IX_OK;
  const long grid = (rows + 3) / 4;
  if (grid > 0x7fffffffL) return IX_DECLINED;
  hipLaunchKernelGGL(k_lp_reduce_parts, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, parts, parts_ld,
                     (int)P, rows, rowmax);
  return ix_launch_status();
}

// ---------------------------------------------------------------------------------------------
static int ix_lp_check(const void* logits, int dtype, long rows, long V, long row_stride, int G) {
  if (!logits || rows < 0 || V <= 0 || row_stride < V) return IX_ERR_ARG;
  if (dtype != IX_DT_F32 && dtype != IX_DT_BF16) return IX_DECLINED;
  if (G < 1 || G > IX_LP_MAX_G || (G & (G - 1)) != 0) return IX_DECLINED;
  if (V % G != 0) return IX_DECLINED;  // unequal leaves change the contract (rowinv.py:376-377)
  if (V > 0x7fffffffL || rows > 0x7fffffffL) return IX_DECLINED;
  const long L = V / G;
  const long NB = (L + IX_LP_BLOCK - 1) / IX_LP_BLOCK;
  if (G * NB > IX_LP_MAX_UNITS) return IX_DECLINED;
  return IX_OK;
}

extern "C" size_t ix_logprob_workspace_bytes(long rows, long V, int G) {
  if (rows <= 0 || V <= 0 || G < 1 || V % G != 0) return 0;
  const long L = V / G;
  const long NB = (L + IX_LP_BLOCK - 1) / IX_LP_BLOCK;
  const long P = (V + IX_LP_SEG - 1) / IX_LP_SEG;
  return (size_t)rows * (size_t)(P + G * NB + 2) * sizeof(float);
}

template <typename T>
static int ix_lp_launch(const T* x, long rows, long V, long row_stride, int G, const int64_t* target,
                        float* out_lp, float* out_lse, float* out_full, long full_stride, float* ws,
                        size_t ws_bytes, int force_shape, const float* row_max_in, hipStream_t st) {
  if (rows == 0) return IX_OK;
  const long L = V / G;
  const int vec = (ix_aligned(x, 8 * sizeof(T)) && (row_stride % 8 == 0) && (L % 8 == 0)) ? 1 : 0;
  // a caller-supplied row max (exact, e.g. from the producing GEMM's epilogue) removes the max
  // pass: the row is then read from HBM once, by the block sums
  const bool split = row_max_in || force_shape == 2 || (force_shape == 0 && rows < IX_LP_SPLIT_BELOW);
  if (!split) {
    hipLaunchKernelGGL((k_lp_row<T>), dim3((unsigned)rows), dim3(512), 0, st, x, row_stride, (int)V, G, target,
                       out_lp, out_lse, out_full, full_stride, vec);
    return ix_launch_status();
  }
  if (rows * (long)((V + IX_LP_SEG - 1) / IX_LP_SEG) > 0x7fffffffL || rows * (long)(G * ((L + IX_LP_BLOCK - 1) / IX_LP_BLOCK)) > 0x7fffffffL)
    return IX_DECLINED;
  if (!ws || ws_bytes < ix_logprob_workspace_bytes(rows, V, G)) return IX_ERR_ARG;
  const int NB = (int)((L + IX_LP_BLOCK - 1) / IX_LP_BLOCK);
  const int PW = (int)((V + IX_LP_SEG - 1) / IX_LP_SEG);  // workspace layout always reserves PW parts
  const int U = G * NB;
  float* ws_pmax = ws;
  float* bsum = ws_pmax + rows * PW;
  float* fin = bsum + rows * U;
  const int P = row_max_in ? 1 : PW;
  const float* pmax = row_max_in ? row_max_in : ws_pmax;
  if (!row_max_in)
    hipLaunchKernelGGL((k_lp_partmax<T>), dim3((unsigned)(rows * P)), dim3(256), 0, st, x, row_stride, (int)V, P,
                       ws_pmax, vec);
  const int ny = (U + 3) / 4;
  const unsigned total = (unsigned)(rows * ny);
  hipLaunchKernelGGL((k_lp_blocksums<T>), dim3(ix_xcd_run_grid(total)), dim3(256), 0, st, x, row_stride, (int)V, G,
                     P, pmax, bsum, vec, ny, total);
  hipLaunchKernelGGL((k_lp_finalize<T>), dim3((unsigned)rows), dim3(64), 0, st, x, row_stride, (int)V, G, P, pmax,
                     bsum, fin, target, out_lp, out_lse);
  if (out_full)
    hipLaunchKernelGGL((k_lp_fullwrite<T>), dim3((unsigned)(rows * PW)), dim3(256), 0, st, x, row_stride, (int)V, fin,
                       out_full, full_stride, vec, PW);
  return ix_launch_status();
}

extern "C" int ix_logprob_rowinv_sampled(const void* logits, int dtype, long rows, long V, long row_stride,
                                         const int64_t* target, int G, float* out_logprob, float* out_lse,
                                         void* workspace, size_t workspace_bytes, int force_shape,
                                         const float* row_max_in, void* stream) {
  int rc = ix_lp_check(logits, dtype, rows, V, row_stride, G);
  if (rc != IX_OK) return rc;
  if (!target || !out_logprob) return IX_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == IX_DT_BF16)
    return ix_lp_launch((const bf16_t*)logits, rows, V, row_stride, G, target, out_logprob, out_lse, nullptr, 0,
                        (float*)workspace, workspace_bytes, force_shape, row_max_in, st);
  return ix_lp_launch((const float*)logits, rows, V, row_stride, G, target, out_logprob, out_lse, nullptr, 0,
                      (float*)workspace, workspace_bytes, force_shape, row_max_in, st);
}

extern "C" int ix_logprob_rowinv_full(const void* logits, int dtype, long rows, long V, long row_stride, int G,
                                      float* out_full, long out_stride, float* out_lse, void* workspace,
                                      size_t workspace_bytes, int force_shape, const float* row_max_in,
                                      void* stream) {
  int rc = ix_lp_check(logits, dtype, rows, V, row_stride, G);
  if (rc != IX_OK) return rc;
  if (!out_full || out_stride < V) return IX_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == IX_DT_BF16)
    return ix_lp_launch((const bf16_t*)logits, rows, V, row_stride, G, nullptr, nullptr, out_lse, out_full,
                        out_stride, (float*)workspace, workspace_bytes, force_shape, row_max_in, st);
  return ix_lp_launch((const float*)logits, rows, V, row_stride, G, nullptr, nullptr, out_lse, out_full,
                      out_stride, (float*)workspace, workspace_bytes, force_shape, row_max_in, st);
}
