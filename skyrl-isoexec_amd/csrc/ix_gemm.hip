// Batch-invariant dense matmuls: the bf16 GEMM behind every linear layer and the LM head, and
// the fp32 GEMM behind the MoE router. Counterpart of the reference's global aten mm/addmm
// override (ops/moe/moe_batch_invariant.py:422-473, ops/mm/mm_tiles.py:127-158) and of its
// pinned non-split-K provider (ops/mm/csrc/cublaslt_pinned.cpp:1-36).
#include "ix_gemm_core.h"
#include "ix_gemm_stream.h"
#include "../../include/isoexec_hip.h"

// Workgroup -> tile map. Hardware hands consecutive workgroup ids to the 8 XCDs round-robin, and each XCD has
// its own L2. The tiles are put in one order -- groups of GM M-tiles x GN weight tiles, about what an XCD's 32
// CUs hold at a time, so that a group pulls GM activation tiles and GN weight tiles through the L2 for GM * GN
// tiles; groups run down the M-tiles of GN weight-tile columns before moving to the next columns -- and that
// order is cut into 8 equal runs, one per XCD: every XCD gets the same number of tiles whatever the shape, and
// a weight tile is fetched by one L2 (two where a run ends inside its column group).
#ifndef IX_GEMM_GM
#define IX_GEMM_GM 8  // M-tiles of a group
#endif
#ifndef IX_GEMM_GN
#define IX_GEMM_GN 4  // weight tiles of a group
#endif
// Tile number idx of XCD xcd's run of that order, for groups of GM x GN tiles.
__device__ __forceinline__ bool ix_tile_of_run(unsigned xcd, unsigned idx, int nb_m, int nb_n, int GM, int GN, int* tm,
                                               int* tn) {
  // 32-bit arithmetic throughout (the launch refuses more than 2^31 tiles): a 64-bit division costs a workgroup
  // about a microsecond before its first fetch.
  const unsigned tiles = (unsigned)nb_m * (unsigned)nb_n;
  // this XCD's run of the tile order: [tiles * xcd / 8, tiles * (xcd + 1) / 8)
  const unsigned q = tiles >> 3, r = tiles & 7u;
  const unsigned lo = q * xcd + ((r * xcd) >> 3), hi = q * (xcd + 1) + ((r * (xcd + 1)) >> 3);
  const unsigned l = lo + idx;
  if (l >= hi) return false;
  const unsigned per_ngroup = (unsigned)GN * (unsigned)nb_m;
  const unsigned ng = l / per_ngroup;
  const unsigned rem = l - ng * per_ngroup;
  const int gn = min(GN, nb_n - (int)ng * GN);  // width of this (possibly last) column group
  const unsigned per_mgroup = (unsigned)GM * (unsigned)gn;
  const unsigned mg = rem / per_mgroup;
  const unsigned r2 = rem - mg * per_mgroup;
  const int gm = min(GM, nb_m - (int)mg * GM);
  const unsigned nl = r2 / (unsigned)gm, ml = r2 - nl * (unsigned)gm;
  *tm = (int)mg * GM + (int)ml;
  *tn = (int)ng * GN + (int)nl;
  return true;
}

__device__ __forceinline__ void ix_store4(bf16_t* p, int valid, bool vec, const float (&v)[4]) {
  ix_store4_bf16(p, valid, vec, v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void ix_store4(float* p, int valid, bool vec, const float (&v)[4]) {
  if (vec && valid >= 4) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (e < valid) p[e] = v[e];
  }
}

// Row-max parts a tile writes per row: one, except the four-wave 256 x 256 tile, which writes one per wave column.
template <int BM, int BN, int WM, int WN, int PW>
__host__ __device__ constexpr int ix_gemm_parts_per_tile() {
  return (BM == 256 && BN == 256 && WM == 2 && WN == 2 && PW == 0) ? WN : 1;
}

__device__ __forceinline__ bool ix_tile_of_block(unsigned bid, int nb_m, int nb_n, int* tm, int* tn) {
  return ix_tile_of_run(bid & 7u, bid >> 3, nb_m, nb_n, IX_GEMM_GM, IX_GEMM_GN, tm, tn);
}

// TC = bf16_t: C is the bf16 round of the fp32 accumulator; TC = float: the accumulator itself.
// row_max_parts (optional): [M, parts_ld] fp32, entry (m, tn) = max over the tile's columns of the
// values stored to C (exact, order-free), so a consumer can skip its own max pass over C.
template <int BM, int BN, int WM, int WN, typename TC, int PW = 0>
__global__ __launch_bounds__((WM * WN + PW) * 64) void k_gemm_bf16_nt(const bf16_t* __restrict__ A, long lda,
                                                              const bf16_t* __restrict__ W, long ldw,
                                                              const bf16_t* __restrict__ bias,
                                                              TC* __restrict__ C, long ldc, int M, int N, int K,
                                                              int nb_m, int nb_n, int vec_store,
                                                              float* __restrict__ row_max_parts, long parts_ld,
                                                              long batch_a, long batch_w, long batch_c) {
  using Cfg = IxGemmCfg<BM, BN, WM, WN, PW>;
  extern __shared__ __align__(16) char ix_lds[];
  // a batch of independent products (bmm): workgroup row blockIdx.y works on matrices batch strides further on
  A += (long)blockIdx.y * batch_a;
  W += (long)blockIdx.y * batch_w;
  C += (long)blockIdx.y * batch_c;
  int tm, tn;
  if (!ix_tile_of_block(blockIdx.x, nb_m, nb_n, &tm, &tn)) return;
  const long m0 = (long)tm * BM;
  const long n0 = (long)tn * BN;
  const int m_valid = (int)min((long)BM, (long)M - m0);
  const int n_valid = (int)min((long)BN, (long)N - n0);

  // Tile-local buffer descriptors: rows past the matrix fall outside the range and read as 0.
  const ix_rsrc_t x_rsrc = ix_make_rsrc(A + m0 * lda, (uint32_t)(((long)(m_valid - 1) * lda + K) * 2));
  const ix_rsrc_t w_rsrc = ix_make_rsrc(W + n0 * ldw, (uint32_t)(((long)(n_valid - 1) * ldw + K) * 2));
  auto x_row = [&](int r) -> uint32_t { return (r < m_valid) ? (uint32_t)(r * lda * 2) : IX_OOB; };
  auto w_row = [&](int r) -> uint32_t { return (r < n_valid) ? (uint32_t)(r * ldw * 2) : IX_OOB; };

  ix_f32x16 acc[Cfg::MI][Cfg::NI];
  ix_acc_zero<Cfg>(acc);
  ix_gemm_mainloop<Cfg>(x_rsrc, x_row, w_rsrc, w_row, K, ix_lds, acc);

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const bool computes = PW == 0 || wave < WM * WN;  // fetching waves hold no results
  float rmax[Cfg::MI];
  // A whole bf16 tile with 16-byte aligned rows takes the wide stores (same values, same places).
  const bool wide = sizeof(TC) == 2 && m_valid == BM && n_valid == BN && (ldc % 8 == 0) && (reinterpret_cast<uintptr_t>(C) % 16 == 0);
  // Compile-time indices throughout: a rolled loop over mi would index the accumulators dynamically and push them to
  // memory. The whole-tile path is instantiated with and without a bias: at 256 values per lane the epilogue is bound by
  // vector-ALU issue, not by the stores (the row maximum costs three instructions per four values and is always taken).
#pragma unroll
  for (int mi = 0; mi < Cfg::MI; ++mi) rmax[mi] = IX_NEG_INF;
  if constexpr (Cfg::MI * Cfg::NI == 16) {
    // the matrix pipeline has drained before the accumulation registers are read by hand below
    asm volatile("s_nop 15\n\ts_nop 15");
  }
  auto whole_tile = [&](auto has_bias_c) {
    constexpr bool HAS_BIAS = decltype(has_bias_c)::value;
    constexpr int NPIECE = Cfg::NI * 2;
    char* buf = ix_lds + wave * ix_store_block32_lds_bytes<NPIECE>();
    ix_static_for<0, Cfg::MI>([&](auto mic) {
      constexpr int mi = decltype(mic)::value;
      uint4 pieces[NPIECE];
      ix_static_for<0, Cfg::NI>([&](auto nic) {
        constexpr int ni = decltype(nic)::value;
        float a16[16];
        ix_acc_read16<(Cfg::MI * Cfg::NI == 16)>(acc[mi][ni], a16);
#pragma unroll
        for (int p = 0; p < 2; ++p) {
          uint2 pk[2];
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const int q = 2 * p + h;
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = a16[q * 4 + e];
            if constexpr (HAS_BIAS) {
              const long n = n0 + wn * Cfg::TN + ni * 32 + ix_acc_row(q * 4, lane);
              const uint2 b4 = *reinterpret_cast<const uint2*>(bias + n);  // n % 4 == 0 and bias is 8-byte aligned
              v[0] = v[0] + __uint_as_float(b4.x << 16);
              v[1] = v[1] + __uint_as_float(b4.x & 0xffff0000u);
              v[2] = v[2] + __uint_as_float(b4.y << 16);
              v[3] = v[3] + __uint_as_float(b4.y & 0xffff0000u);
            }
            rmax[mi] = fmaxf(rmax[mi], fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3])));
            pk[h].x = ix_pack_bf2_hw(v[0], v[1]);
            pk[h].y = ix_pack_bf2_hw(v[2], v[3]);
          }
          pieces[ni * 2 + p] = ix_join_halves(pk[0], pk[1]);
        }
      });
      // whole rows of the wave's TN columns per store instruction instead of 32-byte pieces of 32 rows
      ix_store_block32_via_lds<NPIECE>(buf, pieces,
                                       reinterpret_cast<bf16_t*>(C) + (m0 + wm * Cfg::TM + mi * 32) * ldc + n0 + wn * Cfg::TN,
                                       ldc, 32);
    });
  };
  // Late zero-fills of the ring by other waves' past-the-end fetches must not land on the store buffers.
  if (wide) __syncthreads();
  if (!computes) {
  } else if (wide && (!bias || (reinterpret_cast<uintptr_t>(bias) % 8 == 0))) {
    if (bias) whole_tile(std::true_type{}); else whole_tile(std::false_type{});
  } else {
    ix_static_for<0, Cfg::MI>([&](auto mic) {
      constexpr int mi = decltype(mic)::value;
      const long m = m0 + wm * Cfg::TM + mi * 32 + (lane & 31);
      ix_static_for<0, Cfg::NI>([&](auto nic) {
        constexpr int ni = decltype(nic)::value;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const long n = n0 + wn * Cfg::TN + ni * 32 + ix_acc_row(q * 4, lane);
          const int valid = (int)min(4L, (long)N - n);
          if (valid <= 0 || m >= M) continue;
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            v[e] = acc[mi][ni][q * 4 + e];
            // addmm: the bias joins in fp32 before the single bf16 round.
            if (bias && e < valid) v[e] = v[e] + ix_bf2f(bias[n + e]);
            if (e < valid) rmax[mi] = fmaxf(rmax[mi], v[e]);
          }
          ix_store4(C + m * ldc + n, valid, vec_store != 0, v);
        }
      });
    });
  }
  if (row_max_parts) {
    float* s_max = reinterpret_cast<float*>(ix_lds);  // [WN][BM]
    __syncthreads();                                  // every wave has left the main loop's LDS reads
#pragma unroll
    for (int mi = 0; mi < Cfg::MI; ++mi) {
      float v = fmaxf(rmax[mi], __shfl_xor(rmax[mi], 32, IX_WAVE));
      // rounding is monotonic: the max of the rounded values is the rounded max
      if (sizeof(TC) == 2) v = ix_rbf(v);
      if (computes && lane < 32) s_max[wn * BM + wm * Cfg::TM + mi * 32 + lane] = v;
    }
    __syncthreads();
    for (int r = threadIdx.x; r < m_valid; r += Cfg::NTT) {
      if constexpr (ix_gemm_parts_per_tile<BM, BN, WM, WN, PW>() == WN) {
        // one part per wave column: the layout the streaming form of this tile writes without passing through LDS
#pragma unroll
        for (int w = 0; w < WN; ++w) row_max_parts[(m0 + r) * parts_ld + tn * WN + w] = s_max[w * BM + r];
      } else {
        float v = s_max[r];
#pragma unroll
        for (int w = 1; w < WN; ++w) v = fmaxf(v, s_max[w * BM + r]);
        row_max_parts[(m0 + r) * parts_ld + tn] = v;
      }
    }
  }
}

// ---- the streaming form of the four-wave 256 x 256 tile (pipeline F) -----------------------------------------------
// bf16 output without bias, K a multiple of 64 with at least IX_STREAM_MIN_KT k-tiles, N a multiple of 8, rows of C
// 16-byte aligned. A workgroup takes every (gridDim.x / 8)-th tile of its XCD's run of the tile order.
// Tile sequence of the dense product: position idx of XCD xcd's run of the tile order above.
struct IxDenseStreamSeq {
  const bf16_t* A;
  const bf16_t* W;
  bf16_t* C;
  float* parts;
  long lda, ldw, ldc, parts_ld;
  int M, N, K, nb_m, nb_n, gm, gn;
  __device__ __forceinline__ bool locate(unsigned xcd, unsigned idx, IxStreamTile& t) const {
    int tm, tn;
    if (!ix_tile_of_run(xcd, idx, nb_m, nb_n, gm, gn, &tm, &tn)) return false;
    const long m0 = (long)tm * 256, n0 = (long)tn * 256;
    t.x = A + m0 * lda;
    t.w = W + n0 * ldw;
    t.c = C + m0 * ldc + n0;
    t.part = parts + m0 * parts_ld + tn * 2;
    t.mv = (int)min(256L, (long)M - m0);
    t.nv = (int)min(256L, (long)N - n0);
    return true;
  }
};

template <bool PARTS>
__global__ __launch_bounds__(256) void k_gemm_bf16_nt_stream(const bf16_t* __restrict__ A, long lda,
                                                             const bf16_t* __restrict__ W, long ldw,
                                                             bf16_t* __restrict__ C, long ldc, int M, int N, int K,
                                                             int nb_m, int nb_n, int gm, int gn,
                                                             float* __restrict__ row_max_parts, long parts_ld) {
  using Cfg = IxGemmCfg<256, 256, 2, 2>;
  extern __shared__ __align__(16) char ix_lds[];
  IxPlainStreamJob<Cfg, IxDenseStreamSeq, PARTS> job;
  job.seq.gm = gm;
  job.seq.gn = gn;
  job.seq.A = A;
  job.seq.lda = lda;
  job.seq.W = W;
  job.seq.ldw = ldw;
  job.seq.C = C;
  job.seq.ldc = ldc;
  job.seq.M = M;
  job.seq.N = N;
  job.seq.K = K;
  job.seq.nb_m = nb_m;
  job.seq.nb_n = nb_n;
  job.seq.parts = row_max_parts;
  job.seq.parts_ld = parts_ld;
  ix_gemm_stream4<Cfg>(job, K / IX_BK, ix_lds);
}

static bool ix_gemm_stream_fits(const void* C, long ldc, long M, long N, long K, const void* bias, long batch,
                                long min_tiles) {
  const long tiles = ((M + 255) / 256) * ((N + 255) / 256);
  return !bias && batch == 1 && (K % IX_BK == 0) && K / IX_BK >= IX_STREAM_MIN_KT && (N % 8 == 0) && (ldc % 8 == 0) &&
         ix_aligned(C, 16) && ldc * 512 < 0x40000000L && tiles >= min_tiles;
}

static int ix_gemm_bf16_stream_launch(const bf16_t* A, long lda, const bf16_t* W, long ldw, bf16_t* C, long ldc, long M,
                                      long N, long K, float* parts, long parts_ld, hipStream_t st) {
  using Cfg = IxGemmCfg<256, 256, 2, 2>;
  const long nb_m = (M + 255) / 256, nb_n = (N + 255) / 256;
  if (nb_m * nb_n > 0x7fffffffL) return IX_DECLINED;
  if (parts && parts_ld < nb_n * 2) return IX_ERR_ARG;
  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)k_gemm_bf16_nt_stream<true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            Cfg::LDS_BYTES) != hipSuccess ||
        hipFuncSetAttribute((const void*)k_gemm_bf16_nt_stream<false>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            Cfg::LDS_BYTES) != hipSuccess)
      return IX_ERR_LAUNCH;
    attr_set = true;
  }
  // Group shape of the tile order: with many row tiles the activations are the operand that streams, and a group
  // that is wider in weight tiles re-uses each activation tile more often (163840 x 2048 x 12352: 6.40 -> 6.20 ms,
  // 32768 x 2048 x 151936: 15.7 -> 15.5); with few row tiles the default serves the weights better.
  const int gm = nb_m >= 64 ? 4 : IX_GEMM_GM, gn = nb_m >= 64 ? 16 : IX_GEMM_GN;
  if (parts)
    hipLaunchKernelGGL(k_gemm_bf16_nt_stream<true>, dim3(IX_STREAM_WORKGROUPS), dim3(256), Cfg::LDS_BYTES, st, A, lda, W,
                       ldw, C, ldc, (int)M, (int)N, (int)K, (int)nb_m, (int)nb_n, gm, gn, parts, parts_ld);
  else
    hipLaunchKernelGGL(k_gemm_bf16_nt_stream<false>, dim3(IX_STREAM_WORKGROUPS), dim3(256), Cfg::LDS_BYTES, st, A, lda, W,
                       ldw, C, ldc, (int)M, (int)N, (int)K, (int)nb_m, (int)nb_n, gm, gn, parts, parts_ld);
  return ix_launch_status();
}

template <int BM, int BN, int WM, int WN, typename TC, int PW = 0>
static int ix_gemm_bf16_launch(const bf16_t* A, long lda, const bf16_t* W, long ldw, const bf16_t* bias, TC* C,
                               long ldc, long M, long N, long K, float* parts, long parts_ld, hipStream_t st,
                               long batch = 1, long batch_a = 0, long batch_w = 0, long batch_c = 0) {
  using Cfg = IxGemmCfg<BM, BN, WM, WN, PW>;
  const long nb_m = (M + BM - 1) / BM, nb_n = (N + BN - 1) / BN;
  const long grid = 8 * ((nb_m * nb_n + 7) / 8);  // 8 XCD runs of the tile order, the longest one sets the count
  if (grid > 0x7fffffffL) return IX_DECLINED;
  if (parts && parts_ld < nb_n * ix_gemm_parts_per_tile<BM, BN, WM, WN, PW>()) return IX_ERR_ARG;
  auto kern = k_gemm_bf16_nt<BM, BN, WM, WN, TC, PW>;
  static bool attr_set = false;  // per instantiation
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES) !=
        hipSuccess)
      return IX_ERR_LAUNCH;
    attr_set = true;
  }
  const int vec = (ldc % 4 == 0) && ix_aligned(C, 4 * sizeof(TC));
  if (batch > 65535) return IX_DECLINED;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid, (unsigned)batch), dim3(Cfg::NTT), Cfg::LDS_BYTES, st, A, lda, W, ldw,
                     bias, C, ldc, (int)M, (int)N, (int)K, (int)nb_m, (int)nb_n, vec, parts, parts_ld, batch_a, batch_w,
                     batch_c);
  return ix_launch_status();
}

// Which tile shape runs (0 = choose). Never changes a bit. The choice minimises a small cost model fitted to
// measurements on MI355X: a launch runs in ceil(tiles / slots) waves of workgroups (one or two per CU), a workgroup costs
// about 6 us plus K/64 k-tiles at a per-shape rate, and no shape streams the operands faster than ~5 TB/s. Big
// square tiles win when there are enough of them to fill the chip several times over; a product with few rows or
// few columns takes smaller tiles so that every CU has one.
static int ix_gemm_tile_for(long M, long N, long K, int tile) {
  if (tile != 0) return tile;
  // One 128-wide column of tiles (the router's gating product): 128-row tiles once there are enough of them to fill
  // the chip, the small tile below that (2048 x 2048 x 128: 20.7 -> 8.5 us; equal at 16384 rows).
  if (M > 128 && N <= 128) return M >= 16384 ? 2 : 6;
  // slots: workgroups resident on the chip at once; us_per_ktile: with the CU to itself / shared with a second one;
  // us_fixed: launch, first fetches and the store phase of one workgroup
  struct Shape { int id, bm, bn; double slots, us_per_ktile, us_per_ktile_shared, us_fixed; };
  // preference order on ties: larger tiles first. The 256 x 256 tile runs on four waves (id 4: a third fewer LDS reads,
  // 1.4 us per k-tile) unless the product is short in K, where the eight-wave form's shorter store phase wins.
  static const Shape shapes[] = {{4, 256, 256, 256.0, 1.4, 1.4, 8.0},   {5, 128, 256, 256.0, 0.75, 0.75, 6.0},
                                 {2, 128, 128, 512.0, 0.6, 1.0, 6.0},   {1, 32, 256, 256.0, 0.55, 0.55, 6.0},
                                 {6, 64, 32, 512.0, 0.16, 0.16, 6.0}};
  const double kt = (double)((K + 63) / 64);
  const double stream_us = (double)(N + M) * (double)K * 2.0 / 5.0e6;  // both operands once at 5 TB/s
  int best = 4;
  double best_cost = 1e300, big_cost = 0.0;
  for (const Shape& sh : shapes) {
    const double tiles = (double)((M + sh.bm - 1) / sh.bm) * (double)((N + sh.bn - 1) / sh.bn);
    const double waves = (double)(long)((tiles + sh.slots - 1.0) / sh.slots);
    double cost = waves * (sh.us_fixed + kt * (tiles > 256.0 ? sh.us_per_ktile_shared : sh.us_per_ktile));
    if (cost < stream_us) cost = sh.id == 2 ? 0.9 * stream_us : stream_us;  // two workgroups per CU stream best
    if (sh.id == 4) big_cost = cost;
    if (cost < best_cost * 0.97) {  // a later (smaller) shape must win by a margin
      best_cost = cost;
      best = sh.id;
    }
  }
  // With more than half a big tile of rows, the big tile keeps its place unless another shape is clearly ahead:
  // at scale the smaller shapes pull more bytes through L2 than the per-k-tile rates above say.
  if (M > 128 && big_cost <= 1.25 * best_cost) best = 4;
  return best;
}

// Row-max parts per row of C: one per column tile of the shape that runs.
extern "C" long ix_gemm_bf16_n_tiles(long M, long N, long K, int tile) {
  const int t = ix_gemm_tile_for(M, N, K, tile);
  const long bn = (t == 2) ? 128 : (t == 6) ? 32 : 256;  // ids 1, 3, 4, 5, 7, 8 are 256 wide
  const long per_tile = (t == 4 || t == 7 || t == 8) ? 2 : 1;      // the four-wave tile writes one part per wave column
  return N <= 0 ? 0 : per_tile * ((N + bn - 1) / bn);
}

template <typename TC>
static int ix_gemm_bf16_dispatch(const bf16_t* a, long lda, const bf16_t* w, long ldw, const bf16_t* b, TC* c,
                                 long ldc, long M, long N, long K, int tile, float* parts, long parts_ld,
                                 hipStream_t st, long batch = 1, long sa = 0, long sw = 0, long sc = 0) {
  // `tile` only picks which workgroup owns an element (0 = by M); the bits do not depend on it.
#define IX_BATCH_ARGS , batch, sa, sw, sc
  switch (ix_gemm_tile_for(M * (batch > 1 ? batch : 1), N, K, tile)) {
    case 1: return ix_gemm_bf16_launch<32, 256, 1, 4, TC, 4>(a, lda, w, ldw, b, c, ldc, M, N, K, parts, parts_ld, st IX_BATCH_ARGS);
    case 2: return ix_gemm_bf16_launch<128, 128, 2, 2, TC>(a, lda, w, ldw, b, c, ldc, M, N, K, parts, parts_ld, st IX_BATCH_ARGS);
    case 3: return ix_gemm_bf16_launch<256, 256, 2, 4, TC>(a, lda, w, ldw, b, c, ldc, M, N, K, parts, parts_ld, st IX_BATCH_ARGS);
    case 4:
      if constexpr (sizeof(TC) == 2) {
        // worth it from two tiles per workgroup up
        if (ix_gemm_stream_fits(c, ldc, M, N, K, b, batch, 2 * IX_STREAM_WORKGROUPS))
          return ix_gemm_bf16_stream_launch(a, lda, w, ldw, (bf16_t*)c, ldc, M, N, K, parts, parts_ld, st);
      }
      [[fallthrough]];
    case 7:  // the same tile, one tile per workgroup
      return ix_gemm_bf16_launch<256, 256, 2, 2, TC>(a, lda, w, ldw, b, c, ldc, M, N, K, parts, parts_ld, st IX_BATCH_ARGS);
    case 5: return ix_gemm_bf16_launch<128, 256, 2, 4, TC>(a, lda, w, ldw, b, c, ldc, M, N, K, parts, parts_ld, st IX_BATCH_ARGS);
    case 6: return ix_gemm_bf16_launch<64, 32, 2, 1, TC, 2>(a, lda, w, ldw, b, c, ldc, M, N, K, parts, parts_ld, st IX_BATCH_ARGS);
    case 8:  // the streaming form whatever the number of tiles (declines what it does not serve)
      if constexpr (sizeof(TC) == 2) {
        if (ix_gemm_stream_fits(c, ldc, M, N, K, b, batch, 1))
          return ix_gemm_bf16_stream_launch(a, lda, w, ldw, (bf16_t*)c, ldc, M, N, K, parts, parts_ld, st);
      }
      return IX_DECLINED;
    default: return IX_ERR_ARG;
  }
#undef IX_BATCH_ARGS
}

extern "C" int ix_gemm_bf16_nt(const void* A, long lda, const void* W, long ldw, const void* bias, void* C,
                               int c_dtype, long ldc, long M, long N, long K, int tile, float* row_max_parts,
                               long parts_ld, void* stream) {
  if (!A || !W || !C || M < 0 || N <= 0 || K <= 0) return IX_ERR_ARG;
  if (lda < K || ldw < K || ldc < N) return IX_ERR_ARG;
  if (c_dtype != IX_DT_BF16 && c_dtype != IX_DT_F32) return IX_DECLINED;
  // 16-byte row chunks: every row start and K itself must be a multiple of 8 elements.
  if ((K % 8) || (lda % 8) || (ldw % 8) || !ix_aligned(A, 16) || !ix_aligned(W, 16)) return IX_DECLINED;
  if (M > 0x7fffffffL || N > 0x7fffffffL || K > 0x7fffffffL) return IX_DECLINED;
  if (lda * 2 * 256 >= 0x40000000L || ldw * 2 * 256 >= 0x40000000L) return IX_DECLINED;  // tile offsets < 1 GiB
  if (M == 0) return IX_OK;
  hipStream_t st = (hipStream_t)stream;
  const bf16_t *a = (const bf16_t*)A, *w = (const bf16_t*)W, *b = (const bf16_t*)bias;
  if (c_dtype == IX_DT_BF16)
    return ix_gemm_bf16_dispatch(a, lda, w, ldw, b, (bf16_t*)C, ldc, M, N, K, tile, row_max_parts, parts_ld, st);
  return ix_gemm_bf16_dispatch(a, lda, w, ldw, b, (float*)C, ldc, M, N, K, tile, row_max_parts, parts_ld, st);
}

// aten::bmm of the override (ops/moe/moe_batch_invariant.py:453-464): `batch` independent products in ONE launch, each
// exactly the product ix_gemm_bf16_nt computes (same tiles, same K order, same bits); matrix b of an operand starts
// b * stride elements after matrix 0. The tile shape is chosen for the whole batch (rows M * batch).
extern "C" int ix_gemm_bf16_nt_batched(const void* A, long lda, long stride_a, const void* W, long ldw, long stride_w,
                                       void* C, long ldc, long stride_c, long batch, long M, long N, long K, int tile,
                                       void* stream) {
  if (!A || !W || !C || batch < 0 || M < 0 || N <= 0 || K <= 0) return IX_ERR_ARG;
  if (lda < K || ldw < K || ldc < N) return IX_ERR_ARG;
  if ((K % 8) || (lda % 8) || (ldw % 8) || (stride_a % 8) || (stride_w % 8) || !ix_aligned(A, 16) || !ix_aligned(W, 16))
    return IX_DECLINED;
  if (M > 0x7fffffffL || N > 0x7fffffffL || K > 0x7fffffffL) return IX_DECLINED;
  if (lda * 2 * 256 >= 0x40000000L || ldw * 2 * 256 >= 0x40000000L) return IX_DECLINED;
  if (M == 0 || batch == 0) return IX_OK;
  return ix_gemm_bf16_dispatch((const bf16_t*)A, lda, (const bf16_t*)W, ldw, (const bf16_t*)nullptr, (bf16_t*)C, ldc, M,
                               N, K, tile, (float*)nullptr, 0, (hipStream_t)stream, batch, stride_a, stride_w, stride_c);
}

// ---------------------------------------------------------------------------------------------
// fp32 GEMM (router gating): C[m, n] = sum_k A[m, k] * W[n, k], A bf16 (widened exactly) or
// fp32, W fp32, C fp32. One instruction, v_mfma_f32_32x32x2_f32; instruction j consumes
// k = 2j (lane group 0) and 2j+1 (lane group 1); instructions accumulate left to right.
#define IX_F32_BM 64
#define IX_F32_BN 128
#define IX_F32_BK 32
#define IX_F32_PITCH 33

template <typename TA>
__global__ __launch_bounds__(256) void k_gemm_f32_nt(const TA* __restrict__ A, long lda,
                                                     const float* __restrict__ W, long ldw,
                                                     float* __restrict__ C, long ldc, int M, int N, int K) {
  __shared__ float sA[IX_F32_BM * IX_F32_PITCH];
  __shared__ float sW[IX_F32_BN * IX_F32_PITCH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;  // 2 x 2 waves, wave tile 32 x 64
  const long m0 = (long)blockIdx.x * IX_F32_BM;
  const long n0 = (long)blockIdx.y * IX_F32_BN;
  ix_f32x16 acc[2];
#pragma unroll
  for (int ni = 0; ni < 2; ++ni)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[ni][i] = 0.0f;

  for (int k0 = 0; k0 < K; k0 += IX_F32_BK) {
    // stage A: 64 rows x 32 k, W: 128 rows x 32 k; one element per thread per pass
    for (int q = tid; q < IX_F32_BM * IX_F32_BK; q += 256) {
      const int r = q >> 5, c = q & 31;
      const long m = m0 + r;
      float v = 0.0f;
      if (m < M && k0 + c < K) {
        if constexpr (sizeof(TA) == 2) v = ix_bf2f(A[m * lda + k0 + c]);
        else v = A[m * lda + k0 + c];
      }
      sA[r * IX_F32_PITCH + c] = v;
    }
    for (int q = tid; q < IX_F32_BN * IX_F32_BK; q += 256) {
      const int r = q >> 5, c = q & 31;
      const long n = n0 + r;
      sW[r * IX_F32_PITCH + c] = (n < N && k0 + c < K) ? W[n * ldw + k0 + c] : 0.0f;
    }
    __syncthreads();
    const int fr = lane & 31, fg = lane >> 5;
#pragma unroll
    for (int j = 0; j < IX_F32_BK / 2; ++j) {
      const float a = sA[(wm * 32 + fr) * IX_F32_PITCH + 2 * j + fg];
#pragma unroll
      for (int ni = 0; ni < 2; ++ni) {
        const float b = sW[(wn * 64 + ni * 32 + fr) * IX_F32_PITCH + 2 * j + fg];
        acc[ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[ni], 0, 0, 0);
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int ni = 0; ni < 2; ++ni) {
    const long n = n0 + wn * 64 + ni * 32 + (lane & 31);
    if (n >= N) continue;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const long m = m0 + wm * 32 + ix_acc_row(i, lane);
      if (m < M) C[m * ldc + n] = acc[ni][i];
    }
  }
}

extern "C" int ix_gemm_f32_nt(const void* A, int a_dtype, long lda, const void* W, long ldw, void* C, long ldc,
                              long M, long N, long K, void* stream) {
  if (!A || !W || !C || M < 0 || N <= 0 || K <= 0) return IX_ERR_ARG;
  if (lda < K || ldw < K || ldc < N) return IX_ERR_ARG;
  if (a_dtype != IX_DT_F32 && a_dtype != IX_DT_BF16) return IX_DECLINED;
  if (M > 0x7fffffffL || N > 0x7fffffffL || K > 0x7fffffffL) return IX_DECLINED;
  if (M == 0) return IX_OK;
  const long gm = (M + IX_F32_BM - 1) / IX_F32_BM, gn = (N + IX_F32_BN - 1) / IX_F32_BN;
  if (gn > 65535) return IX_DECLINED;
  hipStream_t st = (hipStream_t)stream;
  if (a_dtype == IX_DT_BF16)
    hipLaunchKernelGGL((k_gemm_f32_nt<bf16_t>), dim3((unsigned)gm, (unsigned)gn), dim3(256), 0, st,
                       (const bf16_t*)A, lda, (const float*)W, ldw, (float*)C, ldc, (int)M, (int)N, (int)K);
  else
    hipLaunchKernelGGL((k_gemm_f32_nt<float>), dim3((unsigned)gm, (unsigned)gn), dim3(256), 0, st,
                       (const float*)A, lda, (const float*)W, ldw, (float*)C, ldc, (int)M, (int)N, (int)K);
  return ix_launch_status();
}
