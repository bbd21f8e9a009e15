// The one bf16 GEMM core every dense and expert matmul of this library runs.
//
//   C[m, n] = sum_k A[m, k] * W[n, k]        A [M, K] and W [N, K] both K-contiguous, fp32 accumulate
//
// The rounding schedule of one output element is fixed and is the same for every M, every tile
// shape and every caller (dense, expert fc1, expert fc2):
//   * one instruction, v_mfma_f32_32x32x16_bf16, activations always the A operand and weights
//     always the B operand;
//   * K is walked in tiles of 64; inside a tile, MFMA step s = 0..3 consumes
//     k = {s*8 .. s*8+7} (lane group 0) and {32+s*8 .. 32+s*8+7} (lane group 1);
//   * steps and tiles accumulate left to right into one fp32 accumulator (no split-K, no
//     second accumulator, no atomics); columns past K read as zero;
//   * one rounding to bf16 at the store (or the fused epilogue's documented chain).
// Tile shapes (BM x BN per workgroup, WM x WN waves) only decide which workgroup owns an
// element, never its arithmetic; that premise is the counterpart of the reference's
// "sequential over MMA k-steps" (ops/collectives/pik/csrc/fused_leaftree.cu:12-19).
#pragma once
#include "ix_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 ix_bf16x8;
typedef __attribute__((ext_vector_type(16))) float ix_f32x16;

#define IX_BK 64

// LDS tile: [rows][64] bf16, row pitch 128 B, 16-byte chunk c of row r stored at chunk slot
// c ^ (r & 7) so that both the staging stores and the MFMA fragment reads spread over banks.
__device__ __forceinline__ int ix_lds_off(int row, int chunk) { return row * 128 + ((chunk ^ (row & 7)) << 4); }

// Accumulator register i of lane l in a 32x32 tile holds row (i/4)*8 + (l/32)*4 + (i%4), column l%32.
__device__ __forceinline__ int ix_acc_row(int i, int lane) { return ((i >> 2) << 3) + ((lane >> 5) << 2) + (i & 3); }

template <int BM, int BN, int WM, int WN>
struct IxGemmCfg {
  static constexpr int NT = WM * WN * 64;
  static constexpr int TM = BM / WM, TN = BN / WN;
  static constexpr int MI = TM / 32, NI = TN / 32;
  static constexpr int A_CH = BM * 8 / NT;  // 16-byte chunks staged per thread per k-tile
  static constexpr int B_CH = BN * 8 / NT;
  static constexpr int LDS_BYTES = 2 * (BM + BN) * 128;
  static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "wave tile must be MFMA multiples");
  static_assert((BM * 8) % NT == 0 && (BN * 8) % NT == 0, "staging must divide evenly");
};

// Row sources for the A operand. Plain: row r of a [M, lda] matrix. Gather: row index table.
struct IxRowsPlain {
  const bf16_t* base;
  long ld;
  long m_lo, m_hi;  // valid global rows [m_lo, m_hi)
  __device__ __forceinline__ const bf16_t* row(long m) const { return (m < m_hi) ? base + m * ld : nullptr; }
};
struct IxRowsGather {
  const bf16_t* base;
  long ld;
  const int* index;  // index[m] = source row of tile row m
  long m_lo, m_hi;
  __device__ __forceinline__ const bf16_t* row(long m) const {
    return (m < m_hi) ? base + (long)index[m] * ld : nullptr;
  }
};

// Weight-row sources for the B operand: tile row r -> pointer to that weight row, or nullptr.
struct IxWRowsPlain {
  const bf16_t* base;  // first weight row of the tile
  long ld;
  int n_valid;
  __device__ __forceinline__ const bf16_t* row(int r) const { return (r < n_valid) ? base + (long)r * ld : nullptr; }
};
// Gate/up interleave for a fused SwiGLU epilogue: each 64-row group of the tile holds 32 gate
// rows (weight rows n0h + 32*w + c) followed by the 32 matching up rows (F + the same), so one
// wave's two MFMA tiles are a gate tile and its up tile with identical lane layout.
struct IxWRowsGlu {
  const bf16_t* base;  // expert's [2F, K] fc1 weight
  long ld;
  int n0h;  // first gate column of the tile
  int F;    // intermediate width
  __device__ __forceinline__ const bf16_t* row(int r) const {
    const int w = r >> 6, half = (r >> 5) & 1, c = r & 31;
    const int col = n0h + w * 32 + c;
    return (col < F) ? base + ((long)half * F + col) * ld : nullptr;
  }
};

// Main loop: accumulates the BM x BN tile whose A rows are rows.row(m0 + r) and whose weight
// rows are wrows.row(r). acc[mi][ni] are the wave's 32x32 tiles.
template <typename Cfg, int BM, int BN, int WM, int WN, typename Rows, typename WRows>
__device__ __forceinline__ void ix_gemm_mainloop(const Rows& rows, long m0, const WRows& wrows, int K, char* lds,
                                                 ix_f32x16 (&acc)[Cfg::MI][Cfg::NI]) {
  constexpr int NT = Cfg::NT;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  char* ldsA[2] = {lds, lds + (BM + BN) * 128};
  char* ldsB[2] = {lds + BM * 128, lds + (BM + BN) * 128 + BM * 128};

  // Staging assignment: chunk q = tid + j*NT -> row q/8, 16-byte chunk q%8.
  const bf16_t* a_ptr[Cfg::A_CH];
  const bf16_t* b_ptr[Cfg::B_CH];
  int a_off[Cfg::A_CH], b_off[Cfg::B_CH];
#pragma unroll
  for (int j = 0; j < Cfg::A_CH; ++j) {
    const int q = tid + j * NT, r = q >> 3, c = q & 7;
    const bf16_t* p = rows.row(m0 + r);
    a_ptr[j] = p ? p + c * 8 : nullptr;
    a_off[j] = ix_lds_off(r, c);
  }
#pragma unroll
  for (int j = 0; j < Cfg::B_CH; ++j) {
    const int q = tid + j * NT, r = q >> 3, c = q & 7;
    const bf16_t* p = wrows.row(r);
    b_ptr[j] = p ? p + c * 8 : nullptr;
    b_off[j] = ix_lds_off(r, c);
  }
  const int kc = tid & 7;  // this thread's chunk column; chunk covers k = kc*8 .. kc*8+7 of the tile

  uint4 a_reg[Cfg::A_CH], b_reg[Cfg::B_CH];
  auto gload = [&](int k0) {
    const bool kin = (k0 + kc * 8) < K;  // K % 8 == 0: a chunk is entirely inside or outside
#pragma unroll
    for (int j = 0; j < Cfg::A_CH; ++j)
      a_reg[j] = (a_ptr[j] && kin) ? *reinterpret_cast<const uint4*>(a_ptr[j] + k0) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int j = 0; j < Cfg::B_CH; ++j)
      b_reg[j] = (b_ptr[j] && kin) ? *reinterpret_cast<const uint4*>(b_ptr[j] + k0) : make_uint4(0, 0, 0, 0);
  };
  auto lstore = [&](int buf) {
#pragma unroll
    for (int j = 0; j < Cfg::A_CH; ++j) *reinterpret_cast<uint4*>(ldsA[buf] + a_off[j]) = a_reg[j];
#pragma unroll
    for (int j = 0; j < Cfg::B_CH; ++j) *reinterpret_cast<uint4*>(ldsB[buf] + b_off[j]) = b_reg[j];
  };

  const int frow = lane & 31, fg = lane >> 5;
  const int KT = (K + IX_BK - 1) / IX_BK;
  gload(0);
  lstore(0);
  __syncthreads();
  for (int kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < KT) gload((kt + 1) * IX_BK);
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int chunk = fg * 4 + s;
      ix_bf16x8 af[Cfg::MI], bfr[Cfg::NI];
#pragma unroll
      for (int mi = 0; mi < Cfg::MI; ++mi) {
        const int r = wm * Cfg::TM + mi * 32 + frow;
        af[mi] = *reinterpret_cast<const ix_bf16x8*>(ldsA[buf] + ix_lds_off(r, chunk));
      }
#pragma unroll
      for (int ni = 0; ni < Cfg::NI; ++ni) {
        const int r = wn * Cfg::TN + ni * 32 + frow;
        bfr[ni] = *reinterpret_cast<const ix_bf16x8*>(ldsB[buf] + ix_lds_off(r, chunk));
      }
#pragma unroll
      for (int mi = 0; mi < Cfg::MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < Cfg::NI; ++ni)
          acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[mi], bfr[ni], acc[mi][ni], 0, 0, 0);
    }
    if (kt + 1 < KT) lstore(buf ^ 1);
    __syncthreads();
  }
}
