// The one bf16 GEMM core every dense and expert matmul of this library runs.
//
//   C[m, n] = sum_k X[m, k] * W[n, k]        X [M, K] and W [N, K] both K-contiguous, fp32 accumulate
//
// The rounding schedule of one output element is fixed and is the same for every M, every tile
// shape and every caller (dense, expert fc1, expert fc2):
//   * one instruction, v_mfma_f32_32x32x16_bf16, weights always the A operand (rows of the
//     instruction's 32x32 result) and activations always the B operand (its columns);
//   * K is walked in tiles of 64; inside a tile, MFMA step s = 0..3 consumes
//     k = {s*8 .. s*8+7} (lane group 0) and {32+s*8 .. 32+s*8+7} (lane group 1);
//   * steps and tiles accumulate left to right into one fp32 accumulator (no split-K, no
//     second accumulator, no atomics); columns past K read as zero;
//   * one rounding to bf16 at the store (or the fused epilogue's documented chain).
// Tile shapes (BM x BN per workgroup, WM x WN waves) only decide which workgroup owns an
// element, never its arithmetic; that premise is the counterpart of the reference's
// "sequential over MMA k-steps" (ops/collectives/pik/csrc/fused_leaftree.cu:12-19).
//
// Data movement: operand tiles go HBM -> LDS directly (buffer_load ... lds, 16 bytes per lane, no
// register staging), two LDS stages, one barrier per k-tile. Out-of-range rows and the K tail
// are handled by the buffer descriptor's range check (they read as zero), so the loop has no
// branches.
#pragma once
#include "ix_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 ix_bf16x8;
typedef __attribute__((ext_vector_type(16))) float ix_f32x16;
typedef __attribute__((address_space(3))) void ix_lds_void;

#define IX_BK 64
#define IX_OOB 0xFFFFFF00u  // a byte offset no buffer descriptor here admits

// LDS tile: [rows][64] bf16, row pitch 128 B; 16-byte chunk c of row r lives at slot c ^ (r & 7),
// so the MFMA fragment reads (32 consecutive rows, one chunk) spread over all banks.
__device__ __forceinline__ int ix_lds_off(int row, int chunk) { return row * 128 + ((chunk ^ (row & 7)) << 4); }

// Register i of lane l of a 32x32 accumulator holds result row (i/4)*8 + (l/32)*4 + (i%4)
// (a weight row, i.e. an output column n) and result column l%32 (a token m).
__device__ __forceinline__ int ix_acc_row(int i, int lane) { return ((i >> 2) << 3) + ((lane >> 5) << 2) + (i & 3); }

template <int BM_, int BN_, int WM_, int WN_>
struct IxGemmCfg {
  static constexpr int BM = BM_, BN = BN_, WM = WM_, WN = WN_;
  static constexpr int NT = WM * WN * 64;
  static constexpr int TM = BM / WM, TN = BN / WN;
  static constexpr int MI = TM / 32, NI = TN / 32;
  static constexpr int X_CH = BM * 8 / NT;  // 16-byte chunks fetched per thread per k-tile
  static constexpr int W_CH = BN * 8 / NT;
  static constexpr int STAGE_BYTES = (BM + BN) * 128;
  static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
  static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "wave tile must be MFMA multiples");
  static_assert((BM * 8) % NT == 0 && (BN * 8) % NT == 0, "fetch must divide evenly");
  static_assert(NT % 64 == 0 && (NT / 8) % 8 == 0, "a thread's k-chunk must not depend on the fetch index");
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t ix_make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), (short)0, (int)bytes, 0x00020000);
}

// Thread t fetches LDS chunk q = t + j*NT of each operand tile: tile row q/8, slot q%8, which
// holds k-chunk (q%8) ^ (row&7). These helpers give the row and the byte offset of that chunk
// inside a row; the caller turns the row into a buffer offset (or IX_OOB for a missing row).
template <typename Cfg>
__device__ __forceinline__ int ix_fetch_row(int j) { return (threadIdx.x + j * Cfg::NT) >> 3; }
__device__ __forceinline__ int ix_fetch_kchunk() { return (threadIdx.x & 7) ^ ((threadIdx.x >> 3) & 7); }

// Main loop. x_voff[j] / w_voff[j]: byte offset (row start + this thread's k-chunk) of fetch j
// into the activation / weight buffer, or IX_OOB. acc[mi][ni]: tokens mi*32.., outputs ni*32..
template <typename Cfg, typename XOff, typename WOff, typename Acc>
__device__ __forceinline__ void ix_gemm_mainloop(__amdgpu_buffer_rsrc_t x_rsrc, const XOff& x_voff,
                                                 __amdgpu_buffer_rsrc_t w_rsrc, const WOff& w_voff, int K,
                                                 char* lds, Acc& acc) {
  constexpr int NT = Cfg::NT, BM = Cfg::BM;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
  const int kc = ix_fetch_kchunk();
  const int KT = (K + IX_BK - 1) / IX_BK;
  // stage layout: [X tile: BM rows][W tile: BN rows]
  const int wave_chunk_byte = (wave * 64) * 16;

  // Only the last k-tile can be partial; its out-of-range chunks are sent out of the buffer's range.
  uint32_t x_last[Cfg::X_CH], w_last[Cfg::W_CH];
  {
    const bool kin = ((KT - 1) * IX_BK + kc * 8) < K;  // K % 8 == 0: a chunk is entirely in or out
#pragma unroll
    for (int j = 0; j < Cfg::X_CH; ++j) x_last[j] = kin ? x_voff[j] : IX_OOB;
#pragma unroll
    for (int j = 0; j < Cfg::W_CH; ++j) w_last[j] = kin ? w_voff[j] : IX_OOB;
  }
  auto fetch = [&](int kt, int stage, const uint32_t* xv, const uint32_t* wv) {
    const int soff = kt * IX_BK * 2;
    char* sbase = lds + stage * Cfg::STAGE_BYTES + wave_chunk_byte;
#pragma unroll
    for (int j = 0; j < Cfg::X_CH; ++j)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (ix_lds_void*)(sbase + j * NT * 16), 16, xv[j], soff, 0, 0);
#pragma unroll
    for (int j = 0; j < Cfg::W_CH; ++j)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(w_rsrc, (ix_lds_void*)(sbase + BM * 128 + j * NT * 16), 16, wv[j],
                                               soff, 0, 0);
  };

  const int frow = lane & 31, fg = lane >> 5;
  int x_foff[Cfg::MI], w_foff[Cfg::NI];  // fragment byte offsets for step 0; step s: ^ (s << 4)
#pragma unroll
  for (int mi = 0; mi < Cfg::MI; ++mi) x_foff[mi] = ix_lds_off(wm * Cfg::TM + mi * 32 + frow, fg * 4);
#pragma unroll
  for (int ni = 0; ni < Cfg::NI; ++ni) w_foff[ni] = BM * 128 + ix_lds_off(wn * Cfg::TN + ni * 32 + frow, fg * 4);

  if (KT == 1) fetch(0, 0, x_last, w_last); else fetch(0, 0, x_voff, w_voff);
  for (int kt = 0; kt < KT; ++kt) {
    const int stage = kt & 1;
    // tile kt has landed (it is the only fetch in flight) and everyone is done with stage^1
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
    __syncthreads();
    if (kt + 2 < KT) fetch(kt + 1, stage ^ 1, x_voff, w_voff);
    else if (kt + 1 < KT) fetch(kt + 1, stage ^ 1, x_last, w_last);
    const char* sb = lds + stage * Cfg::STAGE_BYTES;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      ix_bf16x8 xf[Cfg::MI], wf[Cfg::NI];
      // chunk fg*4+s sits at slot (fg*4+s) ^ (row&7): flipping bits 0-1 of the chunk index flips
      // the same bits of the slot, i.e. byte offset ^ (s << 4)
#pragma unroll
      for (int mi = 0; mi < Cfg::MI; ++mi)
        xf[mi] = *reinterpret_cast<const ix_bf16x8*>(sb + (x_foff[mi] ^ (s << 4)));
#pragma unroll
      for (int ni = 0; ni < Cfg::NI; ++ni)
        wf[ni] = *reinterpret_cast<const ix_bf16x8*>(sb + (w_foff[ni] ^ (s << 4)));
#pragma unroll
      for (int mi = 0; mi < Cfg::MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < Cfg::NI; ++ni)
          acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[ni], xf[mi], acc[mi][ni], 0, 0, 0);
    }
  }
}

template <typename Cfg, typename Acc>
__device__ __forceinline__ void ix_acc_zero(Acc& acc) {
#pragma unroll
  for (int mi = 0; mi < Cfg::MI; ++mi)
#pragma unroll
    for (int ni = 0; ni < Cfg::NI; ++ni)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mi][ni][i] = 0.0f;
}

// Store 4 consecutive output columns of one token (8 bytes when aligned and in range).
__device__ __forceinline__ void ix_store4_bf16(bf16_t* __restrict__ p, int valid, bool vec, float a, float b,
                                               float c, float d) {
  if (vec && valid >= 4) {
    uint2 u;
    u.x = ix_pack_bf2(a, b);
    u.y = ix_pack_bf2(c, d);
    *reinterpret_cast<uint2*>(p) = u;
  } else {
    if (valid > 0) p[0] = ix_f2bf(a);
    if (valid > 1) p[1] = ix_f2bf(b);
    if (valid > 2) p[2] = ix_f2bf(c);
    if (valid > 3) p[3] = ix_f2bf(d);
  }
}
