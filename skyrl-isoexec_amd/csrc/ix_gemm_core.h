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
// register staging) through a ring of LDS stages, one barrier per stage. Out-of-range rows and
// the K tail are handled by the buffer descriptor's range check (they read as zero), so the loop
// has no branches.
#pragma once
#include "ix_common.h"
#include <type_traits>

typedef __attribute__((ext_vector_type(8))) __bf16 ix_bf16x8;
typedef __attribute__((ext_vector_type(16))) float ix_f32x16;
typedef __attribute__((address_space(3))) void ix_lds_void;

#define IX_BK 64
#define IX_OOB 0x7FFFF000u  // a byte offset no buffer descriptor here admits (all are < 1 GiB)

// LDS tiles are [rows][k] bf16 with the 16-byte chunks of a row permuted by an XOR swizzle so that
// an MFMA fragment read (32 consecutive rows, one chunk per lane group) spreads over the banks:
//   full k-tile, row pitch 128 B: chunk c of row r at slot c ^ ix_swz8(r)
//   half k-tile, row pitch  64 B: chunk c of row r at slot c ^ ix_swz4(r)
// The two functions were picked by measuring ds_read_b128 throughput on gfx950 for every XOR of two
// shifts of r: these reach ~188 B/clk/CU, where r&7 / no swizzle reach 118 / 32 (full) and 63 (half).
__device__ __forceinline__ int ix_swz8(int r) { return (r >> 1) & 7; }
__device__ __forceinline__ int ix_swz4(int r) { return (r >> 3) & 3; }
__device__ __forceinline__ int ix_lds_off(int row, int chunk) { return row * 128 + ((chunk ^ ix_swz8(row)) << 4); }

// Register i of lane l of a 32x32 accumulator holds result row (i/4)*8 + (l/32)*4 + (i%4)
// (a weight row, i.e. an output column n) and result column l%32 (a token m).
__device__ __forceinline__ int ix_acc_row(int i, int lane) { return ((i >> 2) << 3) + ((lane >> 5) << 2) + (i & 3); }

// PW_ > 0: PW_ extra waves that only fetch (pipeline D below); NT counts the computing threads, NTT all of them.
template <int BM_, int BN_, int WM_, int WN_, int PW_ = 0>
struct IxGemmCfg {
  static constexpr int BM = BM_, BN = BN_, WM = WM_, WN = WN_, PW = PW_;
  static constexpr int NT = WM * WN * 64;
  static constexpr int NTT = NT + PW * 64;
  static constexpr int TM = BM / WM, TN = BN / WN;
  static constexpr int MI = TM / 32, NI = TN / 32;
  static constexpr int X_CH = BM * 8 / NT;  // 16-byte chunks fetched per thread per k-tile
  static constexpr int W_CH = BN * 8 / NT;
  static constexpr int STAGE_BYTES = (BM + BN) * 128;
  // Pipeline: a ring of four half-k-tile stages when the half-stage fetch divides evenly over the
  // threads, else a ring of FULL_STAGES whole-k-tile stages (the 32-row decode tile).
  static constexpr bool HALF_RING = ((BM * 4) % NT == 0) && ((BN * 4) % NT == 0);
#ifndef IX_FULL_STAGES_MAX
#define IX_FULL_STAGES_MAX 4
#endif
  // as many whole stages as fit in the 160 KiB of LDS, at most IX_FULL_STAGES_MAX, at least 3
  static constexpr int FULL_STAGES = (IX_FULL_STAGES_MAX * STAGE_BYTES <= 160 * 1024) ? IX_FULL_STAGES_MAX : 3;
#define IX_HALF_STAGES_MAX 5
  // as many half-stages as fit in the 160 KiB of LDS, at most IX_HALF_STAGES_MAX, at least 4
  static constexpr int HALF_STAGES =
      (IX_HALF_STAGES_MAX * (STAGE_BYTES / 2) <= 160 * 1024) ? IX_HALF_STAGES_MAX : 4;
  // Square tiles may instead use a ring of whole-k-tile operand units (pipeline C).
  // Five units (the two being consumed, three in flight) for every square tile: the 256-row tile fills the LDS
  // with them, and the 128-row tile's 80 KiB let two workgroups share a CU, each behind its own barrier (measured:
  // +27 % over nine units and one workgroup per CU).
#ifndef IX_UNITS_MAX
#define IX_UNITS_MAX 5
#endif
  static constexpr int UNITS = (160 * 1024) / (BM * 128) > IX_UNITS_MAX ? IX_UNITS_MAX : (160 * 1024) / (BM * 128);
  static constexpr bool UNIT_RING = BM == BN && UNITS >= 5 && X_CH >= 1;
  // Pipeline D (fetching waves): as many whole stages as fit in 144 KiB; a small tile stops at
  // IX_SPLIT_STAGES_SMALL so that two workgroups share a CU.
#ifndef IX_SPLIT_STAGES_SMALL
#define IX_SPLIT_STAGES_SMALL 6
#endif
  static constexpr int SPLIT_STAGES =
      (144 * 1024) / STAGE_BYTES > IX_SPLIT_STAGES_SMALL ? IX_SPLIT_STAGES_SMALL : (144 * 1024) / STAGE_BYTES;
  static constexpr int LDS_BYTES =
      PW > 0 ? SPLIT_STAGES * STAGE_BYTES
             : (UNIT_RING ? UNITS * BM * 128
                          : (HALF_RING ? HALF_STAGES * (STAGE_BYTES / 2) : FULL_STAGES * STAGE_BYTES));
  static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "wave tile must be MFMA multiples");
  static_assert((BM * 8) % NT == 0 && (BN * 8) % NT == 0, "fetch must divide evenly");
  static_assert(NT % 64 == 0, "whole waves");
};

// Raw buffer descriptor (stride 0): base, size in bytes, dword 3 = 32-bit untyped data format.
typedef __attribute__((ext_vector_type(4))) int ix_rsrc_t;
__device__ __forceinline__ ix_rsrc_t ix_make_rsrc(const void* base, uint32_t bytes) {
  const uint64_t b = reinterpret_cast<uint64_t>(base);
  ix_rsrc_t r;
  r.x = __builtin_amdgcn_readfirstlane((int)(uint32_t)b);
  r.y = __builtin_amdgcn_readfirstlane((int)(uint32_t)((b >> 32) & 0xffffu));
  r.z = __builtin_amdgcn_readfirstlane((int)bytes);
  r.w = 0x00020000;
  return r;
}

// 16 bytes per lane, memory -> LDS without passing through registers: lane l's data lands at LDS
// byte address lds_addr + 16*l (lds_addr wave-uniform, carried in M0). Written as inline assembly so
// that the compiler does not count these loads: it would otherwise force "all loads done" before
// every LDS read, and the ring of stages below relies on waiting only for the oldest group
// (explicit s_waitcnt vmcnt(N); vector loads retire in order).
//
// Wait states the compiler does not place for an instruction it cannot see into (asm_hazards.py checks the generated
// code for both): M0 written by a scalar instruction needs one before the load reads it, and a scalar register written
// by a VECTOR instruction (v_readfirstlane, or v_readlane: the reload of a spilled scalar register) needs five before a
// vector-memory instruction reads it as descriptor word or scalar offset -- the load would otherwise go to the address
// the old value gives, and the scalar offset is not even range-checked. IDLE = 0 gives the one state for M0 and is right
// where every scalar operand comes from scalar arithmetic; a kernel short of scalar registers takes IDLE = 3.
template <int IDLE = 0>
__device__ __forceinline__ void ix_dma16(ix_rsrc_t rsrc, uint32_t lds_addr, uint32_t voff, int soff) {
  static_assert(IDLE == 0 || IDLE == 3, "one wait state for M0, or five for scalar operands a vector instruction wrote");
  if constexpr (IDLE == 0)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
                 : "memory", "m0");
  else
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
                 : "memory", "m0");
}
// Stores through a descriptor: an offset outside its range (IX_OOB, or a row past the tile) is dropped by the hardware,
// so a predicated store needs no branch.
typedef __attribute__((ext_vector_type(4))) uint32_t ix_u32x4;
__device__ __forceinline__ ix_rsrc_t ix_rsrc_scalar(ix_rsrc_t r) {  // a descriptor operand must sit in scalar registers
  r.x = __builtin_amdgcn_readfirstlane(r.x);
  r.y = __builtin_amdgcn_readfirstlane(r.y);
  r.z = __builtin_amdgcn_readfirstlane(r.z);
  r.w = __builtin_amdgcn_readfirstlane(r.w);
  return r;
}
// NT: the non-temporal hint -- the line is not kept for a reader that comes soon (for outputs far larger than the
// caches, written once while the same caches feed the operand stream).
template <bool NT = false>
__device__ __forceinline__ void ix_buffer_store16(uint4 v, ix_rsrc_t rsrc, uint32_t voff) {
  const ix_u32x4 d = {v.x, v.y, v.z, v.w};
  // the two idle states after it keep the next instruction from overwriting the data registers while the store still
  // reads them (the compiler would place them itself for a store it knows; it does not look into this one); the five
  // before it let the descriptor words, which a vector instruction has just moved into scalar registers, arrive
  if constexpr (NT)
    asm volatile("s_nop 4\n\tbuffer_store_dwordx4 %0, %1, %2, 0 offen nt\n\ts_nop 1"
                 :
                 : "v"(d), "v"(voff), "s"(ix_rsrc_scalar(rsrc))
                 : "memory");
  else
    asm volatile("s_nop 4\n\tbuffer_store_dwordx4 %0, %1, %2, 0 offen\n\ts_nop 1"
                 :
                 : "v"(d), "v"(voff), "s"(ix_rsrc_scalar(rsrc))
                 : "memory");
}
__device__ __forceinline__ void ix_buffer_store4(uint32_t v, ix_rsrc_t rsrc, uint32_t voff) {
  asm volatile("s_nop 4\n\tbuffer_store_dword %0, %1, %2, 0 offen" : : "v"(v), "v"(voff), "s"(ix_rsrc_scalar(rsrc)) : "memory");
}
// A 4-byte load the compiler does not count (see ix_dma16 for why): the value is NOT there when the statement ends.
// The caller's own wait retires it (vector-memory operations retire in order: any later s_waitcnt vmcnt(n) with at least
// n of them issued after this load), and the value is taken into use through ix_landed() after that wait; until then
// nothing may read or move the register. asm_hazards.py checks all three in the generated code of every build.
__device__ __forceinline__ uint32_t ix_load4_uncounted(const void* base, uint32_t byte_off) {
  uint32_t v;
  asm volatile("global_load_dword %0, %1, %2" : "=&v"(v) : "v"(byte_off), "s"(base));
  return v;
}
__device__ __forceinline__ uint32_t ix_landed(uint32_t v) {
  asm volatile("; ix_landed %0" : "+v"(v));
  return v;
}
// A point the eight values must have been computed by, and that volatile assembly after it cannot pass: keeps the
// compiler from issuing a long run of accumulator reads first and the arithmetic on them afterwards (hundreds of live
// registers).
__device__ __forceinline__ void ix_pin8(const uint32_t (&v)[8]) {
  asm volatile("" : : "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]), "v"(v[4]), "v"(v[5]), "v"(v[6]), "v"(v[7]));
}
__device__ __forceinline__ uint32_t ix_lds_addr(const char* p) {
  return (uint32_t)reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) char*)p);
}

// s_waitcnt immediate for "at most N vector-memory operations outstanding" (expcnt, lgkmcnt unconstrained).
#define IX_VMCNT(N) (((N) & 15) | (((N) >> 4) << 14) | 0x0F70)

// ---- pipeline A: a ring of FULL_STAGES stages, one full k-tile (64) each --------------------------
// Thread t fetches LDS chunk q = t + j*NT of each operand tile: tile row q/8, slot q%8, which
// holds k-chunk (q%8) ^ ix_swz8(row). Every iteration issues the same number of loads (past the end they
// fall outside the buffer range), so "tile kt has landed" is one constant wait.
template <typename Cfg, typename XRow, typename WRow, typename Acc>
__device__ __forceinline__ void ix_gemm_mainloop_full(ix_rsrc_t x_rsrc, const XRow& x_row,
                                                      ix_rsrc_t w_rsrc, const WRow& w_row, int K,
                                                      char* lds, Acc& acc) {
  constexpr int NT = Cfg::NT, BM = Cfg::BM, S = Cfg::FULL_STAGES;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
  const int KT = (K + IX_BK - 1) / IX_BK;
  const uint32_t lds_base = __builtin_amdgcn_readfirstlane(ix_lds_addr(lds) + (wave * 64) * 16);
  const int K2 = K * 2;

  // fetch j of this thread: tile row (tid + j*NT)/8, slot tid%8, i.e. k-chunk slot ^ swz8(row)
  uint32_t x_voff[Cfg::X_CH], w_voff[Cfg::W_CH];
  int x_kb[Cfg::X_CH], w_kb[Cfg::W_CH];
#pragma unroll
  for (int j = 0; j < Cfg::X_CH; ++j) {
    const int r = (tid + j * NT) >> 3;
    x_kb[j] = ((tid & 7) ^ ix_swz8(r)) * 16;
    x_voff[j] = x_row(r) + x_kb[j];
  }
#pragma unroll
  for (int j = 0; j < Cfg::W_CH; ++j) {
    const int r = (tid + j * NT) >> 3;
    w_kb[j] = ((tid & 7) ^ ix_swz8(r)) * 16;
    w_voff[j] = w_row(r) + w_kb[j];
  }

  auto issue = [&](int kt) {
    const int soff = kt * IX_BK * 2;
    const uint32_t sbase = lds_base + (kt % S) * Cfg::STAGE_BYTES;
    // chunks at or past K (the tail of the last tile, and whole tiles past the end) go out of range
#pragma unroll
    for (int j = 0; j < Cfg::X_CH; ++j) {
      const uint32_t dead = (uint32_t)((K2 - 1 - (soff + x_kb[j])) >> 31) & IX_OOB;
      ix_dma16(x_rsrc, sbase + j * NT * 16, x_voff[j] | dead, soff);
    }
#pragma unroll
    for (int j = 0; j < Cfg::W_CH; ++j) {
      const uint32_t dead = (uint32_t)((K2 - 1 - (soff + w_kb[j])) >> 31) & IX_OOB;
      ix_dma16(w_rsrc, sbase + BM * 128 + j * NT * 16, w_voff[j] | dead, soff);
    }
  };

  const int frow = lane & 31, fg = lane >> 5;
  int x_foff[Cfg::MI], w_foff[Cfg::NI];  // fragment byte offsets for step 0; step s: ^ (s << 4)
#pragma unroll
  for (int mi = 0; mi < Cfg::MI; ++mi) x_foff[mi] = ix_lds_off(wm * Cfg::TM + mi * 32 + frow, fg * 4);
#pragma unroll
  for (int ni = 0; ni < Cfg::NI; ++ni) w_foff[ni] = BM * 128 + ix_lds_off(wn * Cfg::TN + ni * 32 + frow, fg * 4);

#pragma unroll
  for (int p = 0; p < S - 1; ++p) issue(p);
  for (int kt = 0; kt < KT; ++kt) {
    __builtin_amdgcn_s_waitcnt(IX_VMCNT((S - 2) * (Cfg::X_CH + Cfg::W_CH)));
    __syncthreads();
    issue(kt + S - 1);  // into the stage consumed in iteration kt-1
    const char* sb = lds + (kt % S) * Cfg::STAGE_BYTES;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      ix_bf16x8 xf[Cfg::MI], wf[Cfg::NI];
      // chunk fg*4+s sits at slot (fg*4+s) ^ swz8(row): flipping bits 0-1 of the chunk index flips
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
  __builtin_amdgcn_s_waitcnt(IX_VMCNT(0));  // drain the out-of-range tail fetches before LDS is reused
}

// ---- pipeline B: a ring of HALF_STAGES (4 or 5) LDS stages of half a k-tile each ------------------
// Half h of k-tile kt holds the 16-byte k-chunks {2h, 2h+1, 4+2h, 5+2h}: exactly what MFMA steps
// s = 2h and 2h+1 consume (lane group 0: chunk s, lane group 1: chunk 4+s), so the K order of pipeline
// A is kept while a fetch is issued three half-tiles ahead of its use. Row pitch 64 B; local chunk lc
// of row r sits at slot lc ^ ((r>>1)&3). Every iteration issues the same number of loads (past the end
// they fall outside the buffer range), so "all but the newest two groups have landed" is one constant.
template <typename Cfg, typename XRow, typename WRow, typename Acc>
__device__ __forceinline__ void ix_gemm_mainloop_h4(ix_rsrc_t x_rsrc, const XRow& x_row,
                                                    ix_rsrc_t w_rsrc, const WRow& w_row, int K,
                                                    char* lds, Acc& acc) {
  constexpr int NT = Cfg::NT, BM = Cfg::BM, BN = Cfg::BN;
  constexpr int XH = BM * 4 / NT, WH = BN * 4 / NT;  // loads per thread per half-stage
  constexpr int HS = (BM + BN) * 64;                 // bytes per half-stage
  static_assert(Cfg::HALF_RING && (NT / 4) % 32 == 0, "half-stage fetch must divide, swizzle independent of j");
  constexpr int NS = Cfg::HALF_STAGES;               // ring length; fetches run NS-1 half-tiles ahead
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
  const int lc = (tid & 3) ^ ix_swz4(tid >> 2);         // local chunk this thread fetches (same for every j)
  const int cb = ((lc & 1) | ((lc >> 1) << 2)) * 16;    // its byte offset in a row for half 0
  const int NH = 2 * ((K + IX_BK - 1) / IX_BK);
  const uint32_t lds_base = __builtin_amdgcn_readfirstlane(ix_lds_addr(lds) + (wave * 64) * 16);
  const int K2 = K * 2;

  uint32_t x_voff[XH], w_voff[WH];
#pragma unroll
  for (int j = 0; j < XH; ++j) x_voff[j] = x_row((tid + j * NT) >> 2) + cb;
#pragma unroll
  for (int j = 0; j < WH; ++j) w_voff[j] = w_row((tid + j * NT) >> 2) + cb;

  auto issue = [&](int i) {
    const int soff = (i >> 1) * (IX_BK * 2) + (i & 1) * 32;
    // chunks at or past K (the tail of the last tile, and whole half-tiles past the end) go out of range
    const uint32_t dead = (uint32_t)((K2 - 1 - (soff + cb)) >> 31) & IX_OOB;
    const uint32_t sbase = lds_base + (i % NS) * HS;
#pragma unroll
    for (int j = 0; j < XH; ++j) ix_dma16(x_rsrc, sbase + j * NT * 16, x_voff[j] | dead, soff);
#pragma unroll
    for (int j = 0; j < WH; ++j) ix_dma16(w_rsrc, sbase + BM * 64 + j * NT * 16, w_voff[j] | dead, soff);
  };

  const int frow = lane & 31, fg = lane >> 5;
  int x_foff[Cfg::MI], w_foff[Cfg::NI];
#pragma unroll
  for (int mi = 0; mi < Cfg::MI; ++mi) {
    const int r = wm * Cfg::TM + mi * 32 + frow;
    x_foff[mi] = r * 64 + (((fg * 2) ^ ix_swz4(r)) << 4);
  }
#pragma unroll
  for (int ni = 0; ni < Cfg::NI; ++ni) {
    const int r = wn * Cfg::TN + ni * 32 + frow;
    w_foff[ni] = BM * 64 + r * 64 + (((fg * 2) ^ ix_swz4(r)) << 4);
  }

  // Software pipeline: the fragments of a step are read from LDS while the previous step's MFMAs
  // run, and the wait + barrier that publishes the next half-tile sits between the two steps of an
  // iteration, so its latency hides behind the second step's MFMAs.
  ix_bf16x8 xa[Cfg::MI], wa[Cfg::NI], xb[Cfg::MI], wb[Cfg::NI];
  auto frags = [&](const char* sb, int ls, ix_bf16x8* xf, ix_bf16x8* wf) {
#pragma unroll
    for (int mi = 0; mi < Cfg::MI; ++mi) xf[mi] = *reinterpret_cast<const ix_bf16x8*>(sb + (x_foff[mi] ^ (ls << 4)));
#pragma unroll
    for (int ni = 0; ni < Cfg::NI; ++ni) wf[ni] = *reinterpret_cast<const ix_bf16x8*>(sb + (w_foff[ni] ^ (ls << 4)));
  };
  auto mfmas = [&](const ix_bf16x8* xf, const ix_bf16x8* wf) {
#pragma unroll
    for (int mi = 0; mi < Cfg::MI; ++mi)
#pragma unroll
      for (int ni = 0; ni < Cfg::NI; ++ni)
        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[ni], xf[mi], acc[mi][ni], 0, 0, 0);
  };

#pragma unroll
  for (int p = 0; p < NS - 1; ++p) issue(p);
  __builtin_amdgcn_s_waitcnt(IX_VMCNT((NS - 2) * (XH + WH)));  // half-tile 0 has landed
  __syncthreads();
  frags(lds, 0, xa, wa);
  for (int i = 0; i < NH; ++i) {
    const char* sb = lds + (i % NS) * HS;
    // sched_barrier(0): keep the compiler's scheduler from sinking the LDS reads below the MFMAs
    frags(sb, 1, xb, wb);
    __builtin_amdgcn_sched_barrier(0);
    mfmas(xa, wa);
    __builtin_amdgcn_sched_barrier(0);
    // half-tile i+1 has landed once at most the NS-3 newer groups are still in flight; after the
    // barrier every wave is past iteration i-1, whose stage the next fetch overwrites
    __builtin_amdgcn_s_waitcnt(IX_VMCNT((NS - 3) * (XH + WH)));
    __syncthreads();
    issue(i + NS - 1);
    frags(lds + ((i + 1) % NS) * HS, 0, xa, wa);
    __builtin_amdgcn_sched_barrier(0);
    mfmas(xb, wb);
    __builtin_amdgcn_sched_barrier(0);
  }
  __builtin_amdgcn_s_waitcnt(IX_VMCNT(0));  // drain the out-of-range tail fetches before LDS is reused
}

// ---- pipeline C: a ring of whole-k-tile OPERAND units (square tiles only) --------------------------
// Unit u = 2*kt holds the W rows of k-tile kt, unit 2*kt+1 its X rows; each is BM rows of 128 bytes, so
// every fetch moves whole 128-byte lines. A W unit is therefore issued two k-tiles before its use and an X unit
// one and a half: the weights are the operand that comes from HBM, the activations are shared and cached. The ring holds NU units: the two being consumed and NU-2 in
// flight. One barrier per k-tile: after it every wave is done with k-tile kt-1, whose two slots take the
// next two units. The K order is that of pipeline A.
template <typename Cfg, typename XRow, typename WRow, typename Acc>
__device__ __forceinline__ void ix_gemm_mainloop_units(ix_rsrc_t x_rsrc, const XRow& x_row,
                                                       ix_rsrc_t w_rsrc, const WRow& w_row, int K,
                                                       char* lds, Acc& acc) {
  constexpr int NT = Cfg::NT, CH = Cfg::X_CH, UNIT = Cfg::BM * 128, NU = Cfg::UNITS;
  static_assert(Cfg::BM == Cfg::BN && NU >= 5, "operand ring needs square tiles and five units");
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
  const int KT = (K + IX_BK - 1) / IX_BK;
  const uint32_t lds_base = __builtin_amdgcn_readfirstlane(ix_lds_addr(lds) + (wave * 64) * 16);
  const int K2 = K * 2;

  uint32_t x_voff[CH], w_voff[CH];
  int kb[CH];
#pragma unroll
  for (int j = 0; j < CH; ++j) {
    const int r = (tid + j * NT) >> 3;
    kb[j] = ((tid & 7) ^ ix_swz8(r)) * 16;
    x_voff[j] = x_row(r) + kb[j];
    w_voff[j] = w_row(r) + kb[j];
  }
  // unit u -> slot u % NU, tracked incrementally
  auto issue = [&](ix_rsrc_t rsrc, const uint32_t (&voff)[CH], int kt, int slot) {
    const int soff = kt * IX_BK * 2;
    const uint32_t sbase = lds_base + slot * UNIT;
#pragma unroll
    for (int j = 0; j < CH; ++j) {
      const uint32_t dead = (uint32_t)((K2 - 1 - (soff + kb[j])) >> 31) & IX_OOB;
      ix_dma16(rsrc, sbase + j * NT * 16, voff[j] | dead, soff);
    }
  };
  const int frow = lane & 31, fg = lane >> 5;
  int x_foff[Cfg::MI], w_foff[Cfg::NI];
#pragma unroll
  for (int mi = 0; mi < Cfg::MI; ++mi) x_foff[mi] = ix_lds_off(wm * Cfg::TM + mi * 32 + frow, fg * 4);
#pragma unroll
  for (int ni = 0; ni < Cfg::NI; ++ni) w_foff[ni] = ix_lds_off(wn * Cfg::TN + ni * 32 + frow, fg * 4);

  ix_bf16x8 xa[Cfg::MI], wa[Cfg::NI], xb[Cfg::MI], wb[Cfg::NI];
  auto frags = [&](const char* xs, const char* ws, int s, ix_bf16x8* xf, ix_bf16x8* wf) {
#pragma unroll
    for (int mi = 0; mi < Cfg::MI; ++mi) xf[mi] = *reinterpret_cast<const ix_bf16x8*>(xs + (x_foff[mi] ^ (s << 4)));
#pragma unroll
    for (int ni = 0; ni < Cfg::NI; ++ni) wf[ni] = *reinterpret_cast<const ix_bf16x8*>(ws + (w_foff[ni] ^ (s << 4)));
  };
  auto mfmas = [&](const ix_bf16x8* xf, const ix_bf16x8* wf) {
#pragma unroll
    for (int mi = 0; mi < Cfg::MI; ++mi)
#pragma unroll
      for (int ni = 0; ni < Cfg::NI; ++ni)
        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[ni], xf[mi], acc[mi][ni], 0, 0, 0);
  };

  // prologue: units 0 .. NU-3
  int is = 0;  // slot of the next unit to issue
#pragma unroll
  for (int u = 0; u < NU - 2; ++u) {
    if (u & 1) issue(x_rsrc, x_voff, u >> 1, is); else issue(w_rsrc, w_voff, u >> 1, is);
    is = is + 1 == NU ? 0 : is + 1;
  }
  int cs = 0;            // slot of the W unit being consumed
  int nu = NU - 2;       // index of the next unit to issue
  for (int kt = 0; kt < KT; ++kt) {
    __builtin_amdgcn_s_waitcnt(IX_VMCNT((NU - 4) * CH));  // units 2kt and 2kt+1 have landed
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      if (nu & 1) issue(x_rsrc, x_voff, nu >> 1, is); else issue(w_rsrc, w_voff, nu >> 1, is);
      is = is + 1 == NU ? 0 : is + 1;
      ++nu;
    }
    const char* ws = lds + cs * UNIT;
    const int xsl = cs + 1 == NU ? 0 : cs + 1;
    const char* xs = lds + xsl * UNIT;
    cs = xsl + 1 == NU ? 0 : xsl + 1;
    // The last quarter of k-tile kt-1 (fragments read before the barrier) is multiplied while the first
    // fragments of k-tile kt travel from LDS: the matrix pipeline has work on both sides of the barrier.
    frags(xs, ws, 0, xa, wa);
    __builtin_amdgcn_sched_barrier(0);
    if (kt > 0) mfmas(xb, wb);
    __builtin_amdgcn_sched_barrier(0);
    frags(xs, ws, 1, xb, wb);
    __builtin_amdgcn_sched_barrier(0);
    mfmas(xa, wa);
    __builtin_amdgcn_sched_barrier(0);
    frags(xs, ws, 2, xa, wa);
    __builtin_amdgcn_sched_barrier(0);
    mfmas(xb, wb);
    __builtin_amdgcn_sched_barrier(0);
    frags(xs, ws, 3, xb, wb);
    __builtin_amdgcn_sched_barrier(0);
    mfmas(xa, wa);
    __builtin_amdgcn_sched_barrier(0);
  }
  mfmas(xb, wb);
  __builtin_amdgcn_s_waitcnt(IX_VMCNT(0));
}

// Compile-time loop: f(integral_constant<int, I>) for I = B .. E-1, so that every index derived from I is a constant
// expression where it is used (arrays indexed this way are split into registers before any loop is unrolled).
template <int B, int E, typename F>
__device__ __forceinline__ void ix_static_for(F&& f) {
  if constexpr (B < E) {
    f(std::integral_constant<int, B>{});
    ix_static_for<B + 1, E>(f);
  }
}

// ---- pipeline E: four waves, one per SIMD, 128 x 128 per wave, statically interleaved ------------------------------
// The 256 x 256 tile on four waves reads a third less from LDS than on eight (each fragment feeds four matrix
// instructions instead of two), but a lone wave per SIMD has nobody to hide behind: whenever it waits, its matrix
// pipeline idles. So the k-tile is written as four phases of 16 matrix instructions with exactly one other
// instruction placed after each: the 8 fragment reads of the NEXT phase after instructions 0..7, one fetch after
// instructions 8, 10, 12, 14 (16 fetches per k-tile, evenly spread so that the four waves never hand the address
// unit a burst). Unit ring of pipeline C: five units, W two k-tiles ahead, X one. The phase that follows the k-tile's
// barrier multiplies the last quarter of the previous k-tile while the first fragments of the new one travel from LDS.
// Same K order as every other pipeline. Measured on MI355X, LM head 4096 x 4096 x 151936: 3.9 ms against 4.3 ms for
// the eight-wave form.
template <typename Cfg, typename XRow, typename WRow, typename Acc>
__device__ __forceinline__ void ix_gemm_mainloop_units4(ix_rsrc_t x_rsrc, const XRow& x_row,
                                                        ix_rsrc_t w_rsrc, const WRow& w_row, int K,
                                                        char* lds, Acc& acc) {
  constexpr int NT = Cfg::NT, CH = Cfg::X_CH, UNIT = Cfg::BM * 128, NU = 5;
  static_assert(Cfg::BM == Cfg::BN && Cfg::MI == 4 && Cfg::NI == 4 && CH == 8 && Cfg::UNITS == NU,
                "four waves of 128 x 128 over a 256 x 256 tile");
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
  const int KT = (K + IX_BK - 1) / IX_BK;
  const uint32_t lds_base = __builtin_amdgcn_readfirstlane(ix_lds_addr(lds) + (wave * 64) * 16);
  const int K2 = K * 2;

  uint32_t x_voff[CH], w_voff[CH];
  int kb[CH];
#pragma unroll
  for (int j = 0; j < CH; ++j) {
    const int r = (tid + j * NT) >> 3;
    kb[j] = ((tid & 7) ^ ix_swz8(r)) * 16;
    x_voff[j] = x_row(r) + kb[j];
    w_voff[j] = w_row(r) + kb[j];
  }
  // chunk j of the X (or W) rows of k-tile t into ring slot `slot`
  auto fetch = [&](bool is_x, int t, int slot, int j) {
    const int soff = t * (IX_BK * 2);
    const uint32_t dead = (uint32_t)((K2 - 1 - (soff + kb[j])) >> 31) & IX_OOB;
    if (is_x) ix_dma16(x_rsrc, lds_base + slot * UNIT + j * NT * 16, x_voff[j] | dead, soff);
    else ix_dma16(w_rsrc, lds_base + slot * UNIT + j * NT * 16, w_voff[j] | dead, soff);
  };
  const int frow = lane & 31, fg = lane >> 5;
  int x_foff[4], w_foff[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    x_foff[i] = ix_lds_off(wm * Cfg::TM + i * 32 + frow, fg * 4);
    w_foff[i] = ix_lds_off(wn * Cfg::TN + i * 32 + frow, fg * 4);
  }
  ix_bf16x8 fa[8], fb[8];  // [0..3] activation fragments, [4..7] weight fragments; two buffers
#define IX_READ_FRAG(F, XS, WS, S, I)                                                                   \
  F[I] = (I) < 4 ? *reinterpret_cast<const ix_bf16x8*>((XS) + (x_foff[(I) & 3] ^ ((S) << 4)))          \
                 : *reinterpret_cast<const ix_bf16x8*>((WS) + (w_foff[(I) & 3] ^ ((S) << 4)))
#define IX_MFMA(F, J)                                                                                   \
  acc[(J) >> 2][(J) & 3] =                                                                              \
      __builtin_amdgcn_mfma_f32_32x32x16_bf16(F[4 + ((J) & 3)], F[(J) >> 2], acc[(J) >> 2][(J) & 3], 0, 0, 0)

  // One phase: 16 matrix instructions on fragment buffer FM; after the even ones a fragment read of step S of the
  // k-tile at (XS, WS) into buffer FR (x0, w0..w3, x1..x3: the order in which the next phase needs them), after
  // instructions 1, 5, 9, 13 one fetch (chunks J0..J0+3 of the X or W rows of k-tile T into ring slot SLOT).
  // fragment reads after matrix instructions 0..7, fetches after 8, 10, 12, 14: the last read is eight matrix
  // instructions old when the k-tile's closing wait asks for it
#define IX_PHASE_READ_SLOT(j) ((j) < 8 ? (j) : -1)
#define IX_PHASE_FETCH_SLOT(j) ((j) >= 8 && ((j) & 1) == 0 ? ((j) - 8) >> 1 : -1)
#define IX_PHASE(FM, FR, XS, WS, S, IS_X, T, SLOT, J0)                                                  \
  ix_static_for<0, 16>([&](auto jc) {                                                                   \
    constexpr int j = decltype(jc)::value;                                                              \
    IX_MFMA(FM, j);                                                                                     \
    __builtin_amdgcn_sched_barrier(0);                                                                  \
    if constexpr (IX_PHASE_READ_SLOT(j) >= 0) {                                                         \
      constexpr int r = IX_PHASE_READ_SLOT(j);                                                          \
      constexpr int f = r == 0 ? 0 : (r <= 4 ? 3 + r : r - 4);                                          \
      IX_READ_FRAG(FR, XS, WS, S, f);                                                                   \
    } else if constexpr (IX_PHASE_FETCH_SLOT(j) >= 0) {                                                 \
      fetch(IS_X, T, SLOT, (J0) + IX_PHASE_FETCH_SLOT(j));                                              \
    }                                                                                                   \
    __builtin_amdgcn_sched_barrier(0);                                                                  \
  })

  // units in ring order: W(0), X(0), W(1), X(1), ...; the prologue fetches the first three and half of the fourth
#pragma unroll
  for (int j = 0; j < CH; ++j) fetch(false, 0, 0, j);
#pragma unroll
  for (int j = 0; j < CH; ++j) fetch(true, 0, 1, j);
#pragma unroll
  for (int j = 0; j < CH; ++j) fetch(false, 1, 2, j);
#pragma unroll
  for (int j = 0; j < 4; ++j) fetch(true, 1, 3, j);
  int slot = 3;  // ring slot of X(kt + 1)
  __builtin_amdgcn_s_waitcnt(IX_VMCNT(CH + 4));  // units 0 and 1 have landed
  __syncthreads();
  int cs = 0;  // slot of the W unit of the k-tile being read
  {
    const char* ws = lds;
    const char* xs = lds + UNIT;
    ix_static_for<0, 8>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      IX_READ_FRAG(fa, xs, ws, 0, i);
    });
  }
  for (int kt = 0; kt < KT; ++kt) {
    const char* ws = lds + cs * UNIT;
    const int xsl = cs + 1 == NU ? 0 : cs + 1;
    const char* xs = lds + xsl * UNIT;
    cs = xsl + 1 == NU ? 0 : xsl + 1;
    const int slot_x = slot, slot_w = slot + 1 == NU ? 0 : slot + 1;  // X(kt+1), W(kt+2)
    slot = slot_w + 1 == NU ? 0 : slot_w + 1;                         // X(kt+2): the slot W(kt) leaves
    IX_PHASE(fa, fb, xs, ws, 1, true, kt + 1, slot_x, 4);   // multiply step 0, read step 1
    IX_PHASE(fb, fa, xs, ws, 2, false, kt + 2, slot_w, 0);  // multiply step 1, read step 2
    IX_PHASE(fa, fb, xs, ws, 3, false, kt + 2, slot_w, 4);  // multiply step 2, read step 3
    // Every fragment of this k-tile is in registers (so its two slots may be overwritten by whoever passes the
    // barrier first), and all fetches but the last eight (the W rows of k-tile kt+2) have landed: k-tile kt+1 is
    // complete.
    __builtin_amdgcn_s_waitcnt(IX_VMCNT(CH) & 0xF0FF);  // also lgkmcnt(0)
    __syncthreads();
    // multiply step 3 while the first fragments of the next k-tile travel from LDS (past the end: stale bytes that
    // nothing multiplies)
    const char* ws1 = lds + cs * UNIT;
    const char* xs1 = lds + (cs + 1 == NU ? 0 : cs + 1) * UNIT;
    IX_PHASE(fb, fa, xs1, ws1, 0, true, kt + 2, slot, 0);
  }
#undef IX_PHASE
#undef IX_PHASE_READ_SLOT
#undef IX_PHASE_FETCH_SLOT
#undef IX_READ_FRAG
#undef IX_MFMA
  __builtin_amdgcn_s_waitcnt(IX_VMCNT(0));
}

// ---- pipeline D: fetching waves and computing waves (small tiles) -----------------------------------------------
// A tile with one or two MFMAs per wave and step is bound by instruction issue (a lone wave issues one instruction
// every four cycles, and a k-tile costs it the fetch instructions, the ring bookkeeping, the LDS reads and the
// MFMAs one after another). Here PW waves issue the fetches and wait for them, the WM*WN others only read
// fragments and multiply; they meet at one barrier per k-tile, which both publishes k-tile kt and frees the stage
// of k-tile kt-1 (its fragments were consumed by MFMAs before the barrier). A ring of SPLIT_STAGES whole k-tiles,
// laid out as in pipeline A; the K order is that of pipeline A.
template <typename Cfg, typename XRow, typename WRow, typename Acc>
__device__ __forceinline__ void ix_gemm_mainloop_split(ix_rsrc_t x_rsrc, const XRow& x_row,
                                                       ix_rsrc_t w_rsrc, const WRow& w_row, int K,
                                                       char* lds, Acc& acc) {
  constexpr int NP = Cfg::PW * 64, BM = Cfg::BM, S = Cfg::SPLIT_STAGES;
  constexpr int XC = BM * 8 / NP, WC = Cfg::BN * 8 / NP;  // 16-byte chunks per fetching thread and k-tile
  static_assert(S >= 3 && (BM * 8) % NP == 0 && (Cfg::BN * 8) % NP == 0, "fetch must divide over the fetching waves");
  static_assert((S - 2) * (XC + WC) <= 63, "the wait counter holds 63 outstanding loads");
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int KT = (K + IX_BK - 1) / IX_BK;
  if (wave >= Cfg::WM * Cfg::WN) {
    // ---- fetching waves
    const int pt = threadIdx.x - Cfg::NT;  // 0 .. NP-1
    const uint32_t lds_base = __builtin_amdgcn_readfirstlane(ix_lds_addr(lds) + ((pt >> 6) * 64) * 16);
    const int K2 = K * 2;
    uint32_t x_voff[XC], w_voff[WC];
    int x_kb[XC], w_kb[WC];
#pragma unroll
    for (int j = 0; j < XC; ++j) {
      const int r = (pt + j * NP) >> 3;
      x_kb[j] = ((pt & 7) ^ ix_swz8(r)) * 16;
      x_voff[j] = x_row(r) + x_kb[j];
    }
#pragma unroll
    for (int j = 0; j < WC; ++j) {
      const int r = (pt + j * NP) >> 3;
      w_kb[j] = ((pt & 7) ^ ix_swz8(r)) * 16;
      w_voff[j] = w_row(r) + w_kb[j];
    }
    auto issue = [&](int kt, int slot) {
      const int soff = kt * IX_BK * 2;
      const uint32_t sbase = lds_base + slot * Cfg::STAGE_BYTES;
#pragma unroll
      for (int j = 0; j < XC; ++j) {
        const uint32_t dead = (uint32_t)((K2 - 1 - (soff + x_kb[j])) >> 31) & IX_OOB;
        ix_dma16(x_rsrc, sbase + j * NP * 16, x_voff[j] | dead, soff);
      }
#pragma unroll
      for (int j = 0; j < WC; ++j) {
        const uint32_t dead = (uint32_t)((K2 - 1 - (soff + w_kb[j])) >> 31) & IX_OOB;
        ix_dma16(w_rsrc, sbase + BM * 128 + j * NP * 16, w_voff[j] | dead, soff);
      }
    };
#pragma unroll
    for (int p = 0; p < S - 1; ++p) issue(p, p);
    int is = S - 1;
    for (int kt = 0; kt < KT; ++kt) {
      __builtin_amdgcn_s_waitcnt(IX_VMCNT((S - 2) * (XC + WC)));  // k-tile kt has landed
      __syncthreads();
      issue(kt + S - 1, is);  // into the stage of k-tile kt-1
      is = is + 1 == S ? 0 : is + 1;
    }
    __builtin_amdgcn_s_waitcnt(IX_VMCNT(0));  // drain the out-of-range tail fetches before LDS is reused
    return;
  }
  // ---- computing waves
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
  const int frow = lane & 31, fg = lane >> 5;
  int x_foff[Cfg::MI], w_foff[Cfg::NI];
#pragma unroll
  for (int mi = 0; mi < Cfg::MI; ++mi) x_foff[mi] = ix_lds_off(wm * Cfg::TM + mi * 32 + frow, fg * 4);
#pragma unroll
  for (int ni = 0; ni < Cfg::NI; ++ni) w_foff[ni] = BM * 128 + ix_lds_off(wn * Cfg::TN + ni * 32 + frow, fg * 4);
  int cs = 0;
  for (int kt = 0; kt < KT; ++kt) {
    __syncthreads();
    const char* sb = lds + cs * Cfg::STAGE_BYTES;
    cs = cs + 1 == S ? 0 : cs + 1;
    ix_bf16x8 xf[4][Cfg::MI], wf[4][Cfg::NI];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
#pragma unroll
      for (int mi = 0; mi < Cfg::MI; ++mi)
        xf[s][mi] = *reinterpret_cast<const ix_bf16x8*>(sb + (x_foff[mi] ^ (s << 4)));
#pragma unroll
      for (int ni = 0; ni < Cfg::NI; ++ni)
        wf[s][ni] = *reinterpret_cast<const ix_bf16x8*>(sb + (w_foff[ni] ^ (s << 4)));
    }
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
      for (int mi = 0; mi < Cfg::MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < Cfg::NI; ++ni)
          acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[s][ni], xf[s][mi], acc[mi][ni], 0, 0, 0);
  }
}

// x_row(r) / w_row(r): byte offset of tile row r inside the operand's buffer, or IX_OOB.
template <typename Cfg, typename XRow, typename WRow, typename Acc>
__device__ __forceinline__ void ix_gemm_mainloop(ix_rsrc_t x_rsrc, const XRow& x_row,
                                                 ix_rsrc_t w_rsrc, const WRow& w_row, int K, char* lds,
                                                 Acc& acc) {
  if constexpr (Cfg::PW > 0)
    ix_gemm_mainloop_split<Cfg>(x_rsrc, x_row, w_rsrc, w_row, K, lds, acc);
  else if constexpr (Cfg::UNIT_RING && Cfg::NT == 256 && Cfg::MI == 4 && Cfg::NI == 4)
    ix_gemm_mainloop_units4<Cfg>(x_rsrc, x_row, w_rsrc, w_row, K, lds, acc);
  else if constexpr (Cfg::UNIT_RING)
    ix_gemm_mainloop_units<Cfg>(x_rsrc, x_row, w_rsrc, w_row, K, lds, acc);
  else if constexpr (Cfg::HALF_RING)
    ix_gemm_mainloop_h4<Cfg>(x_rsrc, x_row, w_rsrc, w_row, K, lds, acc);
  else
    ix_gemm_mainloop_full<Cfg>(x_rsrc, x_row, w_rsrc, w_row, K, lds, acc);
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

// Element e of an accumulator block. With 256 accumulator registers per lane (four waves on a 256 x 256 tile) the
// blocks live in the accumulation registers; read there, at the point of use, a value goes straight into a vector
// register instead of being copied out early and spilled by the register allocator.
template <bool FROM_AGPR>
__device__ __forceinline__ float ix_acc_read(const ix_f32x16& a, int e) {
  if constexpr (FROM_AGPR) {
    float r;
    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(r) : "a"(a[e]));
    return r;
  } else {
    return a[e];
  }
}

// All 16 values of an accumulator block, read before any of them is used: the reads are independent of each other, so a
// lone wave issues them back to back instead of stalling on each read -> convert pair.
template <bool FROM_AGPR>
__device__ __forceinline__ void ix_acc_read16(const ix_f32x16& a, float (&v)[16]) {
#pragma unroll
  for (int e = 0; e < 16; ++e) v[e] = ix_acc_read<FROM_AGPR>(a, e);
}

// A 32x32 accumulator holds, for the token of this lane, output columns (i/4)*8 + hf*4 + i%4. For the column
// blocks q = 2p and 2p+1 the two half-waves swap one packed pair each, after which the lower half holds columns
// 16p .. 16p+7 and the upper half 16p+8 .. 16p+15 of the token: one 16-byte store per lane instead of two
// 8-byte ones. lo/hi: this lane's packed columns of block 2p / 2p+1.
__device__ __forceinline__ uint4 ix_join_halves(uint2 lo, uint2 hi) {
  const auto x = __builtin_amdgcn_permlane32_swap(lo.x, hi.x, false, false);
  const auto y = __builtin_amdgcn_permlane32_swap(lo.y, hi.y, false, false);
  return make_uint4(x[0], y[0], x[1], y[1]);
}

// A 32-row block of a wave's output, NPIECE * 16 columns wide, stored in whole rows. After ix_join_halves a lane holds,
// for token row lane % 32, the 16-byte pieces i = 0 .. NPIECE-1 = columns 16 i + 8 (lane / 32) .. + 7: stored directly,
// one instruction would touch 32 rows with 32 bytes each. Here the pieces pass through a wave-private LDS buffer
// (32 rows of NPIECE * 32 + 16 bytes; the 16 bytes of padding spread the rows over the banks) and come back with
// 2 NPIECE lanes per row, so that an instruction stores 64 / (2 NPIECE) whole rows of NPIECE * 32 contiguous bytes.
// Rows at or past live_rows are not stored. dst = the block's row 0 at the wave's first column; 16-byte aligned, ld % 8
// == 0. No barrier: only this wave touches buf, and a wave's LDS operations complete in order.
template <int NPIECE>
__device__ __forceinline__ void ix_store_block32_via_lds(char* buf, const uint4 (&pc)[NPIECE], bf16_t* dst, long ld,
                                                         int live_rows) {
  constexpr int PITCH = NPIECE * 32 + 16, CPR = NPIECE * 2, RPI = 64 / CPR;
  static_assert(64 % CPR == 0 && 32 % RPI == 0, "pieces per row must divide the wave");
  const int lane = threadIdx.x & 63;
  char* mine = buf + (lane & 31) * PITCH + (lane >> 5) * 16;
#pragma unroll
  for (int i = 0; i < NPIECE; ++i) *reinterpret_cast<uint4*>(mine + i * 32) = pc[i];
  const int rr = lane / CPR, cc = lane % CPR;
#pragma unroll
  for (int j = 0; j < 32 / RPI; ++j) {
    const int row = j * RPI + rr;
    const uint4 v = *reinterpret_cast<const uint4*>(buf + row * PITCH + cc * 16);
    if (row < live_rows) *reinterpret_cast<uint4*>(dst + (long)row * ld + cc * 8) = v;
  }
}
// bytes of LDS one wave needs for it
template <int NPIECE>
constexpr int ix_store_block32_lds_bytes() { return 32 * (NPIECE * 32 + 16); }

// Store 4 consecutive output columns of one token (8 bytes when aligned and in range). Rounding is the hardware
// pack-convert everywhere in the GEMM epilogues (round to nearest even; a NaN stays a NaN and keeps its payload),
// so that wide and narrow stores of the same value give the same bits.
__device__ __forceinline__ void ix_store4_bf16(bf16_t* __restrict__ p, int valid, bool vec, float a, float b,
                                               float c, float d) {
  if (vec && valid >= 4) {
    uint2 u;
    u.x = ix_pack_bf2_hw(a, b);
    u.y = ix_pack_bf2_hw(c, d);
    *reinterpret_cast<uint2*>(p) = u;
  } else {
    if (valid > 0) p[0] = ix_f2bf_hw(a);
    if (valid > 1) p[1] = ix_f2bf_hw(b);
    if (valid > 2) p[2] = ix_f2bf_hw(c);
    if (valid > 3) p[3] = ix_f2bf_hw(d);
  }
}
