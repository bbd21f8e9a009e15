// Pipeline F: a workgroup that streams MANY 256 x 256 tiles through one unbroken operand ring.
//
// Pipeline E (ix_gemm_core.h) spends, per tile, about 2 us before its first matrix instruction (the first operand
// units travel from memory), 4 us after its last one (accumulators -> bf16 -> stores) and half a microsecond between
// workgroups. For a product with K = 768 that is a third of the tile's time. Here a workgroup owns a fixed sequence of
// tiles and
//   * the ring never drains: the last two k-tiles of a tile fetch the first units of the NEXT tile, so the next
//     tile's first matrix instruction follows the previous tile's last one;
//   * at the end of a tile the accumulators are only moved out (rounded to bf16, two per register: 128 vector
//     registers per lane) and the matrix pipeline restarts at once; everything else the epilogue has to do with
//     them -- the row maximum, the exchange between lanes, the stores -- is cut into micro-steps of a few
//     instructions, one per matrix instruction of the next tile's first IX_STREAM_NSK k-tiles, where a lone wave has
//     issue slots to spare;
//   * the LDS is the ring and nothing else (five units = 160 KiB), so the stores go straight from registers.
// Arithmetic per output element is that of every other pipeline: same instruction, same K order, same roundings.
//
// The job object supplies the tile sequence, the operand addresses and the deferred epilogue:
//   bool open_first()                 locate the first tile of this workgroup (false: none); fills nx_xr / nx_wr;
//                                     makes the pending tile an empty one (its micro-steps run but store nothing)
//   void open_next()                  locate the tile after the current one; sets has_next; a missing tile gets
//                                     empty descriptors (its fetches read zeros and touch no memory)
//   void first_voffs()                byte offsets of this thread's chunks of each operand (the same in every tile:
//                                     the descriptors are tile-local)
//   template <int J> uint32_t x_voff() / w_voff()   offset of chunk J; the ring asks for an operand's chunks in the
//                                     cyclic order 0, 1, .. 7, 0, .., so a job may keep one running register
//   void turn_offsets()               called in the second-last k-tile after the last fetch through the current tile's
//                                     offsets: a job whose offsets depend on the tile (gathered rows) turns them to the
//                                     next tile here; nothing in it may make the compiler wait for the operand stream
//   static constexpr int DMA_IDLE     0, or 3 for a job that is short of scalar registers (ix_dma16)
//   void drain(acc)                   accumulators -> pending registers; current tile becomes the pending one
//   void advance()                    next tile becomes the current one
//   template <int I> void micro()     micro-step I of the pending tile's epilogue, I in [0, 64 * NSK)
//   static constexpr int NSK          leading k-tiles of a tile that carry micro-steps (KT >= NSK + 3)
//   static int w_frag_row(ni, rho)    which row of the wave's 128 weight rows in LDS feeds row rho of block ni of the
//                                     matrix instruction: a job picks the permutation that leaves each lane with
//                                     contiguous output columns (ix_stream_col below)
//   static constexpr int stores_after_p1(int slice)   vector-memory stores micro() issues in slots 16 .. 47 of
//                                     k-tile `slice`: they are younger than the fetches the k-tile's closing wait
//                                     is for, so the wait count makes room for them
// Loads and stores retire through one in-order counter on this hardware; every wait below counts both. Nothing inside
// the loop may branch, spill or touch a stack object: the compiler would answer with "wait for all loads", i.e. for
// the whole operand stream.
#pragma once
#include "ix_gemm_core.h"

#define IX_STREAM_NSK 8                       // leading k-tiles of a tile that carry the previous tile's epilogue
#define IX_STREAM_MIN_KT (IX_STREAM_NSK + 3)  // + the three closing k-tiles that turn to the next tile
// Workgroups a streaming kernel launches: one per CU (the ring fills a CU's LDS), a multiple of 8 so that every XCD's run
// of the tile order is shared by the same number of them.
#define IX_STREAM_WORKGROUPS 256
// Non-temporal stores of the output tiles: of the plain job (dense GEMM, the experts' second GEMM: outputs of 64 MB and
// up, written once while the caches feed the operand stream -- 131072 x 768 x 2048: 0.395 -> 0.34 ms, nothing lost at
// large K or in the kernels that read the output next) and of the experts' first GEMM (whose output the second one
// reads back at once: no gain, left off).
#ifndef IX_STREAM_STORE_NT_PLAIN
#define IX_STREAM_STORE_NT_PLAIN true
#endif
#ifndef IX_STREAM_STORE_NT_FC1
#define IX_STREAM_STORE_NT_FC1 false
#endif

// Output layout of the streaming kernels. A lane of a 32 x 32 accumulator block holds result rows 8 g + 4 h + i (g < 4,
// i < 4; h = lane / 32) for the token lane % 32. With the wave's weight rows dealt to (block, row) by
//   column = 64 (ni / 2) + 32 h + 16 (ni % 2) + 4 g + i
// the blocks 2 L and 2 L + 1 of a lane are 32 consecutive output columns of its token: four 16-byte pieces, piece
// pi = 2 (ni % 2) + g / 2 in the packed registers [4 (pi % 2), 4 (pi % 2) + 3] of block 2 L + pi / 2. A 4 x 4 transpose
// inside each quad of lanes (two exchange stages through the lane-permute path, no LDS) then leaves lane q of a quad
// with piece q of the quad's four tokens, so that a store instruction writes 64 contiguous bytes per quad and the two
// half-waves complete the 128-byte line: the address unit takes one request per contiguous segment, and the stores
// share it with the operand stream.
__host__ __device__ constexpr int ix_stream_col(int ni, int rho) {
  return 64 * (ni >> 1) + 32 * ((rho >> 2) & 1) + 16 * (ni & 1) + 4 * (rho >> 3) + (rho & 3);
}
template <int CTRL>
__device__ __forceinline__ uint32_t ix_quad_perm(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, true);
}
// One output of an exchange stage of the transpose: the stage pairs slot a with slot b = a + 1 (stage 1, partner lane
// l ^ 1) or b = a + 2 (stage 2, partner lane l ^ 2); the lane whose partner bit is 0 keeps slot a and takes the
// partner's slot a into its slot b, the other lane keeps slot b and takes the partner's slot b into its slot a.
// SECOND = false: the new slot a; true: the new slot b. One lane permute and one select.
template <int STAGE, bool SECOND>
__device__ __forceinline__ uint32_t ix_quad_exchange(uint32_t a, uint32_t b) {
  const bool keep_a = (threadIdx.x & STAGE) == 0;
  constexpr int CTRL = STAGE == 1 ? 0xB1 : 0x4E;  // quad_perm [1, 0, 3, 2] / [2, 3, 0, 1]
  if constexpr (!SECOND) {
    const uint32_t other = ix_quad_perm<CTRL>(b);
    return keep_a ? a : other;
  } else {
    const uint32_t other = ix_quad_perm<CTRL>(a);
    return keep_a ? other : b;
  }
}

template <int SLICE_, bool ZERO_, int TAIL_>
struct IxKtPlan {
  static constexpr int SLICE = SLICE_;  // -1, or which k-tile's worth of micro-steps to interleave
  static constexpr bool ZERO = ZERO_;   // first k-tile of a tile: its first phase starts the accumulators from zero
  static constexpr int TAIL = TAIL_;    // 0, or 3 / 2 / 1 = third-last / second-last / last k-tile of the tile
};

template <typename Cfg, typename Job>
__device__ __forceinline__ void ix_gemm_stream4(Job& job, int KT, char* lds) {
  constexpr int NT = Cfg::NT, CH = Cfg::X_CH, UNIT = Cfg::BM * 128, NU = 5, NSK = Job::NSK;
  static_assert(Cfg::BM == 256 && Cfg::BN == 256 && Cfg::MI == 4 && Cfg::NI == 4 && CH == 8 && NT == 256,
                "four waves of 128 x 128 over a 256 x 256 tile");
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
  const uint32_t lds_base = __builtin_amdgcn_readfirstlane(ix_lds_addr(lds) + (wave * 64) * 16);

  if (!job.open_first()) return;
  ix_rsrc_t xr_c = job.nx_xr, wr_c = job.nx_wr, xr_n = xr_c, wr_n = wr_c;
  job.first_voffs();
  job.advance();

  // chunk j of k-tile t of the tile that `rsrc` describes into ring slot `slot` (K is a multiple of 64 here: no tail)
  auto fetch = [&](const ix_rsrc_t& rsrc, uint32_t voff, int t, int slot, int j) {
    ix_dma16<Job::DMA_IDLE>(rsrc, lds_base + slot * UNIT + j * NT * 16, voff, t * (IX_BK * 2));
  };
  const int frow = lane & 31, fg = lane >> 5;
  int x_foff[4], w_foff[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    x_foff[i] = ix_lds_off(wm * Cfg::TM + i * 32 + frow, fg * 4);
    w_foff[i] = ix_lds_off(wn * Cfg::TN + Job::w_frag_row(i, frow), fg * 4);
  }
  // Fragments: the four weight fragments of a step are all needed by the step's first four matrix instructions and
  // live until its last four, so they are double-buffered (fa / fb); activation fragment i is used by instructions
  // 4 i .. 4 i + 3 only, so the next step's fragment i is read into the same registers right after instruction 4 i + 3
  // (16 registers instead of 32).
  ix_bf16x8 fx[4], fa[4], fb[4];
  ix_f32x16 acc[4][4];
  const ix_f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

#define IXS_READ_X(XS, S, I) fx[I] = *reinterpret_cast<const ix_bf16x8*>((XS) + (x_foff[I] ^ ((S) << 4)))
#define IXS_READ_W(F, WS, S, I) F[I] = *reinterpret_cast<const ix_bf16x8*>((WS) + (w_foff[I] ^ ((S) << 4)))
#define IXS_MFMA(F, J, Z)                                                                               \
  if constexpr (Z)                                                                                      \
    acc[(J) >> 2][(J) & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(F[(J) & 3], fx[(J) >> 2], zero16, 0, 0, 0); \
  else                                                                                                  \
    acc[(J) >> 2][(J) & 3] =                                                                            \
        __builtin_amdgcn_mfma_f32_32x32x16_bf16(F[(J) & 3], fx[(J) >> 2], acc[(J) >> 2][(J) & 3], 0, 0, 0)
  // One phase (pipeline E's): 16 matrix instructions on weight buffer FM and the activation fragments; after
  // instructions 0, 1, 2, 4 a weight fragment of step S of the k-tile at (XS, WS) into buffer FR, after 3, 7, 11, 15 its
  // activation fragments 0..3, after 8, 10, 12, 14 one fetch (chunks J0..J0+3 of k-tile T of the tile behind RSRC / VOFF
  // into ring slot SLOT); after every instruction micro-step SLICE * 64 + PH * 16 + j.
#define IXS_PHASE(FM, FR, XS, WS, S, RSRC, VOFF, T, SLOT, J0, PH, Z, SLICE)                             \
  ix_static_for<0, 16>([&](auto jc) {                                                                   \
    constexpr int j = decltype(jc)::value;                                                              \
    IXS_MFMA(FM, j, Z);                                                                                 \
    __builtin_amdgcn_sched_barrier(0);                                                                  \
    if constexpr ((j & 3) == 3) {                                                                       \
      IXS_READ_X(XS, S, j >> 2);                                                                        \
    } else if constexpr (j < 3 || j == 4) {                                                             \
      IXS_READ_W(FR, WS, S, j < 3 ? j : 3);                                                             \
    } else if constexpr (j >= 8 && (j & 1) == 0) {                                                      \
      fetch(RSRC, job.template VOFF<(J0) + ((j - 8) >> 1)>(), T, SLOT, (J0) + ((j - 8) >> 1));          \
    }                                                                                                   \
    if constexpr ((SLICE) >= 0) job.template micro<((SLICE) < 0 ? 0 : (SLICE)) * 64 + (PH) * 16 + j>(); \
    __builtin_amdgcn_sched_barrier(0);                                                                  \
  })

  // ---- the first tile's first units: W(0), X(0), W(1) and half of X(1), as in pipeline E
  ix_static_for<0, CH>([&](auto jc) {
    constexpr int j = decltype(jc)::value;
    fetch(wr_c, job.template w_voff<j>(), 0, 0, j);
  });
  ix_static_for<0, CH>([&](auto jc) {
    constexpr int j = decltype(jc)::value;
    fetch(xr_c, job.template x_voff<j>(), 0, 1, j);
  });
  ix_static_for<0, CH>([&](auto jc) {
    constexpr int j = decltype(jc)::value;
    fetch(wr_c, job.template w_voff<j>(), 1, 2, j);
  });
  ix_static_for<0, 4>([&](auto jc) {
    constexpr int j = decltype(jc)::value;
    fetch(xr_c, job.template x_voff<j>(), 1, 3, j);
  });
  int slot = 3;  // ring slot of X(kt + 1)
  int cs = 0;    // slot of the W unit of the k-tile being read
  __builtin_amdgcn_s_waitcnt(IX_VMCNT(CH + 4));  // units 0 and 1 have landed
  __syncthreads();
  ix_static_for<0, 4>([&](auto ic) {
    constexpr int i = decltype(ic)::value;
    IXS_READ_X(lds + UNIT, 0, i);
    IXS_READ_W(fa, lds, 0, i);
  });

  // One k-tile. The ring runs on across tiles: in the last two k-tiles "k-tile kt + 1 / kt + 2" are k-tiles 0 and 1 of
  // the next tile, fetched through the next tile's descriptors and offsets.
  auto ktile = [&](auto plan, int kt) {
    using P = decltype(plan);
    constexpr int TAIL = P::TAIL, SLICE = P::SLICE;
    constexpr bool ZERO = P::ZERO;
    const char* ws = lds + cs * UNIT;
    const int xsl = cs + 1 == NU ? 0 : cs + 1;
    const char* xs = lds + xsl * UNIT;
    cs = xsl + 1 == NU ? 0 : xsl + 1;
    const int slot_x = slot, slot_w = slot + 1 == NU ? 0 : slot + 1;  // X(kt+1), W(kt+2)
    slot = slot_w + 1 == NU ? 0 : slot_w + 1;                         // X(kt+2): the slot W(kt) leaves
    if constexpr (TAIL == 3) {
      job.open_next();
      xr_n = job.nx_xr;
      wr_n = job.nx_wr;
    }
    const int t1 = TAIL == 1 ? 0 : kt + 1;                       // k-tile of the X half fetched in the first phase
    const int t2 = TAIL == 2 ? 0 : (TAIL == 1 ? 1 : kt + 2);     // k-tile of the W unit and the X half after it
    IXS_PHASE(fa, fb, xs, ws, 1, (TAIL == 1 ? xr_n : xr_c), x_voff, t1, slot_x, 4, 0, ZERO, SLICE);
    if constexpr (TAIL == 2) job.turn_offsets();  // the current tile has made its last fetch through them
    IXS_PHASE(fb, fa, xs, ws, 2, ((TAIL == 1 || TAIL == 2) ? wr_n : wr_c), w_voff, t2, slot_w, 0, 1, false, SLICE);
    IXS_PHASE(fa, fb, xs, ws, 3, ((TAIL == 1 || TAIL == 2) ? wr_n : wr_c), w_voff, t2, slot_w, 4, 2, false, SLICE);
    // Every fragment of this k-tile is in registers, and everything older than the W unit just requested (and the
    // stores of this k-tile's micro-steps) has landed: k-tile kt + 1 is complete.
    constexpr int NST = SLICE >= 0 ? Job::stores_after_p1(SLICE < 0 ? 0 : SLICE) : 0;
    __builtin_amdgcn_s_waitcnt(IX_VMCNT(CH + NST) & 0xF0FF);  // also lgkmcnt(0)
    __syncthreads();
    const char* ws1 = lds + cs * UNIT;
    const char* xs1 = lds + (cs + 1 == NU ? 0 : cs + 1) * UNIT;
    IXS_PHASE(fb, fa, xs1, ws1, 0, ((TAIL == 1 || TAIL == 2) ? xr_n : xr_c), x_voff, t2, slot, 0, 3, false, SLICE);
  };

  // The first tile runs the same code as every other: its "pending tile" is the empty one the job starts with (no rows,
  // so its stores go nowhere).
  for (;;) {
    ix_static_for<0, NSK>([&](auto sc) {
      constexpr int s = decltype(sc)::value;
      ktile(IxKtPlan<s, s == 0, 0>{}, s);
    });
    const int kt0 = NSK;
    for (int kt = kt0; kt < KT - 3; ++kt) ktile(IxKtPlan<-1, false, 0>{}, kt);
    ktile(IxKtPlan<-1, false, 3>{}, KT - 3);
    ktile(IxKtPlan<-1, false, 2>{}, KT - 2);
    ktile(IxKtPlan<-1, false, 1>{}, KT - 1);
    // the matrix pipeline has drained before the accumulation registers are read by hand
    asm volatile("s_nop 15\n\ts_nop 15");
    job.drain(acc);
    if (!job.has_next) break;
    job.advance();
    xr_c = xr_n;
    wr_c = wr_n;
  }
#undef IXS_PHASE
#undef IXS_MFMA
#undef IXS_READ_X
#undef IXS_READ_W
  __builtin_amdgcn_s_waitcnt(IX_VMCNT(0));
  // the last tile's epilogue, with nothing to hide behind
  ix_static_for<0, NSK>([&](auto sc) {
    ix_static_for<0, 64>([&](auto qc) { job.template micro<decltype(sc)::value * 64 + decltype(qc)::value>(); });
  });
}

// ---- the job of a plain product (dense GEMM, the experts' second GEMM): C = bf16(X W^T), optional row maximum -----------
// Seq supplies the tile sequence: bool locate(xcd, idx, IxStreamTile&) for position idx of XCD xcd's run, and the operand
// pitches lda / ldw / ldc / parts_ld and K. Requirements (the launch checks them): K % 64 == 0, every tile's column
// count a multiple of 8, ldc % 8 == 0, C 16-byte aligned, 256 * pitch * 2 < 2^30.
struct IxStreamTile {
  const bf16_t* x;  // first activation row of the tile
  const bf16_t* w;  // first weight row
  bf16_t* c;        // the tile's first output element
  float* part;      // the tile's first row-max part (two per token: one per wave column)
  int mv, nv;       // rows and columns that exist
};

template <typename Cfg, typename Seq, bool PARTS>
struct IxPlainStreamJob {
  Seq seq;
  unsigned xcd, idx, stride;
  ix_rsrc_t nx_xr, nx_wr;
  bool has_next;
  IxStreamTile nx, cur;
  ix_rsrc_t p_cr, p_pr;      // pending tile: descriptors of its part of C and of the row-max parts
  uint32_t p_voff, p_pvoff;  // this lane's first output element / part in them
  int p_cols;                // columns left from there
  uint32_t pend[4][4][8];    // the pending tile's outputs, two bf16 per register, accumulator layout
  uint32_t ta[4][4], tb[4][4];  // [slot][dword] after exchange stage 1 / 2
  float rmax;

  __device__ __forceinline__ void locate() {
    has_next = seq.locate(xcd, idx, nx);
    // tile-local descriptors: rows past the tile fall outside the range and read as 0; no tile, no bytes
    nx_xr = ix_make_rsrc(has_next ? nx.x : nullptr, has_next ? (uint32_t)(((long)(nx.mv - 1) * seq.lda + seq.K) * 2) : 0u);
    nx_wr = ix_make_rsrc(has_next ? nx.w : nullptr, has_next ? (uint32_t)(((long)(nx.nv - 1) * seq.ldw + seq.K) * 2) : 0u);
  }
  __device__ __forceinline__ bool open_first() {
    xcd = blockIdx.x & 7u;
    idx = blockIdx.x >> 3;
    stride = gridDim.x >> 3;
    locate();
    // the empty pending tile
    p_cr = ix_make_rsrc(nullptr, 0u);
    p_pr = p_cr;
    p_voff = p_pvoff = IX_OOB;
    p_cols = 0;
    rmax = IX_NEG_INF;
#pragma unroll
    for (int i = 0; i < 128; ++i) pend[i >> 5][(i >> 3) & 3][i & 7] = 0u;
    return has_next;
  }
  __device__ __forceinline__ void open_next() {
    idx += stride;
    locate();
  }
  // One running offset per operand: chunk j sits 32 j rows below chunk 0, and the ring asks for chunks in cyclic order.
  // The step is added by an instruction the compiler cannot hoist, or it would keep all eight sums in registers.
  uint32_t xv, wv;
  int x_step, w_step;
  __device__ __forceinline__ void first_voffs() {
    const int tid = threadIdx.x;
    const int r0 = tid >> 3;
    const uint32_t kb = (uint32_t)(((tid & 7) ^ ix_swz8(r0)) * 16);  // rows 32 apart share the swizzle
    xv = (uint32_t)((long)r0 * seq.lda * 2) + kb;
    wv = (uint32_t)((long)r0 * seq.ldw * 2) + kb;
    x_step = __builtin_amdgcn_readfirstlane((int)(32 * seq.lda * 2));
    w_step = __builtin_amdgcn_readfirstlane((int)(32 * seq.ldw * 2));
  }
  template <int J>
  __device__ __forceinline__ uint32_t x_voff() {
    const uint32_t v = xv;
    asm volatile("v_add_u32 %0, %1, %0" : "+v"(xv) : "s"(J == 7 ? -7 * x_step : x_step));
    return v;
  }
  template <int J>
  __device__ __forceinline__ uint32_t w_voff() {
    const uint32_t v = wv;
    asm volatile("v_add_u32 %0, %1, %0" : "+v"(wv) : "s"(J == 7 ? -7 * w_step : w_step));
    return v;
  }
  __device__ __forceinline__ void turn_offsets() const {}  // tile-local descriptors: the offsets never change
  static constexpr int DMA_IDLE = 0;  // every scalar operand of the loads comes from scalar arithmetic
  static constexpr int NSK = IX_STREAM_NSK;
  // (rows sit at the same offsets in every tile: the descriptors carry the tile)
  __device__ __forceinline__ void advance() { cur = nx; }
  template <typename Acc>
  __device__ __forceinline__ void drain(Acc& acc) {
    ix_static_for<0, 16>([&](auto bc) {
      constexpr int mi = decltype(bc)::value >> 2, ni = decltype(bc)::value & 3;
      float a16[16];
      ix_acc_read16<true>(acc[mi][ni], a16);
#pragma unroll
      for (int i = 0; i < 8; ++i) pend[mi][ni][i] = ix_pack_bf2_hw(a16[2 * i], a16[2 * i + 1]);
      __builtin_amdgcn_sched_barrier(0);  // or every read is scheduled ahead of the first pack: 256 registers in flight
    });
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    // after the quad transposes a lane holds piece (lane % 4) of the four tokens of its quad
    const int r = wm * 128 + (lane & 28), c = wn * 128 + 32 * (lane >> 5) + 8 * (lane & 3);
    // Tile-local descriptor of C: rows past the tile's last fall outside its range and are dropped by the hardware;
    // columns past the matrix are sent out of range by hand (p_cols).
    p_cr = ix_make_rsrc(cur.c, (uint32_t)(((long)(cur.mv - 1) * seq.ldc + cur.nv) * 2));
    p_voff = (uint32_t)(((long)r * seq.ldc + c) * 2);
    p_cols = cur.nv - c;
    if constexpr (PARTS) {
      p_pr = ix_make_rsrc(cur.part, (uint32_t)(((long)(cur.mv - 1) * seq.parts_ld + 2) * 4));
      p_pvoff = (lane < 32) ? (uint32_t)(((long)(wm * 128 + lane) * seq.parts_ld + wn) * 4) : IX_OOB;
    }
  }
  // k-tile s of the next tile carries the blocks (mi = s / 2, ni = 2 L and 2 L + 1, L = s % 2): 64 columns of 32 tokens
  // per wave. Slots 0..7 the row maximum, 8..23 and 24..39 the two exchange stages of the quad transposes, 40..43 the
  // four stores (a 128-byte line per token), 44 the maximum's store.
  static constexpr int stores_after_p1(int s) { return 4 + ((PARTS && (s & 1)) ? 1 : 0); }
  static __device__ __forceinline__ int w_frag_row(int ni, int rho) { return ix_stream_col(ni, rho); }
  template <int I>
  __device__ __forceinline__ void micro() {
    constexpr int s = I / 64, q = I % 64;
    constexpr int mi = s >> 1, L = s & 1;
    if constexpr (PARTS && q < 8) {
      // rounding is monotonic: the maximum of the rounded values is the rounded maximum
      if constexpr (q == 0 && L == 0) rmax = IX_NEG_INF;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        constexpr int k0 = q * 2;
        const uint32_t u = pend[mi][2 * L + ((k0 + h) >> 3)][(k0 + h) & 7];
        rmax = fmaxf(rmax, fmaxf(__uint_as_float(u << 16), __uint_as_float(u & 0xffff0000u)));
      }
    } else if constexpr (q >= 8 && q < 24) {
      // piece pi, dword d of the lane's 64 bytes: pend[mi][2 L + pi / 2][4 (pi % 2) + d]; stage 1 pairs pieces (0, 1), (2, 3)
      constexpr int o = q - 8, d = o >> 2, t = o & 3, a = t & 2;
      ta[t][d] = ix_quad_exchange<1, (t & 1) != 0>(pend[mi][2 * L + (a >> 1)][d], pend[mi][2 * L + (a >> 1)][4 + d]);
    } else if constexpr (q >= 24 && q < 40) {
      constexpr int o = q - 24, d = o >> 2, t = o & 3, a = t & 1;  // stage 2 pairs slots (0, 2), (1, 3)
      tb[t][d] = ix_quad_exchange<2, (t & 2) != 0>(ta[a][d], ta[a + 2][d]);
    } else if constexpr (q >= 40 && q < 44) {
      constexpr int t = q - 40;  // token t of the quad
      const uint32_t off =
          (64 * L < p_cols) ? p_voff + (uint32_t)(((long)(mi * 32 + t) * seq.ldc + 64 * L) * 2) : IX_OOB;
      ix_buffer_store16<IX_STREAM_STORE_NT_PLAIN>(make_uint4(tb[t][0], tb[t][1], tb[t][2], tb[t][3]), p_cr, off);
    } else if constexpr (PARTS && L == 1 && q == 44) {
      const float v = fmaxf(rmax, __shfl_xor(rmax, 32, IX_WAVE));
      ix_buffer_store4(__float_as_uint(v), p_pr,
                       p_pvoff == IX_OOB ? IX_OOB : p_pvoff + (uint32_t)((long)(mi * 32) * seq.parts_ld * 4));
    }
  }
};
