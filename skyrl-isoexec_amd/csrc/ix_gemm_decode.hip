// Dense products with at most 64 rows (a decode step's projections and LM head; the M <= 64 cases of the batch-invariant
// matmul, reference ops/mm/mm_tiles.py:232-326 behind the aten::mm override of ops/moe/moe_batch_invariant.py:422-473):
// C[M, N] = A[M, K] . W[N, K]^T with the weights streamed through registers.
//
// At these sizes the matrix pipes idle and the product is the time memory needs to deliver W once. The ring tiles stage
// W in LDS, so a CU never has more than its LDS in flight; here, as in the decode-size expert kernels (ix_moe.hip):
//   * W is read from a FRAGMENT-PACKED copy (ix_gemm_pack_decode): per (unit of 32 weight rows, k-tile) the 4 KiB a
//     wave's four matrix instructions take as their A operands, in (step, lane) order, so a load instruction is 1 KiB
//     of contiguous memory and a wave walks one contiguous stream;
//   * a lane holds the fragments of the next D = 8 k-tiles in registers (32 loads of 16 bytes in flight per lane; with
//     eight waves on a CU 256 KiB of weight bytes in flight per CU);
//   * the activations -- the same at most 64 rows for every unit -- are staged once per workgroup: each k-tile of A is
//     fetched straight into LDS in B-operand fragment order (memory -> LDS, 1 KiB pieces shared out over the waves), as
//     far ahead as the weights, and every wave reads its B fragments from there. One barrier per k-tile, which couples
//     the waves of a workgroup: four waves per workgroup measured faster than eight (LM head 64 x 2048 x 151936:
//     129 against 137 us; the ring tiles 143), two when the product has few units.
// Arithmetic is that of every tile shape of ix_gemm_bf16_nt: v_mfma_f32_32x32x16_bf16, weights the A operand, K in
// tiles of 64, step s consuming k = 8 s .. 8 s + 7 (lane group 0) and 32 + 8 s .. (lane group 1), one fp32 accumulator
// per element, one hardware bf16 rounding at the store. The walk over K is straight-line code (K / 64 is a template
// argument): at a loop's back edge the compiler's wait bookkeeping falls back to "every load done", which would drain
// the ring at every k-tile.
//
// Waits. Vector-memory operations retire in order. A wave issues, per k-tile, PPW activation pieces (inline assembly:
// the compiler does not count them) and then its 4 weight loads (ordinary loads: the compiler waits for exactly the
// ones a matrix instruction reads; its count misses the pieces in between, so it waits for slightly more than it needs,
// never less). "My pieces of k-tile kt have landed" is an explicit wait: after them came the 4 weight loads of the same
// k-tile and everything of the younger k-tiles in flight.
// Packed layout (16-byte chunk index; r = lane % 32, g = lane / 32):
//   Wf [N / 32][K / 64][s 4][lane 64]    chunk = W[32 u + r][64 kt + 32 g + 8 s .. + 7]
#include "ix_common.h"
#include "ix_gemm_core.h"
#include "../../include/isoexec_hip.h"

#define IX_GD_D 8  // k-tiles of weight fragments (and of activations in LDS) ahead of the matrix instructions

__global__ __launch_bounds__(256) void k_gemm_pack_frag(const bf16_t* __restrict__ W, long ldw, bf16_t* __restrict__ Wf,
                                                        int KT, long chunks) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= chunks) return;
  const int lane = (int)(i & 63), st = (int)((i >> 6) & 3);
  const long rest = i >> 8;
  const int kt = (int)(rest % KT);
  const long u = rest / KT;
  const int r = lane & 31, g = lane >> 5;
  *reinterpret_cast<uint4*>(Wf + i * 8) =
      *reinterpret_cast<const uint4*>(W + (32 * u + r) * ldw + 64 * kt + 32 * g + 8 * st);
}

// TB: 32-row blocks of A (1: M <= 32, 2: M <= 64). NW: waves per workgroup, one unit of 32 weight rows each.
template <int KT, int TB, int NW>
__global__ __launch_bounds__(NW * 64) void k_gemm_dec(const bf16_t* __restrict__ A, long lda, int M,
                                                      const bf16_t* __restrict__ Wf, bf16_t* __restrict__ C, long ldc,
                                                      int units) {
  constexpr int D = IX_GD_D;
  constexpr int PIECES = TB * 4;           // 1 KiB pieces of an activation k-tile: (row block, step)
  constexpr int PPW = PIECES / NW;         // pieces a wave fetches per k-tile
  constexpr int SLOT = PIECES * 1024;      // bytes of an activation k-tile in LDS
  constexpr int PER_KT = PPW + 4;          // vector-memory operations a wave issues per k-tile
  static_assert(PIECES % NW == 0 && PPW >= 1, "the pieces are shared out evenly");
  static_assert(KT >= D, "the ring is filled before the first multiply");
  static_assert(4 + (D - 1) * PER_KT <= 63, "the wait counter has six bits");
  extern __shared__ __align__(16) char ix_gd_lds[];  // (D + 1) slots

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 31, g = lane >> 5;
  const int unit = blockIdx.x * NW + wave;
  const bool has_unit = unit < units;
  // a wave without a unit walks the last one (it still fetches its pieces and meets the barriers) and stores nothing
  const uint4* wp = reinterpret_cast<const uint4*>(Wf) + (long)min(unit, units - 1) * KT * 256 + lane;

  // this wave's pieces: piece p = (row block p / 4, step p % 4); the lane's 16 bytes are A[32 tb + r][32 g + 8 s ..]
  const ix_rsrc_t a_rsrc = ix_make_rsrc(A, (uint32_t)(((long)(M - 1) * lda + (long)KT * 64) * 2));
  uint32_t a_voff[PPW];
  uint32_t a_dst[PPW];
  const uint32_t lds_base = __builtin_amdgcn_readfirstlane(ix_lds_addr(ix_gd_lds));
#pragma unroll
  for (int j = 0; j < PPW; ++j) {
    const int p = wave * PPW + j, tb = p >> 2, s = p & 3;
    const int row = 32 * tb + r;
    a_voff[j] = row < M ? (uint32_t)(((long)row * lda + 32 * g + 8 * s) * 2) : IX_OOB;  // a row A does not have reads as zeros
    a_dst[j] = __builtin_amdgcn_readfirstlane(lds_base + (uint32_t)p * 1024u);  // wave-uniform: it travels in M0
  }
  auto fetch_a = [&](auto ktc) {
    constexpr int kt = decltype(ktc)::value;
#pragma unroll
    for (int j = 0; j < PPW; ++j) ix_dma16(a_rsrc, a_dst[j] + (uint32_t)((kt % (D + 1)) * SLOT), a_voff[j], kt * 128);
  };

  uint4 wreg[D][4];
  auto load_w = [&](auto ktc) {
    constexpr int kt = decltype(ktc)::value;
#pragma unroll
    for (int c = 0; c < 4; ++c) wreg[kt % D][c] = wp[kt * 256 + c * 64];
  };

  ix_f32x16 acc[TB];
#pragma unroll
  for (int tb = 0; tb < TB; ++tb)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[tb][i] = 0.0f;

  ix_static_for<0, D>([&](auto dc) {
    fetch_a(dc);
    load_w(dc);
  });
  __builtin_amdgcn_sched_barrier(0);
  ix_static_for<0, KT>([&](auto kc) {
    constexpr int kt = decltype(kc)::value;
    // younger than this wave's pieces of k-tile kt: its own 4 weight loads and all of the k-tiles after it in flight
    constexpr int younger = 4 + ((kt + D <= KT ? D : KT - kt) - 1) * PER_KT;
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(younger) : "memory");
    // every wave's pieces of k-tile kt are in LDS after the barrier; and every wave has read k-tile kt - 1 out of its
    // slot (its matrix instructions took the fragments before it came here), which the fetch below writes into
    __builtin_amdgcn_s_barrier();
    asm volatile("" : : : "memory");
    const char* slot = ix_gd_lds + (kt % (D + 1)) * SLOT + lane * 16;
    uint4 xf[TB][4];
#pragma unroll
    for (int tb = 0; tb < TB; ++tb)
#pragma unroll
      for (int s = 0; s < 4; ++s) xf[tb][s] = *reinterpret_cast<const uint4*>(slot + (tb * 4 + s) * 1024);
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
      for (int tb = 0; tb < TB; ++tb)
        acc[tb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const ix_bf16x8*>(&wreg[kt % D][s]),
                                                          *reinterpret_cast<const ix_bf16x8*>(&xf[tb][s]), acc[tb], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (kt + D < KT) {
      fetch_a(std::integral_constant<int, kt + D>{});
      load_w(std::integral_constant<int, kt + D>{});
    }
    __builtin_amdgcn_sched_barrier(0);
  });

  if (!has_unit) return;
#pragma unroll
  for (int tb = 0; tb < TB; ++tb) {
    const int m = 32 * tb + r;
    if (m >= M) continue;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const long n = 32L * unit + ix_acc_row(q * 4, lane);
      ix_store4_bf16(C + m * ldc + n, 4, true, acc[tb][q * 4], acc[tb][q * 4 + 1], acc[tb][q * 4 + 2], acc[tb][q * 4 + 3]);
    }
  }
}

// The k-tile counts the straight-line kernels are instantiated for (K = 64 KT).
#define IX_GD_KTS(F) F(16) F(32) F(48) F(64)

static bool ix_gemm_decode_serves(long N, long K) {
  if (N <= 0 || K <= 0 || (N % 32) || (K % 64)) return false;
#define IX_GD_IS(KT_) if (K / 64 == KT_) return true;
  IX_GD_KTS(IX_GD_IS)
#undef IX_GD_IS
  return false;
}

extern "C" int ix_gemm_decode_serves_shape(long N, long K) { return ix_gemm_decode_serves(N, K) ? 1 : 0; }

extern "C" int ix_gemm_pack_decode(const void* W, long ldw, void* Wf, long N, long K, void* stream) {
  if (!W || !Wf || N <= 0 || K <= 0 || ldw < K) return IX_ERR_ARG;
  if (!ix_gemm_decode_serves(N, K) || (ldw % 8) || !ix_aligned(W, 16) || !ix_aligned(Wf, 16)) return IX_DECLINED;
  const long chunks = N * K / 8;
  if ((chunks + 255) / 256 > 0x7fffffffL) return IX_DECLINED;
  hipLaunchKernelGGL(k_gemm_pack_frag, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (const bf16_t*)W, ldw, (bf16_t*)Wf, (int)(K / 64), chunks);
  return ix_launch_status();
}

template <int KT, int TB, int NW>
static int ix_gemm_dec_launch(const bf16_t* A, long lda, int M, const bf16_t* Wf, bf16_t* C, long ldc, int units,
                              hipStream_t st) {
  constexpr int LDS = (IX_GD_D + 1) * TB * 4 * 1024;
  auto kern = k_gemm_dec<KT, TB, NW>;
  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS) != hipSuccess)
      return IX_ERR_LAUNCH;
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)((units + NW - 1) / NW)), dim3(NW * 64), LDS, st, A, lda, M, Wf, C, ldc, units);
  return ix_launch_status();
}

// C[M, N] (bf16, row pitch ldc) = A[M, K] (bf16, row pitch lda) . W^T from the packed copy of W[N, K]; M <= 64.
// Four waves per workgroup once there are units for every CU's eight waves, two below that (more workgroups, each staging
// the activations for fewer units).
extern "C" int ix_gemm_bf16_nt_decode(const void* A, long lda, const void* Wf, void* C, long ldc, long M, long N, long K,
                                      void* stream) {
  if (!A || !Wf || !C || M < 0 || N <= 0 || K <= 0 || lda < K || ldc < N) return IX_ERR_ARG;
  if (M > 64 || !ix_gemm_decode_serves(N, K) || (lda % 8) || (ldc % 4) || !ix_aligned(A, 16) || !ix_aligned(Wf, 16) ||
      !ix_aligned(C, 8))
    return IX_DECLINED;
  if (((M - 1) * lda + K) * 2 >= 0x40000000L || N / 32 > 0x3fffffL) return IX_DECLINED;  // 32-bit offsets
  if (M == 0) return IX_OK;
  hipStream_t st = (hipStream_t)stream;
  const bf16_t *a = (const bf16_t*)A, *wf = (const bf16_t*)Wf;
  bf16_t* c = (bf16_t*)C;
  const int units = (int)(N / 32), m = (int)M;
  const bool wide = units >= 2048;
#define IX_GD_GO(KT_)                                                                                   \
  if (K / 64 == KT_) {                                                                                  \
    if (M > 32) {                                                                                       \
      if (wide) return ix_gemm_dec_launch<KT_, 2, 4>(a, lda, m, wf, c, ldc, units, st);                 \
      return ix_gemm_dec_launch<KT_, 2, 2>(a, lda, m, wf, c, ldc, units, st);                           \
    }                                                                                                   \
    if (wide) return ix_gemm_dec_launch<KT_, 1, 4>(a, lda, m, wf, c, ldc, units, st);                   \
    return ix_gemm_dec_launch<KT_, 1, 2>(a, lda, m, wf, c, ldc, units, st);                             \
  }
  IX_GD_KTS(IX_GD_GO)
#undef IX_GD_GO
  return IX_DECLINED;
}
