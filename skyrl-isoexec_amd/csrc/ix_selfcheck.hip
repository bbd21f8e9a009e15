// Device self-check (reference ops/collectives/pik_bootstrap.py:82-93 `pik_arch_selfcheck` -> pik/arch.py:90-168
// `_verify`: "check on this GPU that no GEMM tiling knob moves the bits of a non-split-K K-reduction"). The reference
// runs one product with a wide exponent spread through every tiling it can compile and counts distinct results; a
// provider whose premise fails on the device it meets is switched off for good. Here the same question is put to the
// library's own kernels, on the device, through its own entry points:
//   bit 0  seeded product, operands with a wide exponent spread: every tile shape and launch form of ix_gemm_bf16_nt
//          (ids 1..8) stores the same bits as id 1;
//   bit 1  small-integer operands (every partial sum exact in fp32, so the result does not depend on any order): every
//          id stores bf16(the integer product), computed independently by a plain integer kernel;
//   bit 2  the row-invariant log-softmax + gather gives the same bits in both of its launch shapes (seeded logits);
//   bit 3  an id declined a shape it documents as served (nothing compared for it).
// The caller owns the scratch memory; nothing is allocated. The call ends with a stream synchronisation and a 16-byte
// copy to the host: it is a set-up call, not a hot-path one.
#include "ix_common.h"
#include "../../include/isoexec_hip.h"

#define IX_SC_M 512
#define IX_SC_N 1024
#define IX_SC_K 1024  // a multiple of 64 and >= 704: the streaming form serves it
#define IX_SC_G 8

// splitmix64 finaliser: a stateless generator, the same values on every launch shape
__device__ __forceinline__ uint64_t ix_sc_mix(uint64_t z) {
  z += 0x9e3779b97f4a7c15ull;
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  return z ^ (z >> 31);
}

// mode 0: sign * 2^e * (1 + m / 128), e in [-12, 12]: a spread of 2^24 between operands, so that a changed
// summation order shows in the rounding of almost every partial sum. mode 1: integers in [-3, 3]. mode 2: the same
// form as mode 0 with e in [-3, 2] (logit-sized values, so that many columns of a row contribute to its sum).
__global__ __launch_bounds__(256) void k_sc_fill(bf16_t* __restrict__ p, long n, uint64_t seed, int mode) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const uint64_t h = ix_sc_mix(seed ^ (uint64_t)i * 0x2545f4914f6cdd1dull);
  if (mode == 0) {
    const uint32_t sign = (uint32_t)(h & 1u) << 15;
    const uint32_t e = 127u - 12u + (uint32_t)((h >> 1) % 25u);
    const uint32_t m = (uint32_t)(h >> 8) & 0x7fu;
    p[i] = (bf16_t)(sign | (e << 7) | m);
  } else if (mode == 1) {
    p[i] = ix_f2bf((float)((int)((h >> 3) % 7u) - 3));
  } else {
    const uint32_t sign = (uint32_t)(h & 1u) << 15;
    const uint32_t e = 127u - 3u + (uint32_t)((h >> 1) % 6u);
    const uint32_t m = (uint32_t)(h >> 8) & 0x7fu;
    p[i] = (bf16_t)(sign | (e << 7) | m);
  }
}

__global__ __launch_bounds__(256) void k_sc_targets(int64_t* __restrict__ t, long rows, long V, uint64_t seed) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < rows) t[i] = (int64_t)(ix_sc_mix(seed + (uint64_t)i) % (uint64_t)V);
}

// Integer truth for mode-1 operands: |sum| <= 9 K < 2^24, exact in int and in fp32; stored as bf16(sum).
__global__ __launch_bounds__(256) void k_sc_int_product(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W,
                                                        bf16_t* __restrict__ C, int M, int N, int K) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long)M * N) return;
  const int m = (int)(i / N), n = (int)(i % N);
  int acc = 0;
  for (int k = 0; k < K; ++k) acc += (int)ix_bf2f(A[(long)m * K + k]) * (int)ix_bf2f(W[(long)n * K + k]);
  C[i] = ix_f2bf((float)acc);
}

// flags[which] = 1 if any 32-bit word differs (every writer stores the same value: no ordering is needed)
__global__ __launch_bounds__(256) void k_sc_compare(const uint32_t* __restrict__ a, const uint32_t* __restrict__ b,
                                                    long words, int* __restrict__ flags, int which) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < words && a[i] != b[i]) flags[which] = 1;
}

// Flips the lowest bit of one 32-bit word: how ix_arch_selfcheck_probe shows that a comparison sees a single bit.
__global__ void k_sc_flip(uint32_t* __restrict__ words, long at) {
  if (threadIdx.x == 0 && blockIdx.x == 0) words[at] ^= 1u;
}

__global__ void k_sc_clear(int* __restrict__ flags) {
  if (threadIdx.x < 4) flags[threadIdx.x] = 0;
}

static inline size_t ix_sc_up(size_t x) { return (x + 255) & ~(size_t)255; }

struct IxScLayout {
  size_t a, w, c_ref, c_got, targets, lp1, lp2, lp_ws, lp_ws_bytes, flags, total;
};

static IxScLayout ix_sc_layout() {
  IxScLayout L;
  size_t at = 0;
  const auto take = [&](size_t bytes) { const size_t here = at; at += ix_sc_up(bytes); return here; };
  L.a = take((size_t)IX_SC_M * IX_SC_K * 2);
  L.w = take((size_t)IX_SC_N * IX_SC_K * 2);
  L.c_ref = take((size_t)IX_SC_M * IX_SC_N * 2);
  L.c_got = take((size_t)IX_SC_M * IX_SC_N * 2);
  L.targets = take((size_t)IX_SC_M * 8);
  L.lp1 = take((size_t)IX_SC_M * 4);
  L.lp2 = take((size_t)IX_SC_M * 4);
  L.lp_ws_bytes = ix_logprob_workspace_bytes(IX_SC_M, IX_SC_N, IX_SC_G);
  L.lp_ws = take(L.lp_ws_bytes);
  L.flags = take(16);
  L.total = at;
  return L;
}

extern "C" size_t ix_arch_selfcheck_workspace_bytes(void) { return ix_sc_layout().total; }

extern "C" int ix_arch_selfcheck(void* workspace, size_t workspace_bytes, unsigned* failed_checks, void* stream) {
  return ix_arch_selfcheck_probe(workspace, workspace_bytes, 0u, failed_checks, stream);
}

// The self-check with one bit of a comparison's reference side flipped first, for every check named in `inject` (bits
// 0..2 as in failed_checks): the call must then report exactly those checks. It is how a test (or a suspicious
// operator) shows that the comparisons have teeth; inject = 0 is the self-check itself.
extern "C" int ix_arch_selfcheck_probe(void* workspace, size_t workspace_bytes, unsigned inject, unsigned* failed_checks,
                                       void* stream) {
  if (failed_checks) *failed_checks = 0;
  const IxScLayout L = ix_sc_layout();
  if (!workspace || !ix_aligned(workspace, 256)) return IX_ERR_ARG;
  if (workspace_bytes < L.total) return IX_ERR_SIZE;
  hipStream_t st = (hipStream_t)stream;
  char* base = static_cast<char*>(workspace);
  bf16_t* A = (bf16_t*)(base + L.a);
  bf16_t* W = (bf16_t*)(base + L.w);
  bf16_t* Cref = (bf16_t*)(base + L.c_ref);
  bf16_t* Cgot = (bf16_t*)(base + L.c_got);
  int64_t* targets = (int64_t*)(base + L.targets);
  float* lp1 = (float*)(base + L.lp1);
  float* lp2 = (float*)(base + L.lp2);
  int* flags = (int*)(base + L.flags);
  const int M = IX_SC_M, N = IX_SC_N, K = IX_SC_K;
  const long nA = (long)M * K, nW = (long)N * K, nC = (long)M * N;
  const auto grid = [](long n) { return dim3((unsigned)((n + 255) / 256)); };
  unsigned declined = 0;

  hipLaunchKernelGGL(k_sc_clear, dim3(1), dim3(64), 0, st, flags);
  for (int mode = 0; mode < 2; ++mode) {
    hipLaunchKernelGGL(k_sc_fill, grid(nA), dim3(256), 0, st, A, nA, 0x1234ull + (uint64_t)mode, mode);
    hipLaunchKernelGGL(k_sc_fill, grid(nW), dim3(256), 0, st, W, nW, 0x9876ull + (uint64_t)mode, mode);
    if (mode == 0) {
      const int rc = ix_gemm_bf16_nt(A, K, W, K, nullptr, Cref, IX_DT_BF16, N, M, N, K, 1, nullptr, 0, stream);
      if (rc < 0) return rc;
      if (rc != IX_OK) return IX_ERR_LAUNCH;  // the reference tile serves every 16-byte aligned shape
    } else {
      hipLaunchKernelGGL(k_sc_int_product, grid(nC), dim3(256), 0, st, A, W, Cref, M, N, K);
    }
    if (inject >> mode & 1u) hipLaunchKernelGGL(k_sc_flip, dim3(1), dim3(64), 0, st, (uint32_t*)Cref, nC / 4 + 17);
    for (int tile = mode == 0 ? 2 : 1; tile <= 8; ++tile) {
      const int rc = ix_gemm_bf16_nt(A, K, W, K, nullptr, Cgot, IX_DT_BF16, N, M, N, K, tile, nullptr, 0, stream);
      if (rc < 0) return rc;
      if (rc != IX_OK) {
        declined |= 1u << tile;
        continue;
      }
      hipLaunchKernelGGL(k_sc_compare, grid(nC / 2), dim3(256), 0, st, (const uint32_t*)Cref, (const uint32_t*)Cgot,
                         nC / 2, flags, mode);
    }
    if (mode == 0) {
      // seeded logits (the product buffer is free again) through both launch shapes of the log-softmax
      hipLaunchKernelGGL(k_sc_fill, grid(nC), dim3(256), 0, st, Cgot, nC, 0x4242ull, 2);
      hipLaunchKernelGGL(k_sc_targets, grid(M), dim3(256), 0, st, targets, (long)M, (long)N, 0x5555ull);
      float* outs[2] = {lp1, lp2};
      for (int shape = 1; shape <= 2; ++shape) {
        const int rc = ix_logprob_rowinv_sampled(Cgot, IX_DT_BF16, M, N, N, targets, IX_SC_G, outs[shape - 1], nullptr,
                                                 base + L.lp_ws, L.lp_ws_bytes, shape, nullptr, stream);
        if (rc < 0) return rc;
        if (rc != IX_OK) declined |= 1u << (8 + shape);
      }
      if (inject >> 2 & 1u) hipLaunchKernelGGL(k_sc_flip, dim3(1), dim3(64), 0, st, (uint32_t*)lp1, (long)(M / 2));
      hipLaunchKernelGGL(k_sc_compare, grid(M), dim3(256), 0, st, (const uint32_t*)lp1, (const uint32_t*)lp2, (long)M,
                         flags, 2);
    }
  }
  if (ix_launch_status() != IX_OK) return IX_ERR_LAUNCH;
  int host_flags[4] = {0, 0, 0, 0};
  if (hipMemcpyAsync(host_flags, flags, sizeof(host_flags), hipMemcpyDeviceToHost, st) != hipSuccess) return IX_ERR_LAUNCH;
  if (hipStreamSynchronize(st) != hipSuccess) return IX_ERR_LAUNCH;
  unsigned failed = 0;
  for (int i = 0; i < 3; ++i)
    if (host_flags[i]) failed |= 1u << i;
  if (declined) failed |= 1u << 3;
  if (failed_checks) *failed_checks = failed;
  return failed ? IX_DECLINED : IX_OK;
}
