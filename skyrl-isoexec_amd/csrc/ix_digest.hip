// Order-invariant digests of a tensor's integer image: position-weighted sums modulo 2^64.
//
//   sum_j = SUM_i (sext(x_i) & mask_j) * w(i)   (mod 2^64),
//   w(i)  = (mix64((i >> 3) ^ salt) ^ ((i & 7) * GOLDEN)) | 1,
//
// mix64 being the splitmix64 finaliser. Addition modulo 2^64 is associative and commutative, so the split
// into lanes, workgroups and partial sums below cannot reach the result: the same bytes give the same sums on
// any device under any decomposition. Up to eight masks are summed in one pass over the data (a ladder of
// mantissa truncations); in segmented form each run of seg_numel elements is summed on its own, its positions
// counted from the start of the run and its salt derived from the run's absolute offset.
// (The scheme of the reference's debug digest: isoexec/debug/thash.py:1-6, 180-196, 312-343 and the kernels
// isoexec/debug/thash_kernels.py:42-104. Those accumulate with integer atomics into a zeroed arena; here a
// workgroup writes its partial sums and a second launch adds them, so nothing has to start at zero.)
#include "ix_common.h"
#include "../../include/isoexec_hip.h"

#define DG_THREADS 256
#define DG_UNROLL 4          // groups whose loads are in flight together
#define DG_MAX_BLOCKS 2048   // upper bound on workgroups per launch along x and on partial rows per segment

static constexpr uint64_t DG_MIX1 = 0xBF58476D1CE4E5B9ull;
static constexpr uint64_t DG_MIX2 = 0x94D049BB133111EBull;
static constexpr uint64_t DG_GOLDEN = 0x9E3779B97F4A7C15ull;

__host__ __device__ __forceinline__ uint64_t dg_mix(uint64_t z) {
  z ^= z >> 30;
  z *= DG_MIX1;
  z ^= z >> 27;
  z *= DG_MIX2;
  return z ^ (z >> 31);
}

struct DgMasks {
  uint32_t lo[IX_DIGEST_MAX_MASKS];
  uint32_t hi[IX_DIGEST_MAX_MASKS];
};

// Eight consecutive elements of EB bytes each, as sign-extended 64-bit integers split into (low word, high word).
// Elements of up to 4 bytes keep only the low word; their high word is the sign, rebuilt where it is needed.
template <int EB>
__device__ __forceinline__ void dg_load8(const char* __restrict__ p, int cnt, bool vec, uint32_t (&lo)[8],
                                         uint32_t (&hi)[8]) {
  if (vec && cnt == 8) {
    if constexpr (EB == 1) {
      const uint2 u = *reinterpret_cast<const uint2*>(p);
      const uint32_t w[2] = {u.x, u.y};
#pragma unroll
      for (int i = 0; i < 8; ++i) lo[i] = (uint32_t)(int32_t)(int8_t)((w[i >> 2] >> (8 * (i & 3))) & 0xffu);
    } else if constexpr (EB == 2) {
      const uint4 u = *reinterpret_cast<const uint4*>(p);
      const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
      for (int i = 0; i < 8; ++i) lo[i] = (uint32_t)(int32_t)(int16_t)((w[i >> 1] >> (16 * (i & 1))) & 0xffffu);
    } else if constexpr (EB == 4) {
      const uint4 a = reinterpret_cast<const uint4*>(p)[0];
      const uint4 b = reinterpret_cast<const uint4*>(p)[1];
      lo[0] = a.x; lo[1] = a.y; lo[2] = a.z; lo[3] = a.w;
      lo[4] = b.x; lo[5] = b.y; lo[6] = b.z; lo[7] = b.w;
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uint4 a = reinterpret_cast<const uint4*>(p)[q];
        lo[2 * q] = a.x; hi[2 * q] = a.y;
        lo[2 * q + 1] = a.z; hi[2 * q + 1] = a.w;
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      lo[i] = 0;
      if constexpr (EB == 8) hi[i] = 0;
      if (i < cnt) {
        if constexpr (EB == 1) lo[i] = (uint32_t)(int32_t)reinterpret_cast<const int8_t*>(p)[i];
        else if constexpr (EB == 2) lo[i] = (uint32_t)(int32_t)reinterpret_cast<const int16_t*>(p)[i];
        else if constexpr (EB == 4) lo[i] = reinterpret_cast<const uint32_t*>(p)[i];
        else {
          const uint2 u = reinterpret_cast<const uint2*>(p)[i];
          lo[i] = u.x;
          hi[i] = u.y;
        }
      }
    }
  }
}

// Adds group g's eight elements, each times its weight, to the NM sums. Absent elements are zero and add nothing.
template <int EB, int NM>
__device__ __forceinline__ void dg_fold(long g, uint64_t salt, const uint32_t (&lo)[8], const uint32_t (&hi)[8],
                                        const DgMasks& masks, uint64_t (&acc)[NM]) {
  const uint64_t wbase = dg_mix((uint64_t)g ^ salt);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint64_t w = (wbase ^ ((uint64_t)i * DG_GOLDEN)) | 1ull;
    const uint32_t sign = EB == 8 ? hi[i] : (uint32_t)((int32_t)lo[i] >> 31);
#pragma unroll
    for (int j = 0; j < NM; ++j) {
      acc[j] += (uint64_t)(lo[i] & masks.lo[j]) * w;
      if (masks.hi[j]) acc[j] += (uint64_t)((sign & masks.hi[j]) * (uint32_t)w) << 32;
    }
  }
}

// One workgroup's share of one segment: groups of eight elements dealt to threads, then a fixed tree over the
// workgroup (any order would do). partials[(segment * nb + blockIdx.x) * NM + j]; with nb == 1 that IS the result.
template <int EB, int NM>
__global__ __launch_bounds__(DG_THREADS) void k_digest_partial(const char* __restrict__ x, long n, long seg_numel,
                                                               long nseg, int segmented, uint64_t salt_or_seed,
                                                               DgMasks masks, uint64_t* __restrict__ partials) {
  __shared__ uint64_t s_part[DG_THREADS / IX_WAVE][NM];
  const int nb = (int)gridDim.x;
  const int lane = threadIdx.x & (IX_WAVE - 1), wave = threadIdx.x / IX_WAVE;
  for (long seg = blockIdx.y; seg < nseg; seg += gridDim.y) {
    const long base = seg * seg_numel;
    const long len = (n - base) < seg_numel ? (n - base) : seg_numel;
    const uint64_t salt = segmented ? (dg_mix(salt_or_seed ^ dg_mix((uint64_t)base + 1)) ^ DG_GOLDEN) : salt_or_seed;
    const long ngroups = (len + 7) >> 3;
    const char* xs = x + base * EB;
    // 16-byte loads need the segment's first byte on a 16-byte boundary (8 for one-byte elements)
    const bool vec = (reinterpret_cast<uintptr_t>(xs) & (EB == 1 ? 7 : 15)) == 0;
    uint64_t acc[NM];
#pragma unroll
    for (int j = 0; j < NM; ++j) acc[j] = 0;
    const long stride = (long)nb * DG_THREADS;
    long g = (long)blockIdx.x * DG_THREADS + threadIdx.x;
    // DG_UNROLL groups per trip: their loads are issued together, then each is folded into the sums
    // (only while all of them are whole groups behind an aligned start: no branch between the loads)
    if (vec) {
      for (; ((g + (DG_UNROLL - 1) * stride) << 3) + 8 <= len; g += DG_UNROLL * stride) {
        uint32_t lo[DG_UNROLL][8], hi[DG_UNROLL][8];
#pragma unroll
        for (int u = 0; u < DG_UNROLL; ++u) dg_load8<EB>(xs + ((g + u * stride) << 3) * EB, 8, true, lo[u], hi[u]);
#pragma unroll
        for (int u = 0; u < DG_UNROLL; ++u) dg_fold<EB, NM>(g + u * stride, salt, lo[u], hi[u], masks, acc);
      }
    }
    for (; g < ngroups; g += stride) {
      const long off = g << 3;
      uint32_t lo[8], hi[8];
      dg_load8<EB>(xs + off * EB, (len - off) < 8 ? (int)(len - off) : 8, vec, lo, hi);
      dg_fold<EB, NM>(g, salt, lo, hi, masks, acc);
    }
#pragma unroll
    for (int j = 0; j < NM; ++j) {
      uint64_t v = acc[j];
#pragma unroll
      for (int d = IX_WAVE / 2; d >= 1; d >>= 1) v += __shfl_xor((unsigned long long)v, d, IX_WAVE);
      if (lane == 0) s_part[wave][j] = v;
    }
    __syncthreads();
    if (threadIdx.x < NM) {
      uint64_t v = 0;
#pragma unroll
      for (int w = 0; w < DG_THREADS / IX_WAVE; ++w) v += s_part[w][threadIdx.x];
      partials[(seg * nb + blockIdx.x) * NM + threadIdx.x] = v;
    }
    __syncthreads();
  }
}

// out[r] = SUM_b partials[(r / nm * nb + b) * nm + r % nm]: one workgroup per result, its loads independent.
__global__ __launch_bounds__(DG_THREADS) void k_digest_finish(const uint64_t* __restrict__ partials, int nb, int nm,
                                                              uint64_t* __restrict__ out) {
  __shared__ uint64_t s_part[DG_THREADS / IX_WAVE];
  const int lane = threadIdx.x & (IX_WAVE - 1), wave = threadIdx.x / IX_WAVE;
  const long r = blockIdx.x;
  const long seg = r / nm;
  const int j = (int)(r % nm);
  uint64_t v = 0;
  for (int b = threadIdx.x; b < nb; b += DG_THREADS) v += partials[(seg * nb + b) * nm + j];
#pragma unroll
  for (int d = IX_WAVE / 2; d >= 1; d >>= 1) v += __shfl_xor((unsigned long long)v, d, IX_WAVE);
  if (lane == 0) s_part[wave] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint64_t total = 0;
#pragma unroll
    for (int w = 0; w < DG_THREADS / IX_WAVE; ++w) total += s_part[w];
    out[r] = total;
  }
}

// Workgroups per segment: enough that a thread sees about four groups, few enough that all segments together stay
// within DG_MAX_BLOCKS partial rows (one row per segment when there are many segments).
static int dg_blocks_per_segment(long nseg, long seg_numel) {
  const long groups = (seg_numel + 7) / 8;
  long nb = (groups + DG_THREADS * 4 - 1) / (DG_THREADS * 4);
  long cap = DG_MAX_BLOCKS / (nseg < 1 ? 1 : nseg);
  if (cap < 1) cap = 1;
  if (nb > cap) nb = cap;
  return nb < 1 ? 1 : (int)nb;
}

extern "C" size_t ix_digest_workspace_words(long nseg, long seg_numel, int nmask) {
  if (nseg < 1 || seg_numel < 0 || nmask < 1) return 0;
  const int nb = dg_blocks_per_segment(nseg, seg_numel);
  return nb == 1 ? 0 : (size_t)nseg * (size_t)nb * (size_t)nmask;
}

template <int EB, int NM>
static void dg_launch(const void* x, long n, long seg_numel, long nseg, int segmented, uint64_t salt_or_seed,
                      const DgMasks& masks, uint64_t* dst, int nb, hipStream_t stream) {
  const unsigned gy = (unsigned)(nseg < 65535 ? nseg : 65535);
  hipLaunchKernelGGL((k_digest_partial<EB, NM>), dim3((unsigned)nb, gy), dim3(DG_THREADS), 0, stream,
                     (const char*)x, n, seg_numel, nseg, segmented, salt_or_seed, masks, dst);
}

template <int EB>
static void dg_launch_nm(int nm, const void* x, long n, long seg_numel, long nseg, int segmented,
                         uint64_t salt_or_seed, const DgMasks& masks, uint64_t* dst, int nb, hipStream_t stream) {
#define DG_CASE(NM_)                                                                                   \
  case NM_: dg_launch<EB, NM_>(x, n, seg_numel, nseg, segmented, salt_or_seed, masks, dst, nb, stream); break;
  switch (nm) {
    DG_CASE(1) DG_CASE(2) DG_CASE(3) DG_CASE(4) DG_CASE(5) DG_CASE(6) DG_CASE(7) DG_CASE(8)
    default: break;
  }
#undef DG_CASE
}

static int dg_run(const void* x, int elem_bytes, long n, long nseg, long seg_numel, int segmented,
                  uint64_t salt_or_seed, const uint64_t* masks, int nmask, uint64_t* workspace,
                  size_t workspace_words, uint64_t* out, void* stream) {
  if (!out || n < 0 || nseg < 1 || seg_numel < 0 || !masks) return IX_ERR_ARG;
  if (nmask < 1 || nmask > IX_DIGEST_MAX_MASKS) return IX_ERR_ARG;
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8) return IX_ERR_ARG;
  if (n > 0 && (!x || !ix_aligned(x, (size_t)elem_bytes))) return IX_ERR_ARG;
  // every segment but the last is full and the last is not empty; an empty tensor is one empty segment
  if (n == 0 ? nseg != 1 : (seg_numel < 1 || nseg != (n + seg_numel - 1) / seg_numel)) return IX_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  DgMasks m;
  for (int j = 0; j < IX_DIGEST_MAX_MASKS; ++j) {
    m.lo[j] = j < nmask ? (uint32_t)masks[j] : 0u;
    m.hi[j] = j < nmask ? (uint32_t)(masks[j] >> 32) : 0u;
  }
  const int nb = dg_blocks_per_segment(nseg, seg_numel);
  const size_t need = nb == 1 ? 0 : (size_t)nseg * (size_t)nb * (size_t)nmask;
  if (need && (!workspace || workspace_words < need)) return IX_ERR_ARG;
  uint64_t* dst = nb == 1 ? out : workspace;
  switch (elem_bytes) {
    case 1: dg_launch_nm<1>(nmask, x, n, seg_numel, nseg, segmented, salt_or_seed, m, dst, nb, st); break;
    case 2: dg_launch_nm<2>(nmask, x, n, seg_numel, nseg, segmented, salt_or_seed, m, dst, nb, st); break;
    case 4: dg_launch_nm<4>(nmask, x, n, seg_numel, nseg, segmented, salt_or_seed, m, dst, nb, st); break;
    default: dg_launch_nm<8>(nmask, x, n, seg_numel, nseg, segmented, salt_or_seed, m, dst, nb, st); break;
  }
  int rc = ix_launch_status();
  if (rc != IX_OK || nb == 1) return rc;
  // nb > 1 only when nseg <= DG_MAX_BLOCKS / 2, so the grid is small
  hipLaunchKernelGGL(k_digest_finish, dim3((unsigned)(nseg * nmask)), dim3(DG_THREADS), 0, st, workspace, nb, nmask,
                     out);
  return ix_launch_status();
}

extern "C" int ix_digest_sums(const void* x, int elem_bytes, long n, uint64_t salt, const uint64_t* masks, int nmask,
                              uint64_t* workspace, size_t workspace_words, uint64_t* out, void* stream) {
  return dg_run(x, elem_bytes, n, 1, n, 0, salt, masks, nmask, workspace, workspace_words, out, stream);
}

extern "C" int ix_digest_segment_sums(const void* x, int elem_bytes, long n, long nseg, long seg_numel, uint64_t seed,
                                      uint64_t mask, uint64_t* workspace, size_t workspace_words, uint64_t* out,
                                      void* stream) {
  return dg_run(x, elem_bytes, n, nseg, seg_numel, 1, seed, &mask, 1, workspace, workspace_words, out, stream);
}
