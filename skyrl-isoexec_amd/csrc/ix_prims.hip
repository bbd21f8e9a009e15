// Elementwise export of the device primitives the kernels share (ix_common.h), plus the
// library's self-description. A host-side checker evaluates a kernel's rounding schedule with
// these exact functions plugged in, which separates "is the order of operations the documented
// one" (bit-exact) from "how close is the device exp/log to libm" (tolerance).
#include "ix_common.h"
#include "../../include/isoexec_hip.h"

__global__ __launch_bounds__(256) void k_prim_unary(int op, const float* __restrict__ x, float* __restrict__ y,
                                                    long n) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const float v = x[i];
  float r;
  switch (op) {
    case IX_PRIM_EXP: r = ix_exp(v); break;
    case IX_PRIM_LOG: r = ix_log(v); break;
    case IX_PRIM_EXP_FAST: r = ix_exp_fast(v); break;
    case IX_PRIM_SIGMOID: r = ix_sigmoid(v); break;
    case IX_PRIM_SILU_DIV: r = ix_silu_div(v); break;
    case IX_PRIM_SOFTPLUS: r = ix_softplus(v); break;
    case IX_PRIM_RSQRT_IEEE: r = ix_rsqrt_ieee(v); break;
    case IX_PRIM_ROUND_BF16: r = ix_rbf(v); break;
    case IX_PRIM_EXP2: r = ix_exp2(v); break;
    default: r = v; break;
  }
  y[i] = r;
}

extern "C" int ix_prim_unary(int op, const float* x, float* y, long n, void* stream) {
  if (!x || !y || n < 0) return IX_ERR_ARG;
  if (op < 0 || op >= IX_PRIM_COUNT) return IX_ERR_ARG;
  if (n == 0) return IX_OK;
  const long grid = (n + 255) / 256;
  if (grid > 0x7fffffffL) return IX_DECLINED;
  hipLaunchKernelGGL(k_prim_unary, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, op, x, y, n);
  return ix_launch_status();
}

extern "C" int ix_abi_version(void) { return IX_ABI_VERSION; }

extern "C" const char* ix_arch_tag(void) { return "gfx950"; }
