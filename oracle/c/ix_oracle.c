/* CPU restatement helpers in plain C: the loops whose rounding uses fused multiply-adds (numpy
 * has none) or that are too slow in Python. TEST INFRASTRUCTURE ONLY -- never linked into, or
 * called from, the product library.
 *
 * Build: gcc -O2 -fPIC -shared -mfma -ffp-contract=off -fno-fast-math ix_oracle.c -o libix_oracle.so -lm
 * (-ffp-contract=off: a fused multiply-add happens only where fmaf() is written.)
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

/* dot of two 8-element slices: (fma chain over 0,2,4,6) + (fma chain over 1,3,5,7) */
static inline float dot8(const float* s, const float* x) {
  float pa = s[0] * x[0];
  float pb = s[1] * x[1];
  pa = fmaf(s[2], x[2], pa);
  pb = fmaf(s[3], x[3], pb);
  pa = fmaf(s[4], x[4], pa);
  pb = fmaf(s[5], x[5], pb);
  pa = fmaf(s[6], x[6], pa);
  pb = fmaf(s[7], x[7], pb);
  return pa + pb;
}

/* adjacent-pairwise tree over n (power of two, <= 32) lane partials, in place */
static inline float lane_tree(float* p, int n) {
  for (int s = 1; s < n; s <<= 1)
    for (int i = 0; i + s < n; i += 2 * s) p[i] = p[i] + p[i + s];
  return p[0];
}

/* Gated delta-rule scan of ONE sequence (reference semantics: the recurrence behind
 * ops/gdn/gdn_ops.py:400-441; state layout [HV, V, K] as the engine pool of
 * ops/gdn/gdn_recurrent_state.py:190-192).
 *   q, k  [T, H, K]   (already l2-normalised; q NOT yet scaled)
 *   v, o  [T, HV, V]
 *   eg    [T, HV]     exp(g) already evaluated (the transcendental stays pluggable in Python)
 *   beta  [T, HV]
 *   state [HV, V, K]  in/out
 *   snap  NULL, or [T, HV, V, K]: state after every token (for mid-sequence store checks)
 * Order per row: S*=eg; kv = tree over K/8 lanes of dot8; d=(v-kv)*beta; S=fma(d,k,S);
 * o = tree over lanes of dot8(S, q*scale). */
void ixo_gdn_scan(const float* q, const float* k, const float* v, const float* eg, const float* beta, float* o,
                  float* state, float* snap, long T, int H, int HV, int K, int V, float scale) {
  const int KS = K / 8;
  float qs[256], part[32];
  for (long t = 0; t < T; ++t) {
    for (int hv = 0; hv < HV; ++hv) {
      const int h = hv / (HV / H);
      const float* kk = k + (t * H + h) * K;
      const float* qq = q + (t * H + h) * K;
      for (int i = 0; i < K; ++i) qs[i] = qq[i] * scale;
      const float e = eg[t * HV + hv], bt = beta[t * HV + hv];
      for (int r = 0; r < V; ++r) {
        float* S = state + ((long)hv * V + r) * K;
        for (int i = 0; i < K; ++i) S[i] = S[i] * e;
        for (int s = 0; s < KS; ++s) part[s] = dot8(S + 8 * s, kk + 8 * s);
        const float kv = lane_tree(part, KS);
        const float d = (v[(t * HV + hv) * V + r] - kv) * bt;
        for (int i = 0; i < K; ++i) S[i] = fmaf(d, kk[i], S[i]);
        for (int s = 0; s < KS; ++s) part[s] = dot8(S + 8 * s, qs + 8 * s);
        o[(t * HV + hv) * V + r] = lane_tree(part, KS);
      }
    }
    if (snap) memcpy(snap + t * (long)HV * V * K, state, sizeof(float) * (size_t)HV * V * K);
  }
}

/* Plain fp32 GEMM C[M,N] = A[M,K] . W[N,K]^T with a sequential fused-multiply-add chain over k.
 * Used as a fast tolerance reference and as the timed CPU baseline of the dense head. */
void ixo_gemm_nt_f32(const float* A, const float* W, float* C, long M, long N, long K) {
  for (long m = 0; m < M; ++m)
    for (long n = 0; n < N; ++n) {
      const float *a = A + m * K, *w = W + n * K;
      float acc = 0.0f;
      for (long kk = 0; kk < K; ++kk) acc = fmaf(a[kk], w[kk], acc);
      C[m * N + n] = acc;
    }
}
