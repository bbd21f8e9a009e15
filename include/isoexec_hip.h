/* C ABI of libisoexec_hip.so: the gfx950 kernels of the batch-invariant token-logprob path.
 *
 * The reference (zanderjiang/SkyRL-IsoExec) has no C ABI on this path; its operator interface is
 * Python (op functions + aten overrides + _register.py declarations) over Triton/CUDA kernels.
 * Each entry point below names the reference function whose arithmetic it replaces; paths are
 * relative to skyrl/backends/skyrl_train/isoexec/ in the reference tree.
 *
 * Conventions
 *   - plain pointers and sizes only; every pointer is DEVICE memory unless stated otherwise;
 *   - the caller owns all memory, outputs and workspaces included; no entry point allocates,
 *     frees, synchronises the device or reads device memory back to the host;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *   - return value: 0 = launched, > 0 = declined (shape/dtype outside the envelope: nothing
 *     was launched, the caller decides), < 0 = error (bad argument or launch failure);
 *   - dtype codes: IX_DT_F32 = 0, IX_DT_BF16 = 1; bf16 values are raw uint16 bit patterns;
 *   - results never depend on batch size, token count, tile choice or launch shape: arguments
 *     named `tile`, `force_shape`, `time_tile`, `BM` choose who computes an element, not how.
 */
#ifndef ISOEXEC_HIP_H
#define ISOEXEC_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define IX_ABI_VERSION 3

#ifndef IX_OK
#define IX_OK 0
#define IX_DECLINED 1
#define IX_ERR_ARG (-1)
#define IX_ERR_LAUNCH (-2)
#define IX_ERR_SIZE (-3) /* input larger than a fixed internal buffer */
#define IX_DT_F32 0
#define IX_DT_BF16 1
#endif

/* primitive codes for ix_prim_unary */
#define IX_PRIM_EXP 0
#define IX_PRIM_LOG 1
#define IX_PRIM_EXP_FAST 2
#define IX_PRIM_SIGMOID 3
#define IX_PRIM_SILU_DIV 4
#define IX_PRIM_SOFTPLUS 5
#define IX_PRIM_RSQRT_IEEE 6
#define IX_PRIM_ROUND_BF16 7
#define IX_PRIM_EXP2 8
#define IX_PRIM_COUNT 9

int ix_abi_version(void);
const char* ix_arch_tag(void); /* "gfx950"; counterpart of core/arch.py:27-51 detect_arch() tags */

/* y[i] = prim(x[i]) with the device's own exp/log/... as the kernels use them. A checker plugs
 * these into the CPU restatement so that order-of-operations parity is bit-exact. No
 * counterpart in the reference (its probes compare kernels against eager torch on device). */
int ix_prim_unary(int op, const float* x, float* y, long n, void* stream);

/* ---- device self-check: ops/collectives/pik_bootstrap.py:82-93 ----------------------------- */

/* pik_arch_selfcheck (pik_bootstrap.py:82-93 -> pik/arch.py:90-168 _verify: "check on this GPU that no GEMM tiling
 * knob moves the bits of a non-split-K K-reduction"; a failure disables the provider for good). Runs on the device,
 * through this library's own entry points: a seeded 512 x 1024 x 1024 product whose operands span 2^24 in magnitude
 * through every tile shape and launch form of ix_gemm_bf16_nt (ids 1..8), compared bit for bit on the device; the same
 * with small-integer operands against an independently computed integer product; and both launch shapes of
 * ix_logprob_rowinv_sampled on seeded logits. workspace: caller-owned device memory, 256-byte aligned, at
 * least ix_arch_selfcheck_workspace_bytes() (about 6 MiB); nothing is allocated. failed_checks (host memory, may be
 * NULL) receives a mask: bit 0 seeded product, bit 1 integer product, bit 2 log-softmax shapes, bit 3 an id declined
 * the shape. Returns IX_OK (every check passed), IX_DECLINED (a check failed: do not serve from this device), < 0
 * (the checks could not run). Ends with a stream synchronisation: a set-up call, not a hot-path one. */
size_t ix_arch_selfcheck_workspace_bytes(void);
int ix_arch_selfcheck(void* workspace, size_t workspace_bytes, unsigned* failed_checks, void* stream);
/* The same call with one bit of the reference side of every check named in `inject` (bits 0..2) flipped first: it must
 * then report exactly those checks. No counterpart in the reference; it shows that each comparison sees a single bit. */
int ix_arch_selfcheck_probe(void* workspace, size_t workspace_bytes, unsigned inject, unsigned* failed_checks,
                            void* stream);

/* ---- log-softmax + target gather: ops/logprobs/rowinv.py ---------------------------------- */

/* Workspace the split launch shape needs (bytes); 0 on invalid arguments. */
size_t ix_logprob_workspace_bytes(long rows, long V, int G);

/* rowinv_sampled_logprobs (rowinv.py:666-712; kernels leaf_sum_exp :136-154, finalize_rows
 * :156-191) at world size 1. logits [rows, V] (row pitch row_stride elements), target int64
 * [rows] (out of range -> logprob 0), G leaves (power of two, V % G == 0 else declined).
 * out_logprob fp32 [rows]; out_lse fp32 [rows] or NULL. force_shape: 0 auto, 1 one workgroup
 * per row, 2 split rows (needs the workspace). row_max_in: NULL, or fp32 [rows] holding each
 * row's exact maximum (e.g. ix_gemm_bf16_nt's row_max_parts reduced by ix_rowmax_reduce): the
 * max pass is skipped and the logits are read once. The workspace is always required with it. */
int ix_logprob_rowinv_sampled(const void* logits, int dtype, long rows, long V, long row_stride,
                              const int64_t* target, int G, float* out_logprob, float* out_lse,
                              void* workspace, size_t workspace_bytes, int force_shape,
                              const float* row_max_in, void* stream);

/* rowinv_full_logprobs (rowinv.py:796-875; kernel full_row_logprobs :193-245): the whole row
 * (x - m) - log S into out_full fp32 [rows, V] (pitch out_stride). */
int ix_logprob_rowinv_full(const void* logits, int dtype, long rows, long V, long row_stride, int G,
                           float* out_full, long out_stride, float* out_lse, void* workspace,
                           size_t workspace_bytes, int force_shape, const float* row_max_in, void* stream);

/* rowmax[r] = max_p parts[r*parts_ld + p], p < P (torch.amax of rowinv.py:479 over partials). */
int ix_rowmax_reduce(const float* parts, long parts_ld, long P, long rows, float* rowmax, void* stream);

/* ---- norms: ops/norms/fused_outnorm.py, zero_centered_norm.py, fused_add_rmsnorm.py -------- */

/* fused_rms_norm_gamma (fused_outnorm.py:159-185) / ZeroCenteredTorchRMSNorm.forward
 * (zero_centered_norm.py:36-37). x, out bf16 [M, N]; weight bf16 [N]; zero_centered != 0 uses
 * gamma = bf16(1 + weight), else gamma = weight. */
int ix_rmsnorm_gamma(const void* x, const void* weight, void* out, long M, long N, float eps,
                     int zero_centered, void* stream);

/* fused_gated_out_norm (fused_outnorm.py:235-271) / _eager_apply_gated_norm
 * (runtimes/megatron/gdn_fla_shim.py:390-425). x, out bf16 [T*HV, N]; gate bf16 viewed
 * [T, HV, N] with token pitch gate_stride_t. */
int ix_gated_out_norm(const void* x, const void* gate, long gate_stride_t, const void* weight, void* out,
                      long T, long HV, long N, float eps, int zero_centered, void* stream);

/* residual add + norm (fused_add_rmsnorm.py:1-25): h = bf16(x + residual) -> h_out, then the
 * norm chain of ix_rmsnorm_gamma on h -> out. */
int ix_add_rmsnorm_gamma(const void* x, const void* residual, const void* weight, void* out, void* h_out,
                         long M, long N, float eps, int zero_centered, void* stream);

/* The tail of a mixture layer in one launch: _fixed_order_combine (moe_batch_invariant.py:276-320, kernel
 * moe_combine_kernel.py:36-76) followed by the residual add + norm (fused_add_rmsnorm.py:1-25). expert_out bf16
 * [rows, N], combine_rows int32 [T, k] (a token's rows in ascending expert order), fp32_acc as in ix_moe_combine;
 * h_out [T, N] = bf16(combine + residual), out [T, N] = the norm chain of ix_rmsnorm_gamma on h_out. Bit for bit
 * ix_moe_combine then ix_add_rmsnorm_gamma, without the [T, N] round trip of the combine's output. Serves N in
 * {512, 1024, 2048, 4096} with k in {2, 4, 8} as instantiated, 16-byte aligned operands; else declined. */
int ix_moe_combine_add_rmsnorm(const void* expert_out, const int* combine_rows, long k, int fp32_acc, const void* residual,
                               const void* weight, void* out, void* h_out, long T, long N, float eps, int zero_centered,
                               void* stream);

/* ---- dense matmuls: ops/moe/moe_batch_invariant.py:422-473 (aten mm/addmm/bmm override),
 *      ops/mm/mm_tiles.py:127-158, ops/mm/csrc/cublaslt_pinned.cpp:319-327 mm(x, w, out, slot) - */

/* C[M,N] = A[M,K] . W[N,K]^T (+ bias[N]), bf16 operands, fp32 accumulate in a fixed K order, no
 * split-K. C is bf16 (one round of the accumulator) or, with c_dtype = IX_DT_F32, the fp32
 * accumulator itself (the router's fp32 gating product when its fp32 weight is bf16-exact).
 * lda/ldw/ldc are row pitches in elements. bias (bf16 [N]) may be NULL. tile: 0 auto; 1..6 name a tile shape
 * (32x256, 128x128, 256x256 on eight waves, 256x256 on four waves, 128x256, 64x32); 4 takes the streaming form of its
 * tile (one workgroup per CU walks many tiles) when the product has at least 512 tiles and the form serves it (bf16 C,
 * no bias, K a multiple of 64 and >= 704, N and ldc multiples of 8, C 16-byte aligned), 7 never does, 8 always does
 * and declines what the form does not serve. Every choice gives the same bits.
 * row_max_parts: NULL, or fp32 [M, parts_ld] receiving per part the max of the stored values (one part per column
 * tile; two for tiles 4, 7, 8), parts_ld >= ix_gemm_bf16_n_tiles(M, N, K, tile). */
int ix_gemm_bf16_nt(const void* A, long lda, const void* W, long ldw, const void* bias, void* C, int c_dtype,
                    long ldc, long M, long N, long K, int tile, float* row_max_parts, long parts_ld,
                    void* stream);
long ix_gemm_bf16_n_tiles(long M, long N, long K, int tile);

/* aten::bmm of the same override (moe_batch_invariant.py:453-464): `batch` independent products A_b [M,K] . W_b [N,K]^T
 * -> C_b [M,N] (bf16) in ONE launch, each computed exactly as ix_gemm_bf16_nt computes it (same bits). Matrix b of an
 * operand starts b * stride elements after matrix 0 (stride_w = 0 shares one weight). batch <= 65535. */
int ix_gemm_bf16_nt_batched(const void* A, long lda, long stride_a, const void* W, long ldw, long stride_w, void* C,
                            long ldc, long stride_c, long batch, long M, long N, long K, int tile, void* stream);

/* The same product for M <= 64 (the M in {1, 7, 64} cases of the override, mm_tiles.py:232-326, where the product is the
 * time memory needs to deliver W once): W is read from a fragment-packed copy made once per weight version, streamed
 * through registers; the activations are staged in LDS per workgroup. Same bits as ix_gemm_bf16_nt (same matrix
 * instruction, same K order, one accumulator per element, one rounding).
 * ix_gemm_pack_decode: Wf (N * K bf16, 16-byte aligned) <- W [N,K] with row pitch ldw. Serves N a multiple of 32 and
 * K in {1024, 2048, 3072, 4096}; ix_gemm_decode_serves_shape(N, K) says so without touching memory (1 = served).
 * ix_gemm_bf16_nt_decode: C [M,N] bf16 (row pitch ldc, a multiple of 4; C 8-byte aligned) = A [M,K] (row pitch lda, a
 * multiple of 8; A 16-byte aligned) . W^T; no bias, no row maxima, M <= 64: declines (IX_DECLINED) anything else. */
int ix_gemm_decode_serves_shape(long N, long K);
int ix_gemm_pack_decode(const void* W, long ldw, void* Wf, long N, long K, void* stream);
int ix_gemm_bf16_nt_decode(const void* A, long lda, const void* Wf, void* C, long ldc, long M, long N, long K,
                           void* stream);

/* Router gating GEMM (moe/_register.py:59-66): C fp32 [M,N] = A[M,K] . W[N,K]^T with W fp32 and
 * A fp32 or bf16 (a_dtype), fp32 accumulate in a fixed K order. */
int ix_gemm_f32_nt(const void* A, int a_dtype, long lda, const void* W, long ldw, void* C, long ldc, long M,
                   long N, long K, void* stream);

/* ---- Device memory that sleeps: ops/gdn/gdn_cpr_sleep.py --------------------------------------- */

/* An arena is a range of device addresses that keeps its place while the memory behind it is given back and taken again
 * (alloc_cpr_arena / cpr_sleep / cpr_wake_up, gdn_cpr_sleep.py:45-124, 217-282: the engine state of the boundary-form
 * GatedDeltaNet layers is discarded at sleep without a host copy and mapped again at the same address at wake, so captured
 * decode graphs stay valid). Built on the HIP virtual-memory calls; IX_DECLINED where the device does not support them.
 * Set-up calls, not hot-path ones: they allocate, and release synchronises the device.
 * ix_arena_create: `bytes` (rounded up to the allocation granularity) mapped and zeroed on `stream`, for the current
 * device; IX_ERR_SIZE if the memory or the address range is not to be had.
 * ix_arena_release_memory: device synchronised, memory unmapped and released; the addresses stay reserved. Touching the
 * range before ix_arena_restore_memory has returned is a memory fault: the caller keeps tensors and graph replays away.
 * ix_arena_restore_memory: fresh memory mapped at the same addresses and zeroed on `stream`.
 * ix_arena_destroy: releases memory and addresses. Calls on an arena come from one thread at a time. */
int ix_arena_create(size_t bytes, void** arena_out, void* stream);
void* ix_arena_base(const void* arena);
size_t ix_arena_bytes(const void* arena);
int ix_arena_is_mapped(const void* arena);
int ix_arena_release_memory(void* arena);
int ix_arena_restore_memory(void* arena, void* stream);
int ix_arena_destroy(void* arena);

/* ---- GatedDeltaNet: ops/gdn/gdn_ops.py ----------------------------------------------------- */

/* gdn_recurrent_kernel (gdn_ops.py:400-441): the delta-rule scan over packed tokens, state pool
 * advanced in place. q,k [tokens, H, K] and v [tokens, HV, V] with token pitches q_pitch,
 * k_pitch, v_pitch (elements; heads contiguous inside a token, so slices of one projection
 * buffer need no copy); o [tokens, HV, V] contiguous, or NULL for a state-only pass; g fp32 [tokens, HV]; beta [tokens, HV];
 * q/k/v/beta/o share io_dtype. state_pool fp32 [rows, HV, V, K]. cu_seqlens int32
 * [N+1]. state_indices int32: pool row for (sequence n, token t) at [n*stride + t]; column 0
 * loads, a positive entry at column t stores after token t, row index <= 0 at column 0 skips
 * the sequence. stride 0 is the compact form: state_indices [N] holds one row per sequence, loaded
 * before its first token and stored once after its last. HV % H == 0 (GQA: head hv reads q/k
 * head hv / (HV/H)). K in {32,64,128,256}.
 * time_tile: bits 0-7 = tokens staged per LDS fill (<= 64, 0 = default; 1 also tells the launcher that every
 * sequence has one token, a decode step); bits 8.. = the layout: state rows held per group of 16 lanes (1, 2 or 4),
 * or 16 for the lane-pair layout (K = 128, compact state form, V % 128 == 0; declined otherwise); 0 = chosen from the
 * grid size. Neither changes results. */
int ix_gdn_scan(const void* q, const void* k, const void* v, const float* g, const void* beta, void* o,
                int io_dtype, long q_pitch, long k_pitch, long v_pitch, float* state_pool,
                const int* cu_seqlens, const int* state_indices, long state_indices_stride, long N, long H,
                long HV, long K, long V, float scale, int time_tile, void* stream);

/* attention.varlen (ops/attention/_register.py:15-47; varlen_backend.py; megatron_varlen_attn.py): causal
 * grouped-query attention with ONE walk over the keys of each query (the reference's num_splits=1
 * pin), so a query's bits do not depend on the launch it ran in. bf16 only, D = 128.
 * q [Tq, HQ, D] with token pitch q_pitch; k, v [*, HKV, D] with token pitch kv_pitch (elements); o
 * [Tq, HQ, D] contiguous. cu_q int32 [N+1] packs the queries. Sequence n's keys are the tokens
 * kv_start[n] .. kv_start[n] + q_pos0[n] + len_q[n] - 1 of k/v; its first query sits at absolute
 * position q_pos0[n] (NULL: 0 for every sequence; a negative entry marks a null lane whose outputs are
 * zero). max_q_len >= the longest query run. HQ % HKV == 0 and HQ / HKV in {1,2,4,8,16,32}.
 * scale must be positive and finite (the running reference point is kept on the unscaled scores);
 * kv_pitch < 2^26. Returns IX_ERR_ARG / IX_DECLINED otherwise. */
int ix_attn_varlen(const void* q, long q_pitch, const void* k, const void* v, long kv_pitch, void* o,
                   const int* cu_q, const long* kv_start, const int* q_pos0, long N, long max_q_len, long HQ,
                   long HKV, long D, float scale, void* stream);

/* rope.rope (ops/rope/_register.py:17-77; rope_fused.py:66-108): rotate-half rotary embedding over the
 * first R lanes of every head, in place, with the three-round bf16 multiply-add
 * bf16(bf16(x*cos) + bf16(rot*sin)). x [tokens, heads, D] with token pitch x_pitch; cos/sin bf16
 * [table_rows, R]; positions int32 [tokens]. A position outside [0, table_rows) reads nothing and makes that
 * token's rotated lanes NaN (positions live on the device, so the host cannot refuse them without a sync). */
int ix_rope_inplace(void* x, long x_pitch, const void* cos_table, const void* sin_table, long table_rows,
                    const int* positions, long tokens, long heads, long D, long R, void* stream);

/* gdn_l2norm (gdn_ops.py:202-213): y = x * (1/sqrt(sum x^2 + eps)) over rows of K.
 * x [tokens, H, K] with token pitch x_pitch; y [tokens, H, K] contiguous. */
int ix_gdn_l2norm(const void* x, long x_pitch, void* y, int io_dtype, long tokens, long H, long K, float eps,
                  void* stream);

/* gdn_gate_and_beta (gdn_ops.py:1197-1210) in the fp32 form of the fused core (gdn/_register.py:33-55):
 * g = -exp(A_log[hv]) * softplus(a + dt_bias[hv]) fp32; beta = sigmoid(b) in io_dtype.
 * a, b [tokens, HV] with token pitches a_pitch, b_pitch (elements; column slices of a wider projection are read in
 * place); g, beta [tokens, HV] contiguous; A_log, dt_bias fp32 [HV]. exp_dtype = the dtype exp(A_log) is held in:
 * IX_DT_F32 for the fused core's form (parameter widened first, gdn/_register.py:33-55), IX_DT_BF16 for the eager
 * form on a bf16 parameter (gdn_ops.py:1197-1210: "A_log.exp() is taken in the parameter's own dtype"; A_log then
 * holds the widened bf16 values and exp's result is rounded to bf16 before the product). */
int ix_gdn_gate(const void* a, long a_pitch, const void* b, long b_pitch, const float* A_log, const float* dt_bias,
                float* g, void* beta, int io_dtype, long tokens, long HV, int exp_dtype, void* stream);

/* Everything a decode step does in front of the scan, one launch (the engine's decode of gdn_recurrent_state.py:628-869:
 * causal_conv1d_update, the two l2norms and the gating, which the reference's fused core folds into its own kernel,
 * gdn_ops.py:513-558): for each of N sequences (one token each) the width-4 conv of x [N, D] (pitch x_pitch,
 * D = 2 H K + HV V) on the W - 1 inputs stored in conv_pool row rows[n], with that window slid in place; q and k heads
 * (channels < 2 H K) l2-normalised; g = -exp(A_log) * softplus(a + dt_bias) fp32 and beta = sigmoid(b) bf16. y [N, D]
 * bf16 contiguous, g / beta [N, HV]. Bit for bit what ix_gdn_conv + ix_gdn_l2norm + ix_gdn_gate (exp_dtype fp32) give.
 * rows[n] <= 0: zero window read, none written. Serves bf16, W = 4, K = 128, 16-byte aligned operands; else declined. */
int ix_gdn_decode_prep(const void* x, long x_pitch, const void* a, long a_pitch, const void* b, long b_pitch,
                       const void* conv_weight, const void* conv_bias, const float* A_log, const float* dt_bias,
                       void* conv_pool, const int* rows, void* y, float* g, void* beta, long N, long H, long K, long HV,
                       long V, long W, int silu, float eps, void* stream);

/* cpr_resolve_rows (gdn_cpr_rows.py:29-80; eager chain gdn_recurrent_state.py:271-284): engine slot ids of a
 * decode batch -> state-pool rows, one launch, host-free. slots int32 or int64 [n] (slots_i64). With slot2row
 * (int64 [map_n]): row = slot2row[clamp(slot, 0, map_n - 1)]; with slot2row NULL: row = slot if 0 <= slot < blocks
 * else 0. rows64 (may be NULL) and rows32 receive the rows. last_used + clock (both or neither): clock[0] += 1 and
 * last_used[row] = clock[0] for every row of the batch (the decode step's use stamp). */
int ix_gdn_resolve_rows(const void* slots, int slots_i64, long n, const int64_t* slot2row, long map_n, long blocks,
                        int64_t* rows64, int* rows32, int64_t* last_used, int64_t* clock, void* stream);

/* cpr_buffer_scatter (gdn_cpr_scatter.py:24-76; eager form in CprGDN.decode, gdn_cpr_state.py): lane n of a decode
 * step appends its prepared k [H*K] (token pitch k_pitch), v [HV*V] (v_pitch), g fp32 [HV], beta [HV] to the
 * open-chunk buffers k_buf [rows, C, H, K], v_buf [rows, C, HV, V], g_buf fp32 [rows, C, HV], b_buf [rows, C, HV] at
 * (row = rows[n], column = pos[row] % C), then pos[row] += 1 for row > 0 and due[row] = row if the new position is
 * a multiple of C else 0. pos int64 [rows]; due int32 [rows]; a live row appears at most once among rows[0..N). */
int ix_gdn_cpr_scatter(const void* k, long k_pitch, const void* v, long v_pitch, const float* g, const void* beta,
                       const int* rows, int64_t* pos, void* k_buf, void* v_buf, float* g_buf, void* b_buf, int* due,
                       int io_dtype, long N, long H, long K, long HV, long V, long C, void* stream);

/* The hand-off that ends CprGDN._resync (gdn_cpr_state.py:644-646): for every row with due[row] > 0,
 * running_state[row] = widen(round_to(snapshot_dtype, entry_state[row])); then due[] is cleared. Both pools fp32
 * [rows, elems], elems % 4 == 0. */
int ix_gdn_cpr_handoff(const float* entry_state, float* running_state, int* due, long rows, long elems,
                       int snapshot_dtype, void* stream);

/* ix_gdn_scan whose output leaves through the layer's gated output norm in the same launch (the composition of
 * runtimes/megatron/gdn_fla_shim.py:390-425 `_eager_apply_gated_norm` after the core, ops/norms/fused_outnorm.py:189-271):
 * o [tokens, HV, V] bf16 receives ix_gated_out_norm(o_scan, gate, norm_weight) instead of o_scan; the bits of the two
 * calls. gate bf16 with token pitch gate_stride_t (elements, a multiple of 8), norm_weight bf16 [V]. Served where the
 * lane-pair layout of the scan runs: one state row per sequence (state_indices [N]), K = V = 128, bf16, N * HV >= 512, no
 * forced time tile of 1 or row code; IX_DECLINED otherwise, before the state is touched (the caller makes the two calls). */
int ix_gdn_scan_gated_norm(const void* q, const void* k, const void* v, const float* g, const void* beta, void* o,
                           long q_pitch, long k_pitch, long v_pitch, float* state_pool, const int* cu_seqlens,
                           const int* state_indices, long N, long H, long HV, long K, long V, float scale,
                           int time_tile, const void* gate, long gate_stride_t, const void* norm_weight,
                           float norm_eps, int zero_centered, void* stream);

/* gdn_causal_conv / gdn_causal_conv_batched (gdn_ops.py:74-170) over packed tokens, and the
 * engine's window-slide update (gdn_recurrent_state.py:686-707,814-825) when every sequence has
 * one token. x bf16 [tokens, D] with token pitch x_pitch (elements; a slice of a wider projection buffer needs
 * no copy), y bf16 [tokens, D] contiguous; weight bf16 [D, W]; bias bf16 [D] or NULL; conv_pool bf16
 * [rows, D, W-1] oldest first. state_rows_in[n] <= 0 (or NULL) = no history; state_rows_out[n]
 * > 0 stores the last W-1 inputs to that row (may equal the input row). */
int ix_gdn_conv(const void* x, long x_pitch, const void* weight, const void* bias, void* y, void* conv_pool,
                const int* cu_seqlens, const int* state_rows_in, const int* state_rows_out, long N,
                long total_tokens, long D, long W, int silu, void* stream);

/* ix_gdn_conv with gdn_l2norm (gdn_ops.py:173-188) of the q and k heads folded into its epilogue, as the fused core does
 * in front of its scan (gdn_ops.py:513-558): channels [0, qk_channels) of y are heads of K channels and leave normalised
 * with `eps`, the others as ix_gdn_conv leaves them. The bits of ix_gdn_conv followed by ix_gdn_l2norm on those columns.
 * Serves K = 128, W = 4, D and qk_channels multiples of 128, x_pitch a multiple of 8, 16-byte aligned operands; IX_DECLINED
 * otherwise (the caller makes the two calls). */
int ix_gdn_conv_l2norm(const void* x, long x_pitch, const void* weight, const void* bias, void* y, void* conv_pool,
                       const int* cu_seqlens, const int* state_rows_in, const int* state_rows_out, long N,
                       long total_tokens, long D, long W, int silu, long qk_channels, long K, float eps, void* stream);

/* ---- MoE: ops/moe ------------------------------------------------------------------------- */

/* fused_router_dense / ref_router_dense (moe_router_o2_kernel.py:272-311,369-386) with mode 0;
 * mode 1 is softmax over all experts, top-k on the probabilities, renormalise. logits fp32
 * [T, E] (pitch ld). Outputs: topk_idx int32 [T,k] and topk_prob fp32 [T,k] in rank order
 * (score desc, index asc on ties); dense_probs fp32 [T,E] / dense_map uint8 [T,E] optional.
 * k must be a power of two <= 16, E <= 512 (else declined). scaling 0 = none. */
int ix_moe_router_topk(const float* logits, long ld, long T, long E, long k, int mode, float scaling,
                       int* topk_idx, float* topk_prob, float* dense_probs, uint8_t* dense_map, void* stream);

/* Sizing helpers (host arithmetic only). */
long ix_moe_max_tiles(long T, long k, long E, long BM);   /* ceil(T*k/BM) + E */
size_t ix_moe_permute_scratch_ints(long T, long E);
int ix_moe_pick_bm(long T, long k, long E);               /* 32, 128 or 256 */

/* fused_permute_index / ref_permute_index (moe_router_o2_kernel.py:313-351,389-397) plus the
 * block map (moe_fused_experts.py:156-205) and the inverse permutation of
 * moe_combine_rows_kernel.py. Integer work only.
 *   counts int32 [E] tokens per expert; offsets int32 [E+1]; sorted_token int32 [T*k]
 *   (expert-major, token ascending); permuted_prob fp32 [T*k]; combine_rows int32 [T,k] = the
 *   token's rows in ascending expert order; tile_meta int32 [1 + 3*max_tiles] = {n_tiles,
 *   tile_expert[], tile_row0[], tile_nrows[]} for row tiles of BM; scratch int32
 *   [ix_moe_permute_scratch_ints]. */
int ix_moe_permute(const int* topk_idx, const float* topk_prob, long T, long E, long k, long BM, int* counts,
                   int* offsets, int* sorted_token, float* permuted_prob, int* combine_rows, int* tile_meta,
                   long max_tiles, int* scratch, void* stream);

/* fused_router_dense + fused_permute_index back to back (moe_router_o2_kernel.py:272-351) for a batch of at most one
 * token tile (T <= 256, a decode step) and E <= 128: ix_moe_router_topk and ix_moe_permute in ONE launch, the same
 * integers and the same weights in every output (arguments as there; no dense outputs, no scratch). Declined beyond
 * those sizes: the caller then makes the two calls. */
int ix_moe_route_one_tile(const float* logits, long ld, long T, long E, long k, int mode, float scaling, long BM,
                          int* topk_idx, float* topk_prob, int* counts, int* offsets, int* sorted_token,
                          float* permuted_prob, int* combine_rows, int* tile_meta, long max_tiles, void* stream);

/* _block_map / fused_block_map (moe_fused_experts.py:156-205, moe_blockmap_kernel.py): the block map for rows that
 * are ALREADY grouped by expert (SequentialMLP.forward's tokens_per_expert, moe_batched_experts.py:301-330). counts
 * int32 or int64 [E] (counts_i64) in device memory; offsets int32 [E+1] (may be NULL) receives the exclusive scan;
 * tile_meta as in ix_moe_permute, max_tiles >= ix_moe_max_tiles(rows, 1, E, BM). rows = the number of rows the
 * caller's buffers hold: the host cannot see the counts, so the kernel keeps every tile inside [0, rows) -- counts that
 * add up to more lose their tail (offsets[E] = min(rows, sum)); counts that add up to less leave the last rows in no
 * tile. Integer work only, one launch, nothing read back by the host. */
int ix_moe_block_map(const void* counts, int counts_i64, long E, long BM, long rows, int* offsets, int* tile_meta,
                     long max_tiles, void* stream);

/* ix_moe_permute for callers that cannot allocate device memory or bring a workspace: code under HIP graph
 * capture, tight serving loops, harnesses that forbid allocation. No counterpart in the reference (its permutation
 * allocates its tables with torch on every call). Same arguments, same kernels and same integers as ix_moe_permute,
 * minus `scratch`: the two internal tables live in a 1 MiB file-scope device array that each GPU holds until the
 * process ends. The call allocates and frees nothing. Limit: ix_moe_permute_scratch_ints(T, E) <=
 * ix_moe_permute_static_max_ints() (262,144 ints: 262,144 tokens at E = 128), else IX_ERR_SIZE and nothing is
 * launched. All calls on one GPU share the array: calls that overlap on one GPU (two streams, two threads) race;
 * calls in stream order do not, and no call depends on what an earlier one left in the array. The first call on a
 * device looks the array's address up in the runtime (no allocation, but a runtime call): ix_moe_permute_static_init()
 * does that lookup for the current device ahead of time, for callers that then enter a stream capture. */
size_t ix_moe_permute_static_max_ints(void);
int ix_moe_permute_static_init(void);
int ix_moe_permute_static(const int* topk_idx, const float* topk_prob, long T, long E, long k, long BM, int* counts,
                          int* offsets, int* sorted_token, float* permuted_prob, int* combine_rows, int* tile_meta,
                          long max_tiles, void* stream);

/* _batched_experts_forward / _fused_forward (moe_batched_experts.py:301-531,
 * moe_fused_experts.py:292-503): grouped fc1 + SwiGLU + prob epilogue, then grouped fc2.
 * x bf16 [T, Hd] (pitch ldx) gathered through sorted_token; W1 bf16 [E, 2F, Hd] (gate rows
 * then up rows); W2 bf16 [E, Hd, F]; inter bf16 [rows, F]; expert_out bf16 [rows, Hd];
 * rows = T*k = the length of sorted_token and permuted_prob (the kernels clamp their reads of both to rows - 1, so it
 * must not exceed what the arrays hold). BM must be the value given to ix_moe_permute. With 256-row tiles and at
 * least 512 tiles of work both GEMMs run as streaming kernels (one workgroup per CU walking many tiles); same bits. */
int ix_moe_experts(const void* x, long ldx, const int* sorted_token, const float* permuted_prob,
                   const void* W1, const void* W2, const int* tile_meta, long max_tiles, long BM, void* inter,
                   void* expert_out, long T, long rows, long Hd, long F, void* stream);

/* The same product with the weight-tile width chosen by the caller: BN = 256 (what ix_moe_experts uses), or
 * BN = 128 with BM = 128 (square 128 x 128 tiles, two workgroups per CU). The tile shape decides which
 * workgroup computes an element, never how: results are bit-identical for every (BM, BN). The reference's
 * counterpart is the BLOCK_M / BLOCK_N choice of its fused expert kernel (moe_fused_experts.py:292-503). */
int ix_moe_experts_tile(const void* x, long ldx, const int* sorted_token, const float* permuted_prob,
                        const void* W1, const void* W2, const int* tile_meta, long max_tiles, long BM, long BN,
                        void* inter, void* expert_out, long T, long rows, long Hd, long F, void* stream);

/* Fragment-packed copies of the experts' two matrices, and the grouped GEMMs of a decode step reading them. No
 * counterpart in the reference (its engine reads the checkpoint layout through vLLM's fused-MoE kernel,
 * moe_fused_experts.py:292-503); the arithmetic is ix_moe_experts' at BM = 32, bit for bit -- only where the weight
 * bytes are fetched from, and through what, differs. A decode step is bound by streaming every touched expert's weights
 * once. Staged in LDS a CU never has more than ~100 KiB of them in flight, and read in place a k-tile of a weight tile is
 * 128 bytes out of each of 256 rows K * 2 bytes apart (a 4 KiB stride for K = 2048: about 4.6 TB/s on this memory system,
 * against 6.3 TB/s for the same bytes laid out contiguously). Packed, every load instruction of the decode kernels is
 * 1 KiB of contiguous memory, taken straight into the registers the matrix instruction reads, four k-tiles ahead.
 * W1f / W2f have the sizes of W1 [E, 2F, Hd] / W2 [E, Hd, F]; 16-byte chunk layouts (chunk = W[row][64 kt + 32 (lane / 32)
 * + 8 s .. + 7], r = lane % 32):
 *   W1f [E][F / 128][wave 4][Hd / 64][b 2][s 4][lane 64]   row = b F + 128 nt + 32 wave + r   (b: gate, up)
 *   W2f [E][Hd / 256][wave 4][F / 64][b 2][s 4][lane 64]   row = 256 nt + 64 wave + 32 b + r
 * Serves Hd % 256 == 0, F % 128 == 0 with Hd / 64 and F / 64 in {8, 12, 16, 24, 32, 48, 64}; else declined. Pack once per
 * weight version (one pass over each matrix), not per step. ix_moe_experts_decode takes a block map of BM = 32. */
int ix_moe_pack_decode(const void* W1, const void* W2, void* W1f, void* W2f, long E, long Hd, long F, void* stream);
int ix_moe_experts_decode(const void* x, long ldx, const int* sorted_token, const float* permuted_prob, const void* W1f,
                          const void* W2f, const int* tile_meta, long max_tiles, void* inter, void* expert_out, long T,
                          long rows, long Hd, long F, void* stream);

/* _fixed_order_combine / _combine_topk_kernel (moe_batch_invariant.py:276-320,
 * moe_combine_kernel.py:36-76): out bf16 [T, Hd] = the token's k rows of expert_out summed in
 * ascending expert order; fp32_acc 0 = bf16 adds (a round per add), 1 = fp32 sum, one round. */
int ix_moe_combine(const void* expert_out, const int* combine_rows, void* out, long T, long Hd, long k,
                   int fp32_acc, void* stream);

/* The eager unpermute with routing weights and any of its dtypes (_deterministic_unpermute,
 * moe_batch_invariant.py:338-385: `permuted_tokens * permuted_probs.unsqueeze(-1)` then _fixed_order_combine, :276-320):
 * out[t] = the left-to-right sum over the token's k rows of expert_out[row] * row_weight[row] (row_weight NULL: no
 * product). expert_out [rows, Hd] in in_dtype; row_weight fp32 values [rows]; arith_dtype = torch's promotion of the
 * token and weight dtypes (IX_DT_BF16: the product and every partial sum are rounded to bf16; IX_DT_F32: nothing is
 * rounded before the store); out [T, Hd] in out_dtype (one round when it is narrower). */
int ix_moe_combine_weighted(const void* expert_out, int in_dtype, const float* row_weight, int arith_dtype,
                            const int* combine_rows, void* out, int out_dtype, long T, long Hd, long k, void* stream);

/* ---- order-invariant digests: debug/thash ------------------------------------------------- */

#define IX_DIGEST_MAX_MASKS 8

/* The weighted modular sums behind tensor_digest / digest_ladder (thash.py:180-217,251-301; the kernel
 * thash_kernels.py:49-90): out[j] = SUM_i (sext(x_i) & masks[j]) * w(i) mod 2^64 for j < nmask <= 8, with
 * w(i) = (mix64((i >> 3) ^ salt) ^ ((i & 7) * 0x9E3779B97F4A7C15)) | 1 and mix64 the splitmix64 finaliser.
 * x = n integers of elem_bytes (1, 2, 4 or 8) each, read as signed; masks = nmask values in HOST memory, read
 * during the call; out = nmask words in device memory; workspace = device words, at least
 * ix_digest_workspace_words(1, n, nmask) of them (may be NULL when that is 0). All nmask sums come from one
 * pass over x. n = 0 gives zeros. */
int ix_digest_sums(const void* x, int elem_bytes, long n, uint64_t salt, const uint64_t* masks, int nmask,
                   uint64_t* workspace, size_t workspace_words, uint64_t* out, void* stream);

/* The per-segment sums behind segment_digests (thash.py:319-354; thash_kernels.py:93-104): x is cut into nseg
 * runs of seg_numel elements (the last may be short; nseg = ceil(n / seg_numel)); out[s] is the sum above over
 * run s alone, positions counted from the run's start, with
 * salt_s = mix64(seed ^ mix64(s * seg_numel + 1)) ^ 0x9E3779B97F4A7C15. One launch covers every segment.
 * workspace as above with ix_digest_workspace_words(nseg, seg_numel, 1). */
int ix_digest_segment_sums(const void* x, int elem_bytes, long n, long nseg, long seg_numel, uint64_t seed,
                           uint64_t mask, uint64_t* workspace, size_t workspace_words, uint64_t* out,
                           void* stream);

/* Host arithmetic only: device words of workspace the two calls above need (0 = none). */
size_t ix_digest_workspace_words(long nseg, long seg_numel, int nmask);

#ifdef __cplusplus
}
#endif
#endif /* ISOEXEC_HIP_H */
