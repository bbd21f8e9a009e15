"""Benchmark of the batch-invariant token-logprob hot path on one MI355X.

Default workload (``dense_head``, BASELINE.json configs[1]): M = 4096 hidden states of width 4096
-> zero-centred RMSNorm -> bf16 LM-head GEMM against [151936, 4096] -> bf16 logits -> row-invariant
log-softmax + target gather. One step = one pass over the 4096 tokens; inputs are resident in HBM
before the timed region. Prints ONE JSON line.

Other workloads (``--workload gdn_decode | moe | hybrid | attention | digest``) time configs[2], configs[3] and configs[4] with
the same contract; they are extra lines for profiling, not the headline.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "skyrl-isoexec_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

PEAK_MFMA_BF16_TFLOPS = 2500.0  # MI355X dense bf16
PEAK_HBM_GBS = 8000.0
# HBM-side bytes per launch of the dominant kernels, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE scaled by
# what the same counters read for a 1 GiB copy (x2.0 / x1.0); see profiles/*.txt. Workload-specific.
MEASURED_TRAFFIC_BYTES = {"dense_head_M4096_gemm": 9.08e9, "gdn_decode_B256": 1.1016e9,
                          "moe_T16384_grouped_gemms": 3.80e9}


class KernelTimer:
    """HIP-event timing of one kernel family on torch's current stream (the stream every entry
    point of the library is launched on)."""

    def __init__(self):
        self.pairs = []

    def __call__(self, fn):
        import torch

        s = torch.cuda.Event(enable_timing=True)
        e = torch.cuda.Event(enable_timing=True)
        s.record()
        out = fn()
        e.record()
        self.pairs.append((s, e))
        return out

    def mean_ms(self):
        return sum(s.elapsed_time(e) for s, e in self.pairs) / max(1, len(self.pairs))


def dense_head(args):
    import torch

    from isoexec_amd.ops.logprobs.rowinv import sampled_forward
    from isoexec_amd.ops.mm.mm_hip import linear_nt
    from isoexec_amd.ops.norms.fused_outnorm import fused_rms_norm_gamma

    dev = "cuda:0"
    M, K, V = args.tokens, 4096, 151936
    gen = torch.Generator(device=dev)
    gen.manual_seed(1)
    h = torch.randn(M, K, device=dev, generator=gen).to(torch.bfloat16)
    w_norm = (0.02 * torch.randn(K, device=dev, generator=gen)).to(torch.bfloat16)  # gamma = 1 + w
    w_lm = torch.empty(V, K, device=dev, dtype=torch.bfloat16)
    for s in range(0, V, 16384):  # chunked so the fp32 temporary stays small
        e = min(V, s + 16384)
        w_lm[s:e] = (0.02 * torch.randn(e - s, K, device=dev, generator=gen)).to(torch.bfloat16)
    target = torch.randint(0, V, (M,), device=dev, generator=gen)

    t_gemm, t_lp, t_norm = KernelTimer(), KernelTimer(), KernelTimer()

    def step(timed):
        wrap = (lambda t, f: t(f)) if timed else (lambda t, f: f())
        x = wrap(t_norm, lambda: fused_rms_norm_gamma(h, w_norm, 1e-6))
        logits, row_max = wrap(t_gemm, lambda: linear_nt(x, w_lm, tile=args.tile, want_row_max=True))
        lp, _ = wrap(t_lp, lambda: sampled_forward(logits, target, 8, row_max=row_max))
        return lp

    for _ in range(args.warmup):
        step(False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        lp = step(True)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert bool(torch.isfinite(lp).all())

    gemm_ms = t_gemm.mean_ms()
    flops = 2.0 * M * V * K
    achieved = flops / (gemm_ms * 1e-3) / 1e12
    lp_ms = t_lp.mean_ms()
    out = {
        "metric": "trainer-fwd & decode tokens/s at bitwise parity; % of HBM/MFMA roofline",
        "value": M * args.steps / dt,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": dt / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "dense_head: RMSNorm(4096) + LM head [151936,4096] + log-softmax/gather",
                   "tokens_per_step": M, "hidden": K, "vocab": V, "gemm_tile": args.tile},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_MFMA_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_MFMA_BF16_TFLOPS,
                     "traffic": MEASURED_TRAFFIC_BYTES["dense_head_M4096_gemm"] if M == 4096 else None,
                     "kernel": "k_gemm_bf16_nt (+ 7 us row-max reduce)", "kernel_ms": gemm_ms},
        "kernels_ms": {"rmsnorm": t_norm.mean_ms(), "gemm": gemm_ms, "logprob": lp_ms},
        "logprob_hbm": {"bound": "hbm", "achieved": M * V * 2 / (lp_ms * 1e-3) / 1e9, "peak": PEAK_HBM_GBS,
                        "unit": "GB/s", "frac": M * V * 2 / (lp_ms * 1e-3) / 1e9 / PEAK_HBM_GBS},
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = dense_head_cpu(h, w_norm, w_lm, target, args.cpu_tokens)
    return out


def dense_head_cpu(h, w_norm, w_lm, target, m):
    """The oracle (CPU restatement of the reference's eager path) on the first ``m`` tokens of the
    same workload, timed on this box's host cores."""
    import numpy as np
    import torch

    from oracle import logprobs as o_lp
    from oracle import norms as o_norms
    from oracle.prims import round_bf16

    hn = h[:m].float().cpu().numpy()
    wn = w_norm.float().cpu().numpy()
    wl = w_lm.float().cpu()  # fp32 copy of the LM head (conversion not timed)
    tn = target[:m].cpu().numpy()
    threads = torch.get_num_threads()
    t0 = time.perf_counter()
    x = o_norms.rms_norm_gamma(hn, wn, 1e-6)
    logits = round_bf16((torch.from_numpy(x) @ wl.T).numpy())
    lp, _ = o_lp.rowinv_sampled(logits, tn, 8)
    dt = time.perf_counter() - t0
    assert np.isfinite(lp).all()
    return {"value": m / dt, "unit": "tokens/s", "cores": threads, "kind": "port",
            "sample": f"first {m} tokens of the same dense_head workload ({dt:.1f} s of CPU work; "
                      f"fp32 torch matmul + numpy oracle norm/logprob)"}


def gdn_decode(args):
    import torch

    from isoexec_amd.ops.gdn.gdn_ops import gdn_recurrent_kernel

    dev = "cuda:0"
    B, H, HV, K, V = args.batch, 16, 32, 128, 128
    q = torch.randn(B, 1, H, K, device=dev).to(torch.bfloat16)
    k = torch.randn(B, 1, H, K, device=dev).to(torch.bfloat16)
    q = q / q.float().norm(dim=-1, keepdim=True).to(torch.bfloat16)
    k = k / k.float().norm(dim=-1, keepdim=True).to(torch.bfloat16)
    v = torch.randn(B, 1, HV, V, device=dev).to(torch.bfloat16)
    g = -torch.nn.functional.softplus(torch.randn(B, 1, HV, device=dev))
    beta = torch.sigmoid(torch.randn(B, 1, HV, device=dev)).to(torch.bfloat16)
    pool = torch.zeros(B + 1, HV, V, K, device=dev)
    rows = torch.arange(1, B + 1, dtype=torch.int32, device=dev)
    timer = KernelTimer()
    fn = lambda: gdn_recurrent_kernel(q, k, v, g, beta, ssm_state=pool, state_indices=rows)
    for _ in range(args.warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        timer(fn)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms = timer.mean_ms()
    by = B * HV * V * K * 4 * 2
    return {"metric": "gdn decode tokens/s", "value": B * args.steps / dt, "unit": "tokens/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt / args.steps * 1e3,
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": f"gdn_decode B={B} HV=32 K=V=128 (state R+W 4 MiB/seq/step)"},
            "roofline": {"bound": "hbm", "achieved": by / (ms * 1e-3) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": by / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
                         "traffic": MEASURED_TRAFFIC_BYTES["gdn_decode_B256"] if B == 256 else None,
                         "kernel": "k_gdn_scan",
                         "kernel_ms": ms}}


def moe(args):
    import torch

    from isoexec_amd.ops.mm.mm_hip import router_gemm
    from isoexec_amd.ops.moe.moe_hip import experts_forward, moe_ffn_forward, permute, router_topk

    dev = "cuda:0"
    T, H, E, F, k = args.tokens, 2048, 128, 768, 8
    x = torch.randn(T, H, device=dev).to(torch.bfloat16)
    wr = (0.02 * torch.randn(E, H, device=dev)).to(torch.bfloat16)
    w1 = (0.02 * torch.randn(E, 2 * F, H, device=dev)).to(torch.bfloat16)
    w2 = (0.02 * torch.randn(E, H, F, device=dev)).to(torch.bfloat16)
    fn = lambda: moe_ffn_forward(x, wr, w1, w2, k, pre_softmax=True)
    timer = KernelTimer()
    for _ in range(args.warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        timer(fn)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms = timer.mean_ms()
    fl = T * 75.5e6
    # the dominant kernels alone: the two grouped GEMMs (fc1 + SwiGLU, fc2) over a fixed routing
    idx, prob, _, _ = router_topk(router_gemm(x, wr), k, pre_softmax=True)
    perm = permute(idx, prob, E)
    t_exp = KernelTimer()
    for _ in range(2):
        experts_forward(x, w1, w2, perm)
    for _ in range(args.steps):
        t_exp(lambda: experts_forward(x, w1, w2, perm))
    torch.cuda.synchronize()
    exp_ms = t_exp.mean_ms()
    exp_fl = 2.0 * T * k * H * (2 * F) + 2.0 * T * k * F * H
    return {"metric": "moe ffn tokens/s", "value": T * args.steps / dt, "unit": "tokens/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt / args.steps * 1e3,
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": f"moe T={T} hidden 2048, 128 experts top-8, inter 768"},
            "roofline": {"bound": "mfma", "achieved": exp_fl / (exp_ms * 1e-3) / 1e12, "peak": PEAK_MFMA_BF16_TFLOPS,
                         "unit": "TFLOP/s", "frac": exp_fl / (exp_ms * 1e-3) / 1e12 / PEAK_MFMA_BF16_TFLOPS,
                         "traffic": MEASURED_TRAFFIC_BYTES["moe_T16384_grouped_gemms"] if T == 16384 else None,
                         "kernel": "k_moe_fc1_glu + k_moe_fc2 (grouped GEMMs)", "kernel_ms": exp_ms},
            "whole_ffn": {"kernel_ms": ms, "achieved": fl / (ms * 1e-3) / 1e12, "unit": "TFLOP/s",
                          "frac": fl / (ms * 1e-3) / 1e12 / PEAK_MFMA_BF16_TFLOPS,
                          "kernels": "router product + router + permutation + grouped GEMMs + combine"}}


def attention(args):
    """Causal grouped-query attention, config 4 layout: ``--seqs`` sequences of prompt + response tokens packed
    (prefill shape), then one decode step for the same sequences out of a key/value cache."""
    import torch

    from isoexec_amd.ops.attention.varlen_attn import KVCache, varlen_attention

    dev = "cuda:0"
    n, L, HQ, HKV, D = args.seqs, args.prompt + args.response, 32, 4, 128
    q = torch.randn(n * L, HQ, D, device=dev).to(torch.bfloat16)
    k = torch.randn(n * L, HKV, D, device=dev).to(torch.bfloat16)
    v = torch.randn(n * L, HKV, D, device=dev).to(torch.bfloat16)
    cu = torch.arange(0, (n + 1) * L, L, dtype=torch.int32, device=dev)
    fn = lambda: varlen_attention(q, k, v, cu, L)
    timer = KernelTimer()
    for _ in range(args.warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        timer(fn)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    ms = timer.mean_ms()
    fl = n * 4.0 * (L * (L + 1) / 2) * HQ * D  # QK^T and PV over the causal half
    # decode: one query per sequence against L cached keys
    cache = KVCache(n, L, HKV, D, device=dev)
    cache.k[1:].copy_(k.view(n, L, HKV, D))
    cache.v[1:].copy_(v.view(n, L, HKV, D))
    kf, vf = cache.flat()
    qd = q.view(n, L, HQ, D)[:, -1].contiguous()
    cud = torch.arange(n + 1, dtype=torch.int32, device=dev)
    kv_start = torch.arange(1, n + 1, dtype=torch.int64, device=dev) * L
    pos0 = torch.full((n,), L - 1, dtype=torch.int32, device=dev)
    dec = lambda: varlen_attention(qd, kf, vf, cud, 1, kv_start=kv_start, q_pos0=pos0)
    tdec = KernelTimer()
    for _ in range(3):
        dec()
    for _ in range(20):
        tdec(dec)
    torch.cuda.synchronize()
    dms = tdec.mean_ms()
    dbytes = n * L * HKV * D * 2 * 2
    return {"metric": "attention prefill tokens/s", "value": n * L / dt, "unit": "tokens/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt * 1e3, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": f"attention: {n} x {L} tokens, 32 query / 4 kv heads, d 128, causal, one key walk"},
            "roofline": {"bound": "mfma", "achieved": fl / (ms * 1e-3) / 1e12, "peak": PEAK_MFMA_BF16_TFLOPS,
                         "unit": "TFLOP/s", "frac": fl / (ms * 1e-3) / 1e12 / PEAK_MFMA_BF16_TFLOPS, "traffic": None,
                         "kernel": "k_attn_varlen<8>", "kernel_ms": ms},
            "decode": {"bound": "hbm", "kernel_ms": dms, "achieved": dbytes / (dms * 1e-3) / 1e9, "peak": PEAK_HBM_GBS,
                       "unit": "GB/s", "frac": dbytes / (dms * 1e-3) / 1e9 / PEAK_HBM_GBS, "batch": n, "context": L}}


def hybrid(args):
    """BASELINE.json configs[4]: the 8-layer hybrid model. One step = one trainer scoring pass over
    ``--seqs`` sequences of prompt + response tokens; the rollout's prefill and decode are timed beside it."""
    import torch

    from isoexec_amd.runtimes.hybrid import HybridConfig, HybridWeights, RolloutEngine, TrainerModel

    dev = "cuda:0"
    cfg = HybridConfig()
    n, prompt, resp = args.seqs, args.prompt, args.response
    w = HybridWeights.make(cfg, seed=0, device=dev)
    g = torch.Generator(device=dev)
    g.manual_seed(1)
    tokens = torch.randint(0, cfg.vocab, (n * (prompt + resp),), device=dev, generator=g)
    lens, plens = [prompt + resp] * n, [prompt] * n
    trainer = TrainerModel(cfg, w)
    fn = lambda: trainer.response_logprobs(tokens, lens, plens)
    for _ in range(args.warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        fn()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    # rollout: prefill once, then timed decode steps at batch n
    engine = RolloutEngine(cfg, w, max_num_seqs=n, max_len=prompt + resp)
    slots = list(range(n))
    prompts = tokens.view(n, -1)[:, :prompt].reshape(-1)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    x = engine.prefill(slots, prompts, plens)
    torch.cuda.synchronize()
    t_prefill = time.perf_counter() - t0
    dec_steps = min(resp - 1, 64)
    nxt = tokens.view(n, -1)[:, prompt:prompt + dec_steps]
    from isoexec_amd.ops.logprobs.rowinv import full_forward, leaves
    for sidx in range(4):
        x = engine.decode(slots, nxt[:, sidx].contiguous())
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for sidx in range(4, dec_steps):
        x = engine.decode(slots, nxt[:, sidx].contiguous())
        full_forward(engine.blocks.logits(x), leaves())
    torch.cuda.synchronize()
    t_dec = (time.perf_counter() - t0) / (dec_steps - 4)
    # the same steps replayed from a captured graph
    graph = engine.capture_decode(slots)
    more = tokens.view(n, -1)[:, prompt + dec_steps:prompt + dec_steps + 40]
    for sidx in range(4):
        graph.step(more[:, sidx].contiguous())
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for sidx in range(4, 40):
        x = graph.step(more[:, sidx].contiguous())
        full_forward(engine.blocks.logits(x), leaves())
    torch.cuda.synchronize()
    t_graph = (time.perf_counter() - t0) / 36
    total = n * (prompt + resp)
    # dense-equivalent flops per token: projections + experts (top-8) + router, and the LM head on scored rows
    per_tok = 0
    for i in range(cfg.layers):
        if cfg.is_attention(i):
            per_tok += 2 * cfg.hidden * ((cfg.q_heads + 2 * cfg.kv_heads) * cfg.head_dim + cfg.q_heads * cfg.head_dim)
        else:
            per_tok += 2 * cfg.hidden * (cfg.gdn_qkv + cfg.gdn_z + 2 * cfg.gdn_v_heads + cfg.gdn_z)
        per_tok += 75.5e6
    fl = total * per_tok + n * resp * 2 * cfg.hidden * cfg.vocab
    return {"metric": "trainer-fwd tokens/s at bitwise parity (hybrid model)", "value": total / dt, "unit": "tokens/s",
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt * 1e3, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": f"hybrid: 8 layers (3 GDN : 1 attention) + MoE, vocab 151936; {n} x ({prompt} + {resp}) tokens"},
            "roofline": {"bound": "mfma", "achieved": fl / dt / 1e12, "peak": PEAK_MFMA_BF16_TFLOPS, "unit": "TFLOP/s",
                         "frac": fl / dt / 1e12 / PEAK_MFMA_BF16_TFLOPS, "traffic": None,
                         "kernel": "whole trainer pass (GEMM flops only; scans, attention and norms not counted)"},
            "rollout": {"prefill_tokens_per_s": n * prompt / t_prefill, "decode_ms_per_step": t_dec * 1e3,
                        "decode_tokens_per_s": n / t_dec, "graph_decode_ms_per_step": t_graph * 1e3,
                        "graph_decode_tokens_per_s": n / t_graph, "batch": n}}


def digest(args):
    """Order-invariant digest of a [tokens, 151936] bf16 logits matrix: the full-precision digest (one mask) and the
    five-mask ladder, each one pass over the tensor. The kernel is timed with events through the C ABI; ``value``
    is whole calls of tensor_digest, host read-back included."""
    import ctypes

    import torch

    from isoexec_amd._lib import check, current_stream, lib
    from isoexec_amd.debug import thash

    dev = "cuda:0"
    rows, vocab = args.tokens, 151936
    x = torch.empty(rows, vocab, dtype=torch.bfloat16, device=dev).normal_()
    n, nbytes = x.numel(), x.numel() * 2
    handle = lib()
    out = torch.empty(8, dtype=torch.int64, device=dev)
    timers = {}
    for label, masks in (("one mask", [0xFFFF]), ("ladder of 5", [0xFFFF, 0xFFFE, 0xFFF8, 0xFFE0, 0xFF80])):
        need = handle.ix_digest_workspace_words(1, n, len(masks))
        work = torch.empty(max(1, need), dtype=torch.int64, device=dev)
        arr = (ctypes.c_uint64 * 8)(*masks)
        call = lambda: check(handle.ix_digest_sums(x.data_ptr(), 2, n, 0x1234, arr, len(masks), work.data_ptr(), need,
                                                   out.data_ptr(), current_stream(x.device)), "ix_digest_sums")
        timers[label] = KernelTimer()
        for _ in range(args.warmup):
            call()
        for _ in range(args.steps):
            timers[label](call)
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        thash.tensor_digest(x)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        thash.tensor_digest(x)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms = timers["one mask"].mean_ms()
    res = {"metric": "digest GB/s", "value": nbytes * args.steps / dt / 1e9, "unit": "GB/s", "n_gpus": 1,
           "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt / args.steps * 1e3, "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "u64", "data": "synthetic",
           "config": {"workload": f"digest: [{rows}, {vocab}] bf16 ({nbytes / 1e9:.2f} GB), tensor_digest per step"},
           "roofline": {"bound": "hbm", "achieved": nbytes / (ms * 1e-3) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                        "frac": nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, "traffic": None,
                        "kernel": "k_digest_partial<2,1> + k_digest_finish", "kernel_ms": ms,
                        "ladder_of_5_ms": timers["ladder of 5"].mean_ms()}}
    if not args.no_cpu_baseline:
        from oracle import thash as OT

        sample_rows = max(1, min(rows, 4096))          # about 10 s of numpy work
        iv = x[:sample_rows].cpu().view(torch.int16).numpy()
        t0 = time.perf_counter()
        OT.tensor_digest(iv, "bfloat16", (sample_rows, vocab))
        cpu = time.perf_counter() - t0
        res["cpu_baseline"] = {"value": sample_rows * vocab * 2 / cpu / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": f"first {sample_rows} rows of the same matrix ({cpu:.1f} s of CPU work; "
                                         "numpy restatement of the digest)"}
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="dense_head", choices=["dense_head", "gdn_decode", "moe", "hybrid", "attention", "digest"])
    ap.add_argument("--seqs", type=int, default=64)
    ap.add_argument("--prompt", type=int, default=2048)
    ap.add_argument("--response", type=int, default=512)
    ap.add_argument("--tokens", type=int, default=None)
    ap.add_argument("--batch", type=int, default=256)
    ap.add_argument("--tile", type=int, default=0)
    ap.add_argument("--cpu-tokens", type=int, default=2048)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (no collectives, no sharding); --gpus must be 1", file=sys.stderr)
        sys.exit(2)
    if args.tokens is None:
        args.tokens = 4096
    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(3)
    out = {"dense_head": dense_head, "gdn_decode": gdn_decode, "moe": moe, "hybrid": hybrid, "attention": attention, "digest": digest}[args.workload](args)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
