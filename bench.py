"""Benchmark of the batch-invariant token-logprob hot path on one MI355X.

Default workload (``hybrid``, BASELINE.json configs[4], the configuration the metric is quoted on): the 8-layer
GatedDeltaNet / attention / mixture-of-experts model, 64 sequences of 2048 prompt + 512 response tokens. One step =
one trainer scoring pass over all 64 x 2560 tokens (``value`` = trainer-forward tokens/s); the rollout's decode at
batch 64 is timed in the same run (``decode_tokens_per_s``). ``roofline`` is the dominant kernel of the pass (the two
grouped expert GEMMs), timed with events around its launches inside the timed steps; ``kernels`` holds the other
kernels the target names, each timed in this run at its own configuration; ``cpu_baseline`` is the CPU oracle
composition of the same model on a stated slice. Weights and inputs come from a host generator (seeded), so they do
not depend on the GPU. Prints ONE JSON line.

Other workloads (``--workload dense_head | gdn_decode | moe | attention | digest | decode | gemm``) time configs[1], [2], [3]
and parts of [4] alone with the same contract; they are for profiling one kernel family, not the headline.
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
# HBM-side bytes per launch of the dominant kernels, NOT measured in this run: from rocprofv3 --pmc FETCH_SIZE /
# WRITE_SIZE of the same workload (scaled by what the same counters read for a 1 GiB copy, x2.0 / x1.0), recorded in
# the named file under profiles/.
MEASURED_TRAFFIC_BYTES = {"dense_head_M4096_gemm": 15.5e9, "gdn_decode_B256": 1.080e9,
                          "moe_T16384_grouped_gemms": 3.61e9, "moe_T163840_grouped_gemms": 32.3e9}
TRAFFIC_SOURCE = {"dense_head_M4096_gemm": "profiles/gemm_bf16_nt__dense_head_M4096.txt",
                  "gdn_decode_B256": "profiles/gdn_scan__decode_B256.txt",
                  "moe_T16384_grouped_gemms": "profiles/moe_ffn__T16384.txt",
                  "moe_T163840_grouped_gemms": "profiles/hybrid_trainer_pass__64x2560.txt"}


def host_gen(seed: int):
    import torch

    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def hrandn(shape, g, dev, std=1.0, dtype=None):
    """N(0, std) drawn on the host from ``g`` (64 M values at a time), cast to ``dtype`` (bf16) on the device."""
    import torch

    dtype = dtype or torch.bfloat16
    out = torch.empty(shape, dtype=dtype, device=dev)
    flat = out.view(-1)
    for lo in range(0, flat.numel(), 1 << 26):
        n = min(1 << 26, flat.numel() - lo)
        flat[lo : lo + n] = (torch.randn(n, generator=g).to(dev) * std).to(dtype)
    return out


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
    gen = host_gen(1)
    h = hrandn((M, K), gen, dev)
    w_norm = hrandn((K,), gen, dev, 0.02)  # gamma = 1 + w
    w_lm = hrandn((V, K), gen, dev, 0.02)
    target = torch.randint(0, V, (M,), generator=gen).to(dev)

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
                     "kernel": "k_gemm_bf16_nt_stream (+ 12 us row-max reduce)", "kernel_ms": gemm_ms},
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
    gen = host_gen(2)
    q = torch.randn(B, 1, H, K, generator=gen)
    k = torch.randn(B, 1, H, K, generator=gen)
    q, k = ((t / t.norm(dim=-1, keepdim=True)).to(torch.bfloat16).to(dev) for t in (q, k))
    v = torch.randn(B, 1, HV, V, generator=gen).to(torch.bfloat16).to(dev)
    g = (-torch.nn.functional.softplus(torch.randn(B, 1, HV, generator=gen))).to(dev)
    beta = torch.sigmoid(torch.randn(B, 1, HV, generator=gen)).to(torch.bfloat16).to(dev)
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
    gen = host_gen(3)
    x = hrandn((T, H), gen, dev)
    wr = hrandn((E, H), gen, dev, 0.02)
    w1 = hrandn((E, 2 * F, H), gen, dev, 0.02)
    w2 = hrandn((E, H, F), gen, dev, 0.02)
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
                         "kernel": "k_moe_fc1_glu_stream + k_moe_fc2_stream (grouped GEMMs)", "kernel_ms": exp_ms},
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
    gen = host_gen(5)
    q = hrandn((n * L, HQ, D), gen, dev)
    k = hrandn((n * L, HKV, D), gen, dev)
    v = hrandn((n * L, HKV, D), gen, dev)
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


def _events_ms(fn, warmup, steps):
    import torch

    timer = KernelTimer()
    for _ in range(warmup):
        fn()
    for _ in range(steps):
        timer(fn)
    torch.cuda.synchronize()
    return timer.mean_ms()


def north_star_kernels(w, dev, steps):
    """The kernels the target names besides the pass's dominant one, each timed here with events at its own
    configuration: grouped expert GEMMs at 16384 tokens (MFMA), the delta-rule scan as a decode step at batch 256 (HBM),
    the log-softmax block sums over [4096, 151936] (HBM), the LM-head GEMM of configs[1] at M = 4096 (MFMA)."""
    import torch

    from isoexec_amd.ops.gdn.gdn_ops import gdn_recurrent_kernel
    from isoexec_amd.ops.logprobs.rowinv import sampled_forward
    from isoexec_amd.ops.mm.mm_hip import linear_nt, router_gemm
    from isoexec_amd.ops.moe.moe_hip import experts_forward, permute, router_topk

    g = host_gen(11)
    out = {}
    # grouped expert GEMMs, configs[3] at T = 16384 (layer 0's experts)
    lw = w.layers[0]
    T, H, E, F, k = 16384, 2048, 128, 768, 8
    x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
    idx, prob, _, _ = router_topk(router_gemm(x, lw["router"]), k, pre_softmax=True)
    perm = permute(idx, prob, E)
    # (a dozen untimed calls first: this leg follows the decode steps, whose small kernels leave the clocks low)
    ms = _events_ms(lambda: experts_forward(x, lw["w1"], lw["w2"], perm), 12, max(steps, 20))
    fl = 2.0 * T * k * H * (2 * F) + 2.0 * T * k * F * H
    out["moe_grouped_gemms_T16384"] = {
        "bound": "mfma", "kernel": "k_moe_fc1_glu_stream + k_moe_fc2_stream", "kernel_ms": ms, "achieved": fl / ms / 1e9,
        "peak": PEAK_MFMA_BF16_TFLOPS, "unit": "TFLOP/s", "frac": fl / ms / 1e9 / PEAK_MFMA_BF16_TFLOPS,
        "traffic": MEASURED_TRAFFIC_BYTES["moe_T16384_grouped_gemms"],
        "traffic_source": TRAFFIC_SOURCE["moe_T16384_grouped_gemms"] + " (not measured in this run)"}
    del x, perm
    # delta-rule scan, decode step at batch 256 (configs[2] dims)
    B, HK, HV, K, V = 256, 16, 32, 128, 128
    q = torch.randn(B, 1, HK, K, generator=g)
    kk = torch.randn(B, 1, HK, K, generator=g)
    q, kk = (t / t.norm(dim=-1, keepdim=True) for t in (q, kk))
    v = torch.randn(B, 1, HV, V, generator=g)
    gate = -torch.nn.functional.softplus(torch.randn(B, 1, HV, generator=g))
    beta = torch.sigmoid(torch.randn(B, 1, HV, generator=g))
    q, kk, v, beta = (t.to(torch.bfloat16).to(dev) for t in (q, kk, v, beta))
    gate = gate.to(dev)
    pool = torch.zeros(B + 1, HV, V, K, device=dev)
    rows = torch.arange(1, B + 1, dtype=torch.int32, device=dev)
    ms = _events_ms(lambda: gdn_recurrent_kernel(q, kk, v, gate, beta, ssm_state=pool, state_indices=rows), 3,
                    max(steps, 20))
    by = B * HV * V * K * 4 * 2
    out["gdn_scan_decode_B256"] = {
        "bound": "hbm", "kernel": "k_gdn_scan", "kernel_ms": ms, "achieved": by / ms / 1e6, "peak": PEAK_HBM_GBS,
        "unit": "GB/s", "frac": by / ms / 1e6 / PEAK_HBM_GBS, "traffic": MEASURED_TRAFFIC_BYTES["gdn_decode_B256"],
        "traffic_source": TRAFFIC_SOURCE["gdn_decode_B256"] + " (not measured in this run)"}
    del pool
    # configs[1]: LM head of hidden 4096 at M = 4096, then the log-softmax over its logits. The [151936, 4096] weight
    # is the model's LM head beside its embedding scaled to the same spread (both host-seeded N(0, .)).
    M, Kd, Vv = 4096, 4096, 151936
    w_lm = torch.cat([w.lm_head, (w.embed.float() * 0.02).to(torch.bfloat16)], dim=1).contiguous()
    h = torch.randn(M, Kd, generator=g).to(torch.bfloat16).to(dev)
    target = torch.randint(0, Vv, (M,), generator=g).to(dev)
    gemm = lambda: linear_nt(h, w_lm, want_row_max=True)
    ms = _events_ms(gemm, 6, steps)
    fl = 2.0 * M * Vv * Kd
    out["lm_head_gemm_M4096_K4096"] = {
        "bound": "mfma", "kernel": "k_gemm_bf16_nt_stream (+ row-max reduce)", "kernel_ms": ms, "achieved": fl / ms / 1e9,
        "peak": PEAK_MFMA_BF16_TFLOPS, "unit": "TFLOP/s", "frac": fl / ms / 1e9 / PEAK_MFMA_BF16_TFLOPS,
        "traffic": MEASURED_TRAFFIC_BYTES["dense_head_M4096_gemm"],
        "traffic_source": TRAFFIC_SOURCE["dense_head_M4096_gemm"] + " (not measured in this run)"}
    # configs[1] at M <= 64: the product is the time memory needs to deliver the 1.245 GB of weights once. The door
    # streams the fragment-packed copy (ix_gemm_bf16_nt_decode); logits written: M * V * 2 B.
    from isoexec_amd.ops.mm.mm_hip import pack_nt_decode

    packed = pack_nt_decode(w_lm)
    for m_small in (16, 64):
        ms = _events_ms(lambda: linear_nt(h[:m_small], packed), 4, max(steps, 20))
        by = Vv * Kd * 2 + m_small * (Vv + Kd) * 2
        out[f"lm_head_gemm_M{m_small}_K4096"] = {
            "bound": "hbm", "kernel": "k_gemm_dec (weights streamed from the packed copy)", "kernel_ms": ms,
            "achieved": by / ms / 1e6, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": by / ms / 1e6 / PEAK_HBM_GBS,
            "traffic": {16: 1.255e9, 64: 1.285e9}[m_small],
            "traffic_source": "profiles/gemm_dec__lm_head_M16_M64_K4096.txt (not measured in this run)"}
    del packed
    logits, row_max = gemm()
    ms = _events_ms(lambda: sampled_forward(logits, target, 8, row_max=row_max), 3, max(steps, 20))
    by = M * Vv * 2
    out["logprob_blocksums_M4096"] = {
        "bound": "hbm", "kernel": "k_lp_blocksums (+ finalize)", "kernel_ms": ms, "achieved": by / ms / 1e6,
        "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": by / ms / 1e6 / PEAK_HBM_GBS, "traffic": 1.245e9,
        "traffic_source": "profiles/logprob_blocksums__dense_head_M4096.txt (not measured in this run)"}
    return out


def decode_bytes_per_step(cfg, n, context, distinct_experts):
    """Bytes a decode step cannot avoid moving at batch ``n`` and mean context ``context``: every byte below is read
    (or read and written) exactly once per step by the algorithm, whatever the kernels do.
      experts   the fc1 + fc2 weights of the experts the step's tokens actually route to (``distinct_experts``: one count
                per layer, read from the step's own routing), 3 * hidden * inter * 2 B each
      gdn       the fp32 delta-rule state of every sequence, read and written: 2 * HV * V * K * 4 B per sequence and layer,
                plus the convolution window (D * (W - 1) * 2 B, read and written)
      kv        the cached keys and values of every sequence: 2 * context * HKV * D * 2 B per sequence and layer
      dense     the projection, router and LM-head weights (read once) and the logits (written once, read once)"""
    gdn_layers = sum(1 for i in range(cfg.layers) if not cfg.is_attention(i))
    att_layers = cfg.layers - gdn_layers
    H = cfg.hidden
    experts = sum(distinct_experts) * 3 * H * cfg.expert_inter * 2
    state = 2 * cfg.gdn_v_heads * cfg.gdn_head_dim * cfg.gdn_head_dim * 4 + 2 * cfg.gdn_qkv * (cfg.conv_width - 1) * 2
    gdn = gdn_layers * n * state
    kv = att_layers * n * 2 * context * cfg.kv_heads * cfg.head_dim * 2
    gdn_proj = (cfg.gdn_qkv + cfg.gdn_z + 2 * cfg.gdn_v_heads) * H + H * cfg.gdn_z
    att_proj = (cfg.q_heads + 2 * cfg.kv_heads) * cfg.head_dim * H + H * cfg.q_heads * cfg.head_dim
    dense = (gdn_layers * gdn_proj + att_layers * att_proj + cfg.layers * cfg.experts * H + cfg.vocab * H) * 2
    dense += 2 * n * cfg.vocab * 2
    parts = {"expert_weights": experts, "gdn_state": gdn, "kv_cache": kv, "dense_weights_and_logits": dense}
    return float(sum(parts.values())), {k: float(v) for k, v in parts.items()}


def decode_roofline(cfg, engine, slots, tokens_step, ms_per_step):
    """HBM roofline of one decode step: the step's own routing says how many experts' weights it has to read."""
    import torch

    log = []
    engine.blocks.routing_log = log
    try:
        engine.decode(slots, tokens_step)
    finally:
        engine.blocks.routing_log = None
    distinct = [int(torch.unique(ids).numel()) for ids in log]
    context = sum(engine.context[s] for s in slots) / len(slots)
    total, parts = decode_bytes_per_step(cfg, len(slots), context, distinct)
    return {"bound": "hbm", "bytes_per_step": total, "bytes_by_part": parts, "distinct_experts_per_layer": distinct,
            "mean_context": context, "ms_per_step": ms_per_step, "achieved": total / (ms_per_step * 1e-3) / 1e9,
            "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": total / (ms_per_step * 1e-3) / 1e9 / PEAK_HBM_GBS}


def rollout_leg(cfg, w, tokens, n, prompt, resp, graph_steps=36):
    """The rollout side of configs[4]: prefill of ``n`` prompts (timed on its second run: the first pays for module
    loads and allocator growth), then decode steps at batch ``n`` with the full-row logprobs the engine reports,
    eager and replayed from a captured graph."""
    import torch

    from isoexec_amd.ops.logprobs.rowinv import full_forward, leaves
    from isoexec_amd.runtimes.hybrid import RolloutEngine

    plens = [prompt] * n
    engine = RolloutEngine(cfg, w, max_num_seqs=n, max_len=prompt + resp)
    slots = list(range(n))
    prompts = tokens.view(n, -1)[:, :prompt].reshape(-1)
    engine.prefill(slots, prompts, plens)
    for s in slots:
        engine.release(s)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    x = engine.prefill(slots, prompts, plens)
    torch.cuda.synchronize()
    t_prefill = time.perf_counter() - t0
    dec_steps = min(resp - 1, 64)
    nxt = tokens.view(n, -1)[:, prompt:prompt + dec_steps]
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
    more = tokens.view(n, -1)[:, prompt + dec_steps:prompt + dec_steps + 4 + graph_steps]
    for sidx in range(4):
        graph.step(more[:, sidx].contiguous())
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for sidx in range(4, 4 + graph_steps):
        x = graph.step(more[:, sidx].contiguous())
        full_forward(engine.blocks.logits(x), leaves())
    torch.cuda.synchronize()
    t_graph = (time.perf_counter() - t0) / graph_steps
    roof = decode_roofline(cfg, engine, slots, more[:, 0].contiguous(), t_graph * 1e3)
    del engine, graph
    return {"prefill_tokens_per_s": n * prompt / t_prefill, "prefill_ms": t_prefill * 1e3,
            "decode_ms_per_step": t_dec * 1e3, "eager_decode_tokens_per_s": n / t_dec,
            "graph_decode_ms_per_step": t_graph * 1e3, "graph_decode_tokens_per_s": n / t_graph, "batch": n,
            "decode_roofline": roof}


def gemm(args):
    """One dense product ``[m, k] x [n, k]^T`` of the batch-invariant GEMM at a shape of the trainer pass (what the traffic
    profiles of the large products run): ``value`` = TFLOP/s, HIP events around each call."""
    import torch

    from isoexec_amd.ops.mm.mm_hip import linear_nt, pack_nt_decode

    dev = "cuda:0"
    g = host_gen(21)
    M, K, N = args.m, args.k, args.n
    a = hrandn((M, K), g, dev)
    w = hrandn((N, K), g, dev, std=0.02)
    if args.packed:  # at most 64 rows: the weight is streamed from its fragment-packed copy
        w = pack_nt_decode(w)
        if w is None or M > 64:
            raise SystemExit("--packed serves m <= 64, n a multiple of 32 and k in {1024, 2048, 3072, 4096}")
    fn = lambda: linear_nt(a, w, tile=args.tile, want_row_max=args.row_max)
    ms = _events_ms(fn, args.warmup, args.steps)
    fl = 2.0 * M * N * K
    algo = 2.0 * (M * K + N * K + M * N)
    if args.packed:
        return {"metric": "dense GEMM GB/s (weights streamed)", "value": algo / ms / 1e6, "unit": "GB/s", "n_gpus": 1,
                "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
                "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
                "config": {"workload": f"gemm_bf16_nt_decode {M} x {K} x {N} (packed weight)"},
                "roofline": {"bound": "hbm", "achieved": algo / ms / 1e6, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                             "frac": algo / ms / 1e6 / PEAK_HBM_GBS, "traffic": None, "algorithmic_bytes": algo}}
    return {"metric": "dense GEMM TFLOP/s", "value": fl / ms / 1e9, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16", "data": "synthetic",
            "config": {"workload": f"gemm_bf16_nt {M} x {K} x {N} (tile {args.tile}, row max {bool(args.row_max)})"},
            "roofline": {"bound": "mfma", "achieved": fl / ms / 1e9, "peak": PEAK_MFMA_BF16_TFLOPS, "unit": "TFLOP/s",
                         "frac": fl / ms / 1e9 / PEAK_MFMA_BF16_TFLOPS, "traffic": None,
                         "algorithmic_bytes": algo}}


def decode(args):
    """The rollout leg of configs[4] alone (what the decode profiles run): ``value`` = decode tokens/s at batch
    ``--seqs`` from the captured graph, ``roofline`` = the step against HBM."""
    import torch

    from isoexec_amd.runtimes.hybrid import HybridConfig, HybridWeights

    dev = "cuda:0"
    cfg = HybridConfig()
    n, prompt, resp = args.seqs, args.prompt, args.response
    w = HybridWeights.make(cfg, seed=0, device=dev, host_rng=True)
    tokens = torch.randint(0, cfg.vocab, (n * (prompt + resp),), generator=host_gen(4)).to(dev)
    leg = rollout_leg(cfg, w, tokens, n, prompt, resp, graph_steps=max(args.steps, 8))
    roof = leg.pop("decode_roofline")
    return {"metric": "decode tokens/s", "value": leg["graph_decode_tokens_per_s"], "unit": "tokens/s", "n_gpus": 1,
            "steps": max(args.steps, 8), "warmup": 4, "ms_per_step": leg["graph_decode_ms_per_step"],
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": f"hybrid (BASELINE configs[4]) rollout: decode at batch {n} after {prompt}-token prompts, "
                                   "full-row logprobs per step, replayed from a captured graph"},
            "roofline": {**roof, "traffic": None}, "rollout": leg}


def hybrid_cpu_baseline(cfg, w, tokens, seqs, prompt, resp):
    """The CPU oracle composition of the same model (same weights) scoring a slice of the same token stream: the first
    ``seqs`` sequences cut to ``prompt`` + ``resp`` tokens each, on this box's host cores."""
    import torch

    from oracle import hybrid as o_hybrid

    wn = o_hybrid.weights_from_torch(w)   # fp32 copies of the bf16 weights (conversion not timed)
    L = tokens.numel() // 64
    tok = tokens.view(64, L)[:seqs, : prompt + resp].reshape(-1).cpu().numpy()
    oracle = o_hybrid.HybridOracle(cfg, wn)
    t0 = time.perf_counter()
    lps = oracle.response_logprobs(tok, [prompt + resp] * seqs, [prompt] * seqs)
    dt = time.perf_counter() - t0
    assert all(bool((lp <= 0).all()) for lp in lps)
    return {"value": seqs * (prompt + resp) / dt, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"trainer scoring pass of the same model and weights over the first {seqs} sequences cut to "
                      f"{prompt} + {resp} tokens ({dt:.1f} s of CPU work; numpy/BLAS fp32 oracle composition)"}


def hybrid(args):
    """BASELINE.json configs[4]: the 8-layer hybrid model. One step = one trainer scoring pass over ``--seqs``
    sequences of prompt + response tokens; the rollout's prefill and decode are timed beside it."""
    import torch

    from isoexec_amd.ops.moe import moe_hip
    from isoexec_amd.runtimes.hybrid import HybridConfig, HybridWeights, RolloutEngine, TrainerModel

    dev = "cuda:0"
    cfg = HybridConfig()
    n, prompt, resp = args.seqs, args.prompt, args.response
    w = HybridWeights.make(cfg, seed=0, device=dev, host_rng=True)
    tokens = torch.randint(0, cfg.vocab, (n * (prompt + resp),), generator=host_gen(4)).to(dev)
    lens, plens = [prompt + resp] * n, [prompt] * n
    trainer = TrainerModel(cfg, w)
    fn = lambda: trainer.response_logprobs(tokens, lens, plens)
    for _ in range(args.warmup):
        fn()
    torch.cuda.synchronize()
    # events around every launch of the grouped expert GEMMs inside the timed steps (same stream as the kernels)
    t_experts = KernelTimer()
    real_experts = moe_hip.experts_forward
    moe_hip.experts_forward = lambda *a, **k: t_experts(lambda: real_experts(*a, **k))
    try:
        t0 = time.perf_counter()
        for _ in range(args.steps):
            lp = fn()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / args.steps
    finally:
        moe_hip.experts_forward = real_experts
    assert all(bool(torch.isfinite(t).all()) for t in lp)
    total = n * (prompt + resp)
    exp_ms = t_experts.mean_ms()
    exp_fl = 2.0 * total * cfg.topk * cfg.hidden * (2 * cfg.expert_inter) + 2.0 * total * cfg.topk * cfg.expert_inter * cfg.hidden
    leg = rollout_leg(cfg, w, tokens, n, prompt, resp)
    t_graph = leg["graph_decode_ms_per_step"] * 1e-3
    out = {"metric": "trainer-fwd & decode tokens/s at bitwise parity; % of HBM/MFMA roofline", "value": total / dt,
           "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt * 1e3,
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
           "config": {"workload": f"hybrid (BASELINE configs[4]): 8 layers (3 GatedDeltaNet : 1 attention) + MoE 128 experts "
                                  f"top-8, vocab 151936; trainer scoring pass over {n} x ({prompt} + {resp}) tokens",
                      "tokens_per_step": total, "rng": "host torch.Generator (weights seed 0, tokens seed 4)"},
           "decode_tokens_per_s": n / t_graph,
           "roofline": {"bound": "mfma", "achieved": exp_fl / exp_ms / 1e9, "peak": PEAK_MFMA_BF16_TFLOPS,
                        "unit": "TFLOP/s", "frac": exp_fl / exp_ms / 1e9 / PEAK_MFMA_BF16_TFLOPS,
                        "traffic": MEASURED_TRAFFIC_BYTES["moe_T163840_grouped_gemms"] if total == 163840 else None,
                        "traffic_source": TRAFFIC_SOURCE["moe_T163840_grouped_gemms"] + " (not measured in this run)",
                        "kernel": f"k_moe_fc1_glu_stream + k_moe_fc2_stream (grouped expert GEMMs, {total} tokens x top-8 per launch "
                                  f"pair, {cfg.layers} pairs per pass)", "kernel_ms": exp_ms,
                        "share_of_step": cfg.layers * exp_ms / (dt * 1e3)},
           "rollout": leg}
    out["kernels"] = north_star_kernels(w, dev, max(args.steps, 10))
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = hybrid_cpu_baseline(cfg, w, tokens, args.cpu_seqs, args.cpu_prompt, args.cpu_response)
    return out


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
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default="hybrid", choices=["dense_head", "gdn_decode", "moe", "hybrid", "attention", "digest", "decode", "gemm"])
    ap.add_argument("--seqs", type=int, default=64)
    ap.add_argument("--prompt", type=int, default=2048)
    ap.add_argument("--response", type=int, default=512)
    ap.add_argument("--tokens", type=int, default=None)
    ap.add_argument("--batch", type=int, default=256)
    ap.add_argument("--tile", type=int, default=0)
    ap.add_argument("--m", type=int, default=32768)
    ap.add_argument("--k", type=int, default=2048)
    ap.add_argument("--n", type=int, default=151936)
    ap.add_argument("--row-max", type=int, default=0)
    ap.add_argument("--packed", action="store_true")
    ap.add_argument("--cpu-tokens", type=int, default=2048)
    ap.add_argument("--cpu-seqs", type=int, default=4)
    ap.add_argument("--cpu-prompt", type=int, default=160)
    ap.add_argument("--cpu-response", type=int, default=32)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (no collectives, no sharding, no figure at several GPUs); "
              "--gpus must be 1", file=sys.stderr)
        sys.exit(2)
    if args.tokens is None:
        args.tokens = 16384 if args.workload == "moe" else 4096
    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(3)
    out = {"dense_head": dense_head, "gdn_decode": gdn_decode, "moe": moe, "hybrid": hybrid, "attention": attention, "digest": digest,
           "decode": decode, "gemm": gemm}[args.workload](args)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
