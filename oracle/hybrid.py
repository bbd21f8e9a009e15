"""Oracle: the hybrid GatedDeltaNet / attention / mixture-of-experts model as ONE composition of the per-op
restatements in this package -- the trainer's full-sequence scoring pass, sequence by sequence, on the CPU.

TEST INFRASTRUCTURE ONLY (imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg; the product
never imports it). Every arithmetic step is one of the pinned functions of oracle/{norms,mm,gdn,moe,attention,
logprobs}.py; this file adds only the wiring, which follows the layer layout the reference runs through Megatron
(GPTModel layer loop; mixer = GatedDeltaNet via ops/gdn/gdn_ops.py:513-558 and the gated norm of
runtimes/megatron/gdn_fla_shim.py:390-425, or attention via ops/attention + ops/rope; MoE via
ops/moe/moe_batch_invariant.py:394-416 and moe_batched_experts.py:496-503; the scored rows through
ops/logprobs/rowinv.py:666-712). The wiring itself is pinned by tests/test_oracle_hybrid.py: an independent float64
forward of the same model written with library routines (torch.nn.functional softmax / silu / rms_norm formulas),
within a stated tolerance, and structural invariants (a sequence alone == the same sequence in a batch; a prefix's
logprobs do not depend on what follows).

Weights are a dict of float32 numpy arrays holding bf16-representable values:
    embed [V, H], lm_head [V, H], final_norm [H], layers[i] = {pre_norm, post_norm, router [E, H], w1 [E, 2F, H],
    w2 [E, H, F]} + attention {qkv_proj, o_proj} or GatedDeltaNet {in_proj, conv_weight [D, W], conv_bias [D],
    A_log, dt_bias [HV], out_norm [K], out_proj}.
"""

from __future__ import annotations

import numpy as np

from . import attention as o_attn
from . import gdn as o_gdn
from . import logprobs as o_lp
from . import moe as o_moe
from . import norms as o_norms
from .prims import DEFAULT, F32, Prims, round_bf16


def default_matmul(a: np.ndarray, w: np.ndarray) -> np.ndarray:
    """``a . w^T`` with fp32 accumulation (numpy's order), unrounded."""
    return (a.astype(F32) @ w.astype(F32).T).astype(F32)


def matmul_fp64(a: np.ndarray, w: np.ndarray) -> np.ndarray:
    return (a.astype(np.float64) @ w.astype(np.float64).T).astype(F32)


class HybridOracle:
    """``cfg`` needs the attributes of isoexec_amd.runtimes.hybrid.HybridConfig (hidden, layers, attention_every,
    gdn_k_heads, gdn_v_heads, gdn_head_dim, conv_width, q_heads, kv_heads, head_dim, rope_theta, max_positions,
    experts, topk, expert_inter, moe_combine_dtype, eps). ``routing[layer]`` (optional) = int top-k expert ids
    ``[T, k]`` for the packed tokens: the discrete choice is then taken from there (probabilities are still this
    function's own: softmax over all experts, the chosen ones renormalised)."""

    def __init__(self, cfg, weights: dict, prims: Prims = DEFAULT, matmul=None, routing=None):
        self.cfg, self.w, self.prims = cfg, weights, prims
        self.mm = matmul or default_matmul
        self.routing = routing
        self.cos, self.sin = o_attn.rope_tables(cfg.max_positions, cfg.head_dim, cfg.rope_theta)

    def is_attention(self, layer: int) -> bool:
        return (layer + 1) % self.cfg.attention_every == 0

    def linear(self, x, w):
        return round_bf16(self.mm(x, w))

    # ---- mixers (one sequence at a time: nothing crosses sequences)
    def gdn_mixer(self, lw, x):
        c = self.cfg
        K, HK, HV = c.gdn_head_dim, c.gdn_k_heads, c.gdn_v_heads
        kd, vd = HK * K, HV * K
        proj = self.linear(x, lw["in_proj"])
        qkv, z = proj[:, : 2 * kd + vd], proj[:, 2 * kd + vd : 2 * kd + 2 * vd].reshape(-1, HV, K)
        b, a = proj[:, 2 * kd + 2 * vd : 2 * kd + 2 * vd + HV], proj[:, 2 * kd + 2 * vd + HV :]
        y, _ = o_gdn.causal_conv(qkv, lw["conv_weight"], lw["conv_bias"], prims=self.prims)
        q = o_gdn.l2norm(y[:, :kd].reshape(-1, HK, K))
        k = o_gdn.l2norm(y[:, kd : 2 * kd].reshape(-1, HK, K))
        v = y[:, 2 * kd :].reshape(-1, HV, K)
        g, beta = o_gdn.gate_and_beta(a, b, lw["A_log"], lw["dt_bias"], prims=self.prims)
        state = np.zeros((HV, K, K), dtype=F32)
        o = o_gdn.scan(q, k, v, g, beta, state, io_bf16=True, prims=self.prims)
        normed = o_norms.gated_out_norm(o, z, lw["out_norm"], c.eps, prims=self.prims)
        return self.linear(normed.reshape(x.shape[0], vd), lw["out_proj"])

    def attention_mixer(self, lw, x):
        c = self.cfg
        D, HQ, HKV = c.head_dim, c.q_heads, c.kv_heads
        T = x.shape[0]
        proj = self.linear(x, lw["qkv_proj"])
        pos = np.arange(T, dtype=np.int32)
        q = o_attn.rope(proj[:, : HQ * D].reshape(T, HQ, D), self.cos, self.sin, pos)
        k = o_attn.rope(proj[:, HQ * D : (HQ + HKV) * D].reshape(T, HKV, D), self.cos, self.sin, pos)
        v = proj[:, (HQ + HKV) * D :].reshape(T, HKV, D)
        o = o_attn.attend_causal(q, k, v, prims=self.prims)
        return self.linear(o.reshape(T, HQ * D), lw["o_proj"])

    def moe(self, layer, lw, x, token0):
        c = self.cfg
        logits = self.mm(x, lw["router"])
        forced = None if self.routing is None else np.asarray(self.routing[layer][token0 : token0 + x.shape[0]])
        idx, prob = o_moe.router_topk(logits, c.topk, 1, prims=self.prims, forced_idx=forced)
        counts, st, pp, cr = o_moe.permute(idx.astype(np.int32), prob, c.experts)
        eo, _ = o_moe.expert_chain(x, lw["w1"], lw["w2"], st, pp, counts, prims=self.prims, matmul=self.mm)
        return o_moe.combine(eo, cr, fp32_acc=c.moe_combine_dtype == "fp32")

    # ---- the residual stream
    def hidden_states(self, tokens: np.ndarray, token0: int = 0) -> np.ndarray:
        """One sequence ``tokens [T]`` -> final-normed hidden states ``[T, H]``. ``token0``: its first token's index
        in the packed batch (only used to look up supplied routing)."""
        c, w = self.cfg, self.w
        h = w["embed"][tokens].astype(F32)
        x = o_norms.rms_norm_gamma(h, w["layers"][0]["pre_norm"], c.eps)
        for i in range(c.layers):
            lw = w["layers"][i]
            mixed = self.attention_mixer(lw, x) if self.is_attention(i) else self.gdn_mixer(lw, x)
            x, h = o_norms.add_rms_norm_gamma(mixed, h, lw["post_norm"], c.eps)
            delta = self.moe(i, lw, x, token0)
            nxt = w["layers"][i + 1]["pre_norm"] if i + 1 < c.layers else w["final_norm"]
            x, h = o_norms.add_rms_norm_gamma(delta, h, nxt, c.eps)
        return x

    def response_logprobs(self, tokens: np.ndarray, lens, prompt_lens, leaves: int = 8) -> list:
        """Packed ``tokens``; per sequence the fp32 logprobs of tokens ``prompt_len .. len-1``, each scored from the
        hidden state one position earlier (the trainer's contract)."""
        out, start = [], 0
        for n, p in zip(lens, prompt_lens):
            seq = np.asarray(tokens[start : start + n])
            x = self.hidden_states(seq, start)
            logits = self.linear(x[p - 1 : n - 1], self.w["lm_head"])
            lp, _ = o_lp.rowinv_sampled(logits, seq[p:n].astype(np.int64), leaves, prims=self.prims)
            out.append(lp)
            start += n
        return out


def weights_from_torch(w) -> dict:
    """HybridWeights (device tensors) -> the dict of float32 numpy arrays this oracle takes."""
    f = lambda t: t.detach().float().cpu().numpy()
    return {"embed": f(w.embed), "lm_head": f(w.lm_head), "final_norm": f(w.final_norm),
            "layers": [{k: f(v) for k, v in lw.items()} for lw in w.layers]}
