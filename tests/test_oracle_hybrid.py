"""Pins the WIRING of oracle/hybrid.py (every arithmetic step it calls is pinned in the other oracle tests): an
independent float64 forward of the same model, written here with torch library routines (softmax, silu, conv1d,
scaled-dot-product formulas) and a plain token loop for the delta rule, must agree within a stated tolerance; and the
structural invariants a trainer pass has (a sequence alone == inside a batch; a prefix's logprobs do not depend on what
follows it; supplied routing == own routing when it is the same routing)."""

import types

import numpy as np
import torch

from oracle import hybrid as o_hybrid
from oracle.prims import round_bf16

F64 = torch.float64


def small_cfg():
    return types.SimpleNamespace(hidden=64, vocab=512, layers=4, attention_every=2, gdn_k_heads=2, gdn_v_heads=4,
                                 gdn_head_dim=32, conv_width=4, q_heads=4, kv_heads=2, head_dim=32, rope_theta=1.0e6,
                                 max_positions=128, experts=8, topk=2, expert_inter=32, moe_combine_dtype="fp32",
                                 eps=1.0e-6)


def make_weights(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    bf = lambda shape, std: (torch.randn(shape, generator=g) * std).to(torch.bfloat16).float().numpy()
    H = cfg.hidden
    kd, vd = cfg.gdn_k_heads * cfg.gdn_head_dim, cfg.gdn_v_heads * cfg.gdn_head_dim
    w = {"embed": bf((cfg.vocab, H), 1.0), "lm_head": bf((cfg.vocab, H), 0.05), "final_norm": bf((H,), 0.02),
         "layers": []}
    for i in range(cfg.layers):
        lw = {"pre_norm": bf((H,), 0.02), "post_norm": bf((H,), 0.02), "router": bf((cfg.experts, H), 0.1),
              "w1": bf((cfg.experts, 2 * cfg.expert_inter, H), 0.1), "w2": bf((cfg.experts, H, cfg.expert_inter), 0.1)}
        if (i + 1) % cfg.attention_every == 0:
            lw["qkv_proj"] = bf(((cfg.q_heads + 2 * cfg.kv_heads) * cfg.head_dim, H), 0.1)
            lw["o_proj"] = bf((H, cfg.q_heads * cfg.head_dim), 0.1)
        else:
            lw["in_proj"] = bf((2 * kd + 2 * vd + 2 * cfg.gdn_v_heads, H), 0.1)
            lw["conv_weight"] = bf((2 * kd + vd, cfg.conv_width), 0.4)
            lw["conv_bias"] = bf((2 * kd + vd,), 0.1)
            lw["A_log"] = (torch.randn(cfg.gdn_v_heads, generator=g) * 0.3).numpy()
            lw["dt_bias"] = (torch.randn(cfg.gdn_v_heads, generator=g) * 0.3).numpy()
            lw["out_norm"] = bf((cfg.gdn_head_dim,), 0.02)
            lw["out_proj"] = bf((H, vd), 0.1)
        w["layers"].append(lw)
    return w


# ---------------------------------------------------------------- the independent float64 forward
def t64(a):
    return torch.from_numpy(np.asarray(a)).to(F64)


def rms(x, w, eps):
    return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * (1.0 + t64(w))


def reference_hidden(cfg, w, tokens):
    T = len(tokens)
    h = t64(w["embed"])[torch.as_tensor(tokens)]
    for i in range(cfg.layers):
        lw = w["layers"][i]
        x = rms(h, lw["pre_norm"], cfg.eps)
        if (i + 1) % cfg.attention_every == 0:
            D, HQ, HKV = cfg.head_dim, cfg.q_heads, cfg.kv_heads
            proj = x @ t64(lw["qkv_proj"]).T
            q, k, v = proj[:, : HQ * D].view(T, HQ, D), proj[:, HQ * D : (HQ + HKV) * D].view(T, HKV, D), proj[:, (HQ + HKV) * D :].view(T, HKV, D)
            inv = 1.0 / cfg.rope_theta ** (torch.arange(0, D, 2, dtype=F64) / D)
            ang = torch.arange(T, dtype=F64)[:, None] * inv[None, :]
            cos, sin = torch.cat([ang.cos(), ang.cos()], -1)[:, None, :], torch.cat([ang.sin(), ang.sin()], -1)[:, None, :]
            rot = lambda t: torch.cat([-t[..., D // 2 :], t[..., : D // 2]], -1)
            q, k = q * cos + rot(q) * sin, k * cos + rot(k) * sin
            k, v = k.repeat_interleave(HQ // HKV, 1), v.repeat_interleave(HQ // HKV, 1)
            s = torch.einsum("thd,shd->hts", q, k) / D ** 0.5
            s = s.masked_fill(torch.ones(T, T).triu(1).bool()[None], float("-inf"))
            o = torch.einsum("hts,shd->thd", torch.softmax(s, -1), v).reshape(T, HQ * D)
            mixed = o @ t64(lw["o_proj"]).T
        else:
            K, HK, HV = cfg.gdn_head_dim, cfg.gdn_k_heads, cfg.gdn_v_heads
            kd, vd = HK * K, HV * K
            proj = x @ t64(lw["in_proj"]).T
            qkv, z = proj[:, : 2 * kd + vd], proj[:, 2 * kd + vd : 2 * kd + 2 * vd].view(T, HV, K)
            b, a = proj[:, 2 * kd + 2 * vd : 2 * kd + 2 * vd + HV], proj[:, 2 * kd + 2 * vd + HV :]
            y = torch.nn.functional.conv1d(torch.nn.functional.pad(qkv.T[None], (cfg.conv_width - 1, 0)),
                                           t64(lw["conv_weight"])[:, None, :], t64(lw["conv_bias"]), groups=2 * kd + vd)[0].T
            y = torch.nn.functional.silu(y)
            l2 = lambda t: t / torch.sqrt((t * t).sum(-1, keepdim=True) + 1e-6)
            q = l2(y[:, :kd].view(T, HK, K)).repeat_interleave(HV // HK, 1) * K ** -0.5
            k = l2(y[:, kd : 2 * kd].view(T, HK, K)).repeat_interleave(HV // HK, 1)
            v = y[:, 2 * kd :].view(T, HV, K)
            g = -torch.exp(t64(lw["A_log"])) * torch.nn.functional.softplus(a + t64(lw["dt_bias"]))
            beta = torch.sigmoid(b)
            S = torch.zeros(HV, K, K, dtype=F64)    # [head, v, k]
            o = torch.zeros(T, HV, K, dtype=F64)
            for t in range(T):                       # the delta rule, token by token
                S = S * torch.exp(g[t])[:, None, None]
                pred = torch.einsum("hvk,hk->hv", S, k[t])
                S = S + torch.einsum("hv,hk->hvk", (v[t] - pred) * beta[t][:, None], k[t])
                o[t] = torch.einsum("hvk,hk->hv", S, q[t])
            normed = rms(o, lw["out_norm"], cfg.eps) * torch.nn.functional.silu(z)
            mixed = normed.reshape(T, vd) @ t64(lw["out_proj"]).T
        h = h + mixed
        x = rms(h, lw["post_norm"], cfg.eps)
        p = torch.softmax(x @ t64(lw["router"]).T, -1)
        tv, ti = torch.topk(p, cfg.topk, dim=-1)
        tv = tv / tv.sum(-1, keepdim=True)
        delta = torch.zeros_like(h)
        for t in range(T):
            for pj, ej in zip(tv[t], ti[t]):
                u = x[t] @ t64(lw["w1"][ej]).T
                F = cfg.expert_inter
                delta[t] += (torch.nn.functional.silu(u[:F]) * u[F:] * pj) @ t64(lw["w2"][ej]).T
        h = h + delta
    return rms(h, w["final_norm"], cfg.eps), None


def reference_logprobs(cfg, w, tokens, p):
    x, _ = reference_hidden(cfg, w, tokens)
    logits = x[p - 1 : len(tokens) - 1] @ t64(w["lm_head"]).T
    lp = torch.log_softmax(logits, -1)
    return lp.gather(1, torch.as_tensor(tokens[p:])[:, None])[:, 0].numpy()


def test_wiring_against_an_independent_float64_forward():
    cfg, w = small_cfg(), make_weights(small_cfg())
    rng = np.random.default_rng(1)
    tokens = rng.integers(0, cfg.vocab, size=24)
    oracle = o_hybrid.HybridOracle(cfg, w)
    got = oracle.response_logprobs(tokens, [24], [9])[0]
    want = reference_logprobs(cfg, w, tokens, 9)
    # bf16 activations through 4 layers: a few parts in a hundred of a logit; a wiring mistake (a swapped slice, a
    # missing residual, a wrong norm weight) moves logprobs by whole units
    assert got.shape == want.shape == (15,)
    assert np.abs(got - want).max() < 0.12, np.abs(got - want).max()
    assert np.abs(got - want).mean() < 0.04
    assert np.std(want) > 0.3          # the model is not uniform: the comparison says something


def test_sequences_do_not_see_each_other_and_prefixes_do_not_see_the_future():
    cfg, w = small_cfg(), make_weights(small_cfg(), seed=2)
    rng = np.random.default_rng(3)
    lens, plens = [20, 7, 13], [5, 3, 12]
    tokens = rng.integers(0, cfg.vocab, size=sum(lens))
    oracle = o_hybrid.HybridOracle(cfg, w)
    batch = oracle.response_logprobs(tokens, lens, plens)
    alone = oracle.response_logprobs(tokens[20:27], [7], [3])[0]
    assert np.array_equal(batch[1].view(np.uint32), alone.view(np.uint32))
    longer = oracle.response_logprobs(tokens[:20], [20], [5])[0]
    prefix = oracle.response_logprobs(tokens[:12], [12], [5])[0]
    assert np.array_equal(longer[:7].view(np.uint32), prefix.view(np.uint32))


def test_supplied_routing_reproduces_own_routing_and_changes_the_result_when_it_differs():
    from oracle import moe as o_moe

    cfg, w = small_cfg(), make_weights(small_cfg(), seed=4)
    tokens = np.random.default_rng(5).integers(0, cfg.vocab, size=16)
    own = o_hybrid.HybridOracle(cfg, w)
    base = own.response_logprobs(tokens, [16], [4])[0]
    # record the oracle's own choices layer by layer, then feed them back
    chosen = []
    real = o_moe.router_topk

    def spy(logits, k, mode=0, scaling=None, prims=None, forced_idx=None):
        idx, prob = real(logits, k, mode, scaling, prims=prims or own.prims, forced_idx=forced_idx)
        chosen.append(idx.copy())
        return idx, prob

    o_moe.router_topk = spy
    try:
        own.response_logprobs(tokens, [16], [4])
    finally:
        o_moe.router_topk = real
    fed = o_hybrid.HybridOracle(cfg, w, routing=chosen).response_logprobs(tokens, [16], [4])[0]
    assert np.array_equal(fed.view(np.uint32), base.view(np.uint32))
    other = [np.roll(c, 1, axis=1) % cfg.experts for c in chosen]          # swap rank order: same experts
    swapped = o_hybrid.HybridOracle(cfg, w, routing=other).response_logprobs(tokens, [16], [4])[0]
    assert np.abs(swapped - base).max() < 0.05                             # same experts, other rank order: tiny
    wrong = [(c + 1) % cfg.experts for c in chosen]
    moved = o_hybrid.HybridOracle(cfg, w, routing=wrong).response_logprobs(tokens, [16], [4])[0]
    assert np.abs(moved - base).max() > 0.05
