"""Oracle: MoE router, permutation, expert SwiGLU chain and combine (reference
ops/moe/moe_router_o2_kernel.py:87-174,369-397; ops/moe/moe_batched_experts.py:496-503;
ops/moe/moe_batch_invariant.py:276-320; ops/moe/moe_combine_kernel.py:36-76).

Pinned by (tests/test_oracle_gdn_moe.py): ``torch.topk`` / ``torch.softmax`` on CPU for the router
(mode 1 is the HF Qwen3-MoE form: softmax over all experts, top-k, renormalise); tie and NaN
cases from the reference kernel's comments (lowest index wins, NaN -> -inf); the eager
``argsort(stable)`` permutation of ``ref_permute_index``; a brute-force per-expert loop with
float64 matmuls for the expert chain; ascending-expert combine against an explicit loop.
"""

from __future__ import annotations

import numpy as np

from .prims import DEFAULT, F32, Prims, pairwise_tree, round_bf16


def _topk_rank(scores: np.ndarray, k: int):
    """Winners by (score desc, index asc). ``scores [T, E]`` with NaN already mapped to -inf."""
    T, E = scores.shape
    order = np.lexsort((np.broadcast_to(np.arange(E), (T, E)), -scores.astype(np.float64)), axis=1)
    # lexsort: last key primary -> -score ascending == score descending; ties by index ascending.
    idx = order[:, :k]
    return idx.astype(np.int32), np.take_along_axis(scores, idx, axis=1)


def _tree_k(t: np.ndarray) -> np.ndarray:
    k = t.shape[-1]
    assert k & (k - 1) == 0
    return pairwise_tree(t)


def router_topk(logits: np.ndarray, k: int, mode: int = 0, scaling: float | None = None, prims: Prims = DEFAULT,
                forced_idx: np.ndarray | None = None):
    """Returns ``(idx [T,k] int32 in rank order, prob [T,k] fp32)``. ``forced_idx [T,k]`` replaces the selection
    (the winners and their rank order are taken from it; every value is still computed here), for comparing a
    composed model whose discrete choices must be like for like.
    mode 0: top-k on logits, softmax over the winners (``ref_router_dense``);
    mode 1: softmax over all E (sum: per-lane columns e % 64 left to right over e // 64, then the
    adjacent-pairwise tree over the 64 lanes), top-k on the probabilities, renormalise."""
    s = logits.astype(F32).copy()
    s[np.isnan(s)] = -np.inf
    T, E = s.shape
    if mode == 1:
        m = s.max(axis=1, keepdims=True)
        e = prims.exp((s - m).astype(F32))
        chunks = -(-E // 64)
        pad = np.zeros((T, chunks * 64), dtype=F32)
        pad[:, :E] = e
        pad = pad.reshape(T, chunks, 64)
        z = np.zeros((T, 64), dtype=F32)
        for c in range(chunks):
            z = (z + pad[:, c]).astype(F32)
        z = pairwise_tree(z)
        s = (e / z[:, None]).astype(F32)
    if forced_idx is None:
        idx, vals = _topk_rank(s, k)
    else:
        idx = np.asarray(forced_idx).astype(np.int32)
        vals = np.take_along_axis(s, idx.astype(np.int64), axis=1)
    if mode == 0:
        p = prims.exp((vals - vals[:, :1]).astype(F32))
    else:
        p = vals.astype(F32)
    den = _tree_k(p)
    p = (p / den[:, None]).astype(F32)
    if scaling:
        p = (p * F32(scaling)).astype(F32)
    return idx, p


def dense_from_topk(idx, prob, E):
    T, k = idx.shape
    dp = np.zeros((T, E), dtype=F32)
    dm = np.zeros((T, E), dtype=bool)
    rows = np.arange(T)[:, None]
    dp[rows, idx] = prob
    dm[rows, idx] = True
    return dp, dm


def permute(idx: np.ndarray, prob: np.ndarray, E: int):
    """Expert-major, token-ascending permutation. Returns ``(counts [E], sorted_token [T*k],
    permuted_prob [T*k], combine_rows [T,k])`` with combine_rows in ascending expert order."""
    T, k = idx.shape
    flat_e = idx.reshape(-1).astype(np.int64)
    flat_t = np.repeat(np.arange(T), k)
    order = np.lexsort((flat_t, flat_e))  # by expert, then token
    sorted_token = flat_t[order].astype(np.int32)
    permuted_prob = prob.reshape(-1)[order].astype(F32)
    counts = np.bincount(flat_e, minlength=E).astype(np.int32)
    pos = np.empty(T * k, dtype=np.int64)
    pos[order] = np.arange(T * k)
    pos = pos.reshape(T, k)
    asc = np.argsort(idx, axis=1, kind="stable")
    combine_rows = np.take_along_axis(pos, asc, axis=1).astype(np.int32)
    return counts, sorted_token, permuted_prob, combine_rows


def expert_chain(x, w1, w2, sorted_token, permuted_prob, counts, prims: Prims = DEFAULT, matmul=None):
    """Rows in permuted order: ``inter = bf16(x W1^T)``; ``s = bf16(silu(gate))``;
    ``h = bf16(s * up)``; ``a = bf16(h * prob)``; ``y = bf16(a W2^T)``. ``matmul(a, w)`` computes
    ``a . w^T`` in fp32 (default: numpy)."""
    mm = matmul or (lambda a, w: (a.astype(F32) @ w.astype(F32).T).astype(F32))
    E, F2, H = w1.shape
    F = F2 // 2
    rows = sorted_token.shape[0]
    inter_all = np.zeros((rows, F), dtype=F32)
    out = np.zeros((rows, H), dtype=F32)
    start = 0
    for e in range(E):
        c = int(counts[e])
        if c == 0:
            continue
        sl = slice(start, start + c)
        xe = x[sorted_token[sl]].astype(F32)
        inter = round_bf16(mm(xe, w1[e]))
        gate, up = inter[:, :F], inter[:, F:]
        s = round_bf16(prims.silu_div(gate))
        h = round_bf16((s * up).astype(F32))
        a = round_bf16((h * permuted_prob[sl, None]).astype(F32))
        inter_all[sl] = a
        out[sl] = round_bf16(mm(a, w2[e]))
        start += c
    return out, inter_all


def combine(expert_out, combine_rows, fp32_acc=False):
    T, k = combine_rows.shape
    acc = expert_out[combine_rows[:, 0]].astype(F32)
    for r in range(1, k):
        acc = (acc + expert_out[combine_rows[:, r]].astype(F32)).astype(F32)
        if not fp32_acc:
            acc = round_bf16(acc)
    return round_bf16(acc)


def moe_ffn(x, router_w, w1, w2, k, mode=0, logit_bias=None, prims: Prims = DEFAULT, logits=None):
    """Whole FFN for ``x [T, H]`` (bf16-representable fp32). ``logits`` may be supplied (e.g. the
    device's own router GEMM output) so that the discrete top-k decision is compared like for like."""
    if logits is None:
        logits = (x.astype(F32) @ router_w.astype(F32).T).astype(F32)
        if logit_bias is not None:
            logits = (logits + logit_bias.astype(F32)[None, :]).astype(F32)
    idx, prob = router_topk(logits, k, mode, prims=prims)
    counts, st, pp, cr = permute(idx, prob, router_w.shape[0])
    eo, _ = expert_chain(x, w1, w2, st, pp, counts, prims=prims)
    return combine(eo, cr)
