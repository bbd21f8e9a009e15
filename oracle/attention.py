"""CPU restatement of the attention and rotary-embedding algorithms (test infrastructure only).

Attention follows the reference's contract for this op -- causal grouped-query attention with a
single walk of the keys, so a query's value is independent of the call it ran in
(isoexec/ops/attention/_register.py:15-47, varlen_backend.py:1-10) -- in the block-wise online form
the device kernel fixes: blocks of 32 keys, an fp32 reference point (a running maximum of the unscaled
scores that moves only when exceeded by more than 2^8), fp32 denominator and accumulator, probabilities 2 ** fma(s, c, -m c) with c = scale * log2(e), bf16 probabilities into the
value product, one reciprocal of the denominator at the end. The two matrix products are computed here in float64 and
rounded once to fp32: the device's matrix instruction sums the same products in an order that is not
part of its public contract, so oracle and kernel agree to the last few fp32 bits of a block, not bit
for bit, except on inputs whose partial sums are exact in any order (the known-answer cases).

``rope`` restates isoexec/ops/rope/rope_fused.py:66-108 (rotate-half, three bf16 rounds) and is
bit-exact.

Pinned by tests/test_oracle_attention.py: against a float64 softmax attention, against closed forms
(one key, equal scores, a dominant key), by block-size independence of the exact-arithmetic cases,
and, for rope, against rotation identities (norm preservation, position 0 is the identity, angle
addition) and hand-computed vectors.
"""

from __future__ import annotations

import numpy as np

from .prims import DEFAULT, LOG2E, Prims, pairwise_tree, round_bf16

F32 = np.float32
BLOCK = 32
LAZY = F32(8.0)


def _half_of(key_in_block: np.ndarray) -> np.ndarray:
    """Which half-wave holds a key of a block: keys (k % 8) < 4 sit in half 0."""
    return (key_in_block % 8) // 4


def attend_one(q, K, V, scale, prims: Prims = DEFAULT, block: int = BLOCK):
    """One query ``q [D]`` over keys ``K [L, D]`` / values ``V [L, D]`` (all of them visible).
    Returns ``o [D]`` as fp32 holding bf16 values."""
    L, D = K.shape
    m = F32(-np.inf)
    l = [F32(0.0), F32(0.0)]  # one share of the denominator per half-wave
    O = np.zeros(D, dtype=F32)
    q64 = q.astype(np.float64)
    c = F32(F32(scale) * LOG2E)  # scale > 0: the running maximum is kept in unscaled units
    for b0 in range(0, L, block):
        kb, vb = K[b0 : b0 + block], V[b0 : b0 + block]
        n = kb.shape[0]
        s = (kb.astype(np.float64) @ q64).astype(F32)
        bm = F32(s.max())
        # the reference point moves only when the block maximum exceeds it by more than 2^8 (in the exponent)
        with np.errstate(invalid="ignore"):
            m_new = bm if F32(F32(bm - m) * c) > LAZY else m
        alpha = prims.exp2(np.array([F32(m - m_new) * c], dtype=F32))[0] if np.isfinite(m) else F32(0.0)
        mc = F32(m_new * c)
        p = np.zeros(block, dtype=F32)
        # fused multiply-add: the product is exact in float64, the difference is rounded once more there
        # (a double rounding that moves the fp32 result by at most one ulp in rare cases)
        p[:n] = prims.exp2((s.astype(np.float64) * np.float64(c) - np.float64(mc)).astype(F32))
        # Row sum: each half-wave adds its 16 keys as two 8-trees, then half 0 + half 1.
        idx = np.arange(block)
        halves = []
        for hf in (0, 1):
            mine = p[_half_of(idx) == hf]  # ascending key order = register order
            acc = F32(pairwise_tree(mine[:8][None, :])[0])
            for c0 in range(8, len(mine), 8):
                acc = F32(acc + F32(pairwise_tree(mine[c0 : c0 + 8][None, :])[0]))
            halves.append(acc)
        l = [F32(F32(l[hf] * alpha) + halves[hf]) for hf in (0, 1)]
        pv = (round_bf16(p[:n]).astype(np.float64) @ vb.astype(np.float64)).astype(F32)
        O = ((O * alpha).astype(F32) + pv).astype(F32)
        m = F32(m_new)
    return round_bf16((O * F32(F32(1.0) / F32(l[0] + l[1]))).astype(F32))


def attend_causal(q, k, v, scale=None, q_pos0: int = 0, prims: Prims = DEFAULT, block: int = BLOCK):
    """One sequence. ``q [Tq, HQ, D]``; ``k, v [q_pos0 + Tq, HKV, D]``; query t sits at absolute
    position ``q_pos0 + t`` and sees keys ``0 .. q_pos0 + t``. Returns ``o [Tq, HQ, D]``."""
    Tq, HQ, D = q.shape
    HKV = k.shape[1]
    group = HQ // HKV
    scale = D ** -0.5 if scale is None else scale
    out = np.zeros((Tq, HQ, D), dtype=F32)
    for t in range(Tq):
        n = q_pos0 + t + 1
        for h in range(HQ):
            g = h // group
            out[t, h] = attend_one(q[t, h], k[:n, g], v[:n, g], scale, prims, block)
    return out


def attend_fp64(q, k, v, scale=None, q_pos0: int = 0):
    """Textbook softmax attention in float64: the independent reference."""
    Tq, HQ, D = q.shape
    HKV = k.shape[1]
    group = HQ // HKV
    scale = D ** -0.5 if scale is None else scale
    q, k, v = q.astype(np.float64), k.astype(np.float64), v.astype(np.float64)
    out = np.zeros((Tq, HQ, D))
    for h in range(HQ):
        g = h // group
        s = q[:, h] @ k[:, g].T * scale
        mask = np.arange(k.shape[0])[None, :] > (q_pos0 + np.arange(Tq))[:, None]
        s[mask] = -np.inf
        s -= s.max(axis=1, keepdims=True)
        p = np.exp(s)
        out[:, h] = (p / p.sum(axis=1, keepdims=True)) @ v[:, g]
    return out


def rope_tables(max_positions: int, rotary_dim: int, theta: float = 1.0e6):
    """cos/sin ``[max_positions, R]`` holding bf16 values: float64 trigonometry of
    ``p * theta ** (-2 (d mod R/2) / R)``, rounded to fp32 then bf16."""
    half = rotary_dim // 2
    inv = 1.0 / (float(theta) ** (np.arange(half, dtype=np.float64) * 2.0 / rotary_dim))
    ang = np.arange(max_positions, dtype=np.float64)[:, None] * inv[None, :]
    ang = np.concatenate([ang, ang], axis=1)
    return round_bf16(np.cos(ang).astype(F32)), round_bf16(np.sin(ang).astype(F32))


def rope(x, cos, sin, positions):
    """``x [T, heads, D]`` (bf16 values), ``cos/sin [P, R]``: rotate the first R lanes of every head."""
    x = x.astype(F32)
    R = cos.shape[1]
    half = R // 2
    c = cos[positions][:, None, :].astype(F32)
    s = sin[positions][:, None, :].astype(F32)
    head = x[..., :R]
    rot = np.concatenate([(head[..., half:] * F32(-1.0)).astype(F32), head[..., :half]], axis=-1)
    y = round_bf16((round_bf16((head * c).astype(F32)) + round_bf16((rot * s).astype(F32))).astype(F32))
    return np.concatenate([y, x[..., R:]], axis=-1)
