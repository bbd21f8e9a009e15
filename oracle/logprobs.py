"""Oracle: row-invariant log-softmax + target gather (reference ops/logprobs/rowinv.py:136-245,547-570).

Pinned by (tests/test_oracle_dense.py): fp64 ``x_t - logsumexp(x)`` truth on random and
adversarial rows (the reference's own probe, rowinv_gpu.py:112-131 and tolerance rowinv.py:21-22);
the closed form for a constant row (S == V exactly); ``combine_order`` against the schedule the
reference documents for G=8 (pik/plan.py:104-119); invariance to row count and to which rows
share a call; a brute-force scalar evaluation of the same tree on tiny V.
"""

from __future__ import annotations

import numpy as np

from .prims import DEFAULT, F32, Prims, pairwise_tree

BLOCK = 4096  # rowinv.py:23


def combine_order(g: int) -> list[tuple[int, int, int]]:
    """Balanced in-place fold schedule ``(dst, lhs, rhs)`` over G leaves (pik/plan.py:104-119)."""
    order = []
    s = 1
    while s < g:
        for i in range(0, g - s, 2 * s):
            order.append((i, i, i + s))
        s *= 2
    return order


def block_sum(terms: np.ndarray) -> np.ndarray:
    """``terms [..., 4096]`` (masked columns already 0): 512 column sums over the 8 chunks left to
    right, then the adjacent-pairwise tree over the 512 columns."""
    t = terms.astype(F32).reshape(*terms.shape[:-1], 8, 512)
    cols = np.zeros(t.shape[:-2] + (512,), dtype=F32)
    for c in range(8):
        cols = (cols + t[..., c, :]).astype(F32)
    return pairwise_tree(cols)


def leaf_sums(x: np.ndarray, row_max: np.ndarray, g: int, prims: Prims = DEFAULT) -> np.ndarray:
    """``[rows, G]`` Kahan-fp32 leaf sums of ``exp(x - m)`` (rowinv.py:136-154)."""
    rows, vocab = x.shape
    L = vocab // g
    out = np.zeros((rows, g), dtype=F32)
    xf = x.astype(F32)
    m = row_max.astype(F32)[:, None]
    for leaf in range(g):
        acc = np.zeros(rows, dtype=F32)
        comp = np.zeros(rows, dtype=F32)
        for off in range(0, L, BLOCK):
            n = min(BLOCK, L - off)
            seg = xf[:, leaf * L + off : leaf * L + off + n]
            terms = np.zeros((rows, BLOCK), dtype=F32)
            terms[:, :n] = prims.exp_fast((seg - m).astype(F32))
            bs = block_sum(terms)
            y = (bs - comp).astype(F32)
            t = (acc + y).astype(F32)
            comp = ((t - acc).astype(F32) - y).astype(F32)
            acc = t
        out[:, leaf] = acc
    return out


def fold_leaves(leaf: np.ndarray) -> np.ndarray:
    slots = [leaf[:, i].astype(F32) for i in range(leaf.shape[1])]
    for dst, lhs, rhs in combine_order(leaf.shape[1]):
        slots[dst] = (slots[lhs] + slots[rhs]).astype(F32)
    return slots[0]


def rowinv_sampled(x: np.ndarray, target: np.ndarray, g: int = 8, prims: Prims = DEFAULT):
    """Returns ``(logprob [rows], lse [rows])`` fp32. ``x`` holds fp32 values (bf16 logits widened)."""
    x = x.astype(F32)
    rows, vocab = x.shape
    if vocab % g:
        raise ValueError("V must be divisible by G (rowinv.py:376-377)")
    m = x.max(axis=1).astype(F32)
    s = fold_leaves(leaf_sums(x, m, g, prims))
    log_s = prims.log(s)
    valid = (target >= 0) & (target < vocab)
    safe = np.where(valid, target, 0)
    sampled = x[np.arange(rows), safe]
    out = np.where(valid, ((sampled - m).astype(F32) - log_s).astype(F32), F32(0.0)).astype(F32)
    return out, (m + log_s).astype(F32)


def rowinv_full(x: np.ndarray, g: int = 8, prims: Prims = DEFAULT) -> np.ndarray:
    """``[rows, V]`` fp32 ``(x - m) - log S`` (rowinv.py:193-245)."""
    x = x.astype(F32)
    m = x.max(axis=1).astype(F32)
    log_s = prims.log(fold_leaves(leaf_sums(x, m, g, prims)))
    return ((x - m[:, None]).astype(F32) - log_s[:, None]).astype(F32)


def truth_fp64(x: np.ndarray, target: np.ndarray) -> np.ndarray:
    """Textbook ``x_t - logsumexp(x)`` in float64: the independent reference."""
    x = x.astype(np.float64)
    m = x.max(axis=1, keepdims=True)
    lse = m[:, 0] + np.log(np.exp(x - m).sum(axis=1))
    return x[np.arange(x.shape[0]), target] - lse
