"""Pins the attention and rotary-embedding restatements (CPU only).

Attention: against textbook float64 softmax attention, and on closed forms that a dropped rescale,
a wrong mask edge or a mis-grouped head would break. Rope: rotation identities and a hand vector.
"""

import numpy as np
import pytest

from oracle import attention as A
from oracle.prims import round_bf16


def bf(a):
    return round_bf16(np.asarray(a, dtype=np.float32))


def random_case(T, HQ, HKV, D, seed, q_pos0=0):
    rng = np.random.default_rng(seed)
    return (bf(rng.standard_normal((T, HQ, D))), bf(rng.standard_normal((q_pos0 + T, HKV, D))),
            bf(rng.standard_normal((q_pos0 + T, HKV, D))))


@pytest.mark.parametrize("T,HQ,HKV,q_pos0", [(70, 4, 2, 0), (5, 8, 1, 61), (33, 2, 2, 31)])
def test_matches_float64_softmax_attention(T, HQ, HKV, q_pos0):
    q, k, v = random_case(T, HQ, HKV, 64, seed=T, q_pos0=q_pos0)
    got = A.attend_causal(q, k, v, q_pos0=q_pos0)
    want = A.attend_fp64(q, k, v, q_pos0=q_pos0)
    assert np.abs(got - want).max() <= 2.0 ** -8 * max(1.0, np.abs(want).max())
    assert np.array_equal(got, bf(got))  # outputs are bf16 values


def test_block_size_changes_only_rounding():
    q, k, v = random_case(80, 2, 1, 32, seed=9)
    a = A.attend_causal(q, k, v, block=32)
    b = A.attend_causal(q, k, v, block=16)
    assert np.abs(a - b).max() <= 2.0 ** -7 and (a != b).mean() < 0.2


def test_single_key_returns_its_value_exactly():
    q, k, v = random_case(1, 4, 2, 64, seed=1)
    got = A.attend_causal(q, k, v)
    assert np.array_equal(got[0, :2], np.stack([v[0, 0]] * 2)) and np.array_equal(got[0, 2:], np.stack([v[0, 1]] * 2))


def test_zero_query_averages_the_visible_values():
    T, D = 45, 32
    rng = np.random.default_rng(2)
    v = bf(rng.integers(-8, 9, size=(T, 1, D)))
    q = np.zeros((T, 1, D), np.float32)
    k = bf(rng.standard_normal((T, 1, D)))
    got = A.attend_causal(q, k, v)
    for t in (0, 1, 31, 32, 44):
        mean = v[: t + 1, 0].astype(np.float64).mean(axis=0)
        assert np.abs(got[t, 0] - mean).max() <= 2.0 ** -8 * 8
    # Causality: changing a later key or value leaves earlier queries untouched.
    k2, v2 = k.copy(), v.copy()
    k2[40:], v2[40:] = 3.0, -5.0
    again = A.attend_causal(q + 1.0, k2, v2)
    base = A.attend_causal(q + 1.0, k, v)
    assert np.array_equal(again[:40], base[:40]) and not np.array_equal(again[40:], base[40:])


def test_dominant_key_in_a_late_block_wins_after_rescaling():
    """A key whose score exceeds the rest by 60 sits in the third block: every earlier accumulator is
    rescaled to nothing, so the output is that key's value. A dropped rescale fails this."""
    T, D = 90, 32
    rng = np.random.default_rng(3)
    q = np.zeros((1, 1, D), np.float32)
    q[0, 0, 0] = 8.0
    k = np.zeros((T, 1, D), np.float32)
    k[70, 0, 0] = 60.0 / 8.0 * (D ** 0.5)
    v = bf(rng.standard_normal((T, 1, D)))
    got = A.attend_causal(q, k, v, q_pos0=T - 1)
    assert np.abs(got[0, 0] - v[70, 0]).max() <= 2.0 ** -8 * np.abs(v[70, 0]).max() + 1e-6


def test_query_heads_share_the_right_key_head():
    q, k, v = random_case(20, 8, 2, 32, seed=4)
    full = A.attend_causal(q, k, v)
    for h in range(8):
        alone = A.attend_causal(q[:, h : h + 1], k[:, h // 4 : h // 4 + 1], v[:, h // 4 : h // 4 + 1])
        assert np.array_equal(full[:, h], alone[:, 0])


def test_context_offset_equals_the_tail_of_a_full_pass():
    q, k, v = random_case(50, 2, 1, 32, seed=5)
    full = A.attend_causal(q, k, v)
    tail = A.attend_causal(q[37:], k, v, q_pos0=37)
    assert np.array_equal(tail, full[37:])


# ------------------------------------------------------------------ rope


def test_rope_tables_and_hand_vector():
    cos, sin = A.rope_tables(4, 4, theta=100.0)
    # R = 4: inverse frequencies 1 and 0.1; lanes (0, 2) share the first, (1, 3) the second.
    assert np.array_equal(cos[0], np.ones(4, np.float32)) and np.array_equal(sin[0], np.zeros(4, np.float32))
    assert cos[2, 0] == bf(np.cos(2.0)) and cos[2, 2] == cos[2, 0] and sin[3, 1] == bf(np.sin(0.3)) and sin[3, 3] == sin[3, 1]
    x = bf(np.array([[[1.0, 2.0, 3.0, 4.0, 7.0]]]))
    y = A.rope(x, cos, sin, np.array([2]))
    c0, s0, c1, s1 = cos[2, 0], sin[2, 0], cos[2, 1], sin[2, 1]
    want = [bf(bf(1 * c0) + bf(-3 * s0)), bf(bf(2 * c1) + bf(-4 * s1)), bf(bf(3 * c0) + bf(1 * s0)), bf(bf(4 * c1) + bf(2 * s1)), 7.0]
    assert np.array_equal(y[0, 0], np.array([float(np.asarray(w).reshape(-1)[0]) for w in want], np.float32))


def test_rope_is_a_rotation():
    rng = np.random.default_rng(6)
    cos, sin = A.rope_tables(512, 64, theta=1e6)
    x = bf(rng.standard_normal((6, 3, 80)))
    pos = np.array([0, 1, 7, 100, 300, 511])
    y = A.rope(x, cos, sin, pos)
    assert np.array_equal(y[0], x[0])  # position 0 is the identity
    assert np.array_equal(y[..., 64:], x[..., 64:])  # lanes past R are copied
    n0 = np.linalg.norm(x[..., :64].astype(np.float64), axis=-1)
    n1 = np.linalg.norm(y[..., :64].astype(np.float64), axis=-1)
    assert np.abs(n1 / n0 - 1).max() < 2.0 ** -6
    # Relative-position property: <rope(a, p), rope(b, p')> depends on p - p' (to bf16 accuracy).
    a, b = bf(rng.standard_normal((1, 1, 64))), bf(rng.standard_normal((1, 1, 64)))
    dots = []
    for p in (5, 105, 405):
        ra, rb = A.rope(a, cos, sin, np.array([p + 20])), A.rope(b, cos, sin, np.array([p]))
        dots.append(float((ra.astype(np.float64) * rb.astype(np.float64)).sum()))
    assert max(dots) - min(dots) < 0.25 and abs(dots[0]) > 0.01
    # The sign convention: lane d mixes with lane d + R/2, negated on the low side.
    e = np.zeros((1, 1, 64), np.float32)
    e[0, 0, 40] = 1.0  # lane 8 of the upper half
    r = A.rope(e, cos, sin, np.array([3]))
    assert r[0, 0, 8] == bf(-sin[3, 8]) and r[0, 0, 40] == cos[3, 40] and np.count_nonzero(r) == 2
