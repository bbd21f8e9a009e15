"""GPU parity of the attention and rope kernels.

Attention's two matrix products run on the matrix cores, whose internal summation order is not
public, so the oracle comparison on random inputs carries a tolerance (stated below), exactly as for
the dense GEMM. What is bit-exact: inputs whose partial sums are exact in any order (known answers),
and every invariance -- a query's bits do not depend on the other queries, on how the sequence was cut
into calls, or on where its keys live.
"""

import numpy as np
import pytest
import torch

from _util import DevicePrims, bf16_to_np, cpu_gen, np_bits, np_to_bf16, same_bits
from oracle import attention as o_attn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
D = 128


@pytest.fixture(scope="module")
def dprims():
    return DevicePrims(DEV)


def attn(q, k, v, lens, **kw):
    from isoexec_amd.ops.attention.varlen_attn import varlen_attention

    cu = torch.tensor(np.cumsum([0] + list(lens)), dtype=torch.int32, device=DEV)
    return varlen_attention(q, k, v, cu, max(lens), **kw)


def rand_qkv(T, HQ, HKV, seed):
    g = cpu_gen(seed)
    mk = lambda h: torch.randn(T, h, D, generator=g).to(torch.bfloat16)
    return mk(HQ), mk(HKV), mk(HKV)


@pytest.mark.parametrize("HQ,HKV", [(8, 1), (4, 4), (32, 4), (2, 1), (16, 1)])
def test_known_answers_are_bit_exact(HQ, HKV, dprims):
    """Scores are small integers with the maximum at key 0, values are small integers: every partial
    sum is exact in any order, so kernel and oracle must agree on every bit. Pins the causal mask, the
    head grouping, the key order of the value product and the denominator's summation order."""
    lens = [1, 2, 31, 32, 33, 64]
    T = sum(lens)
    rng = np.random.default_rng(HQ * 10 + HKV)
    group = HQ // HKV
    q = np.zeros((T, HQ, D), np.float32)
    k = np.zeros((T, HKV, D), np.float32)
    for h in range(HQ):
        q[:, h, (7 * h) % D] = 8.0  # head h reads lane 7h of its key head
    v = rng.integers(-4, 5, size=(T, HKV, D)).astype(np.float32)
    start = 0
    for n in lens:
        for g in range(HKV):
            for h in range(g * group, (g + 1) * group):
                k[start : start + n, g, (7 * h) % D] = -rng.integers(0, 5, size=n)
                k[start, g, (7 * h) % D] = 0  # key 0 holds the maximum
        start += n
    got = attn(np_to_bf16(q, DEV), np_to_bf16(k, DEV), np_to_bf16(v, DEV), lens, scale=0.125)
    start = 0
    for n in lens:
        sl = slice(start, start + n)
        want = o_attn.attend_causal(q[sl], k[sl], v[sl], scale=0.125, prims=dprims)
        assert np.array_equal(np_bits(bf16_to_np(got[sl])), np_bits(want)), n
        start += n


def test_growing_maximum_known_answers_are_bit_exact(dprims):
    """scale = float32(ln 2) makes the exponent factor exactly 1, so integer scores give probabilities
    that are exact powers of two; with values in {-1, 0, 1} every partial sum stays exact in any order.
    The scores grow along the keys so that the reference point is moved (a rise of 10 and of 9), is
    left alone (a rise of 6, and of exactly 8, the boundary), and probabilities above 1 (up to 2^8)
    enter the value product and the denominator."""
    HQ, HKV = 8, 1
    lens = [130, 45]
    T = sum(lens)
    rng = np.random.default_rng(77)
    q = np.zeros((T, HQ, D), np.float32)
    k = np.zeros((T, HKV, D), np.float32)
    v = rng.integers(-1, 2, size=(T, HKV, D)).astype(np.float32)
    for h in range(HQ):
        q[:, h, 7 * h] = 1.0
    start = 0
    for n in lens:
        for h in range(HQ):
            s = np.zeros(n)
            j = np.arange(n)
            blk1 = (j > 40) & (j < 64)
            s[blk1] = rng.integers(4, 11, size=blk1.sum())
            s[40:41] = 10  # rise of 10 over the reference 0: moved
            blk2 = (j >= 64) & (j < 96)
            s[blk2] = rng.integers(6, 11, size=blk2.sum())
            if n > 70:
                s[70] = 16  # rise of 6: not moved, probability 2^6
            blk3 = (j >= 96) & (j < 128)
            s[blk3] = rng.integers(10, 14, size=blk3.sum())
            if n > 120:
                s[[100, 120]] = 18  # rise of exactly 8: not moved, probability 2^8
            if n > 128:
                s[128:] = 19  # rise of 9: moved
            k[start : start + n, 0, 7 * h] = s
        start += n
    scale = float(np.float32(np.log(2.0)))
    assert np.float32(scale) * np.float32(1.44269504088896340736) == np.float32(1.0)
    got = attn(np_to_bf16(q, DEV), np_to_bf16(k, DEV), np_to_bf16(v, DEV), lens, scale=scale)
    start = 0
    for n in lens:
        sl = slice(start, start + n)
        want = o_attn.attend_causal(q[sl], k[sl], v[sl], scale=scale, prims=dprims)
        assert np.array_equal(np_bits(bf16_to_np(got[sl])), np_bits(want)), n
        start += n


def test_random_inputs_within_tolerance_of_oracle_and_float64(dprims):
    """Config-4 head layout (32 query heads, 4 key/value heads, d 128). Tolerance: 2^-7 of the
    output scale against the oracle (one bf16 ulp where an fp32 sum lands near a rounding boundary),
    2^-6 against float64 softmax attention."""
    lens = [150, 37]
    T = sum(lens)
    q, k, v = rand_qkv(T, 32, 4, seed=1)
    got = bf16_to_np(attn(q.to(DEV), k.to(DEV), v.to(DEV), lens))
    start = 0
    for n in lens:
        sl = slice(start, start + n)
        f = lambda t: bf16_to_np(t[sl])
        want = o_attn.attend_causal(f(q), f(k), f(v), prims=dprims)
        truth = o_attn.attend_fp64(f(q), f(k), f(v))
        scale = np.abs(truth).max()
        assert np.abs(got[sl] - want).max() <= 2.0 ** -7 * scale
        assert (got[sl] != want).mean() < 0.05
        assert np.abs(got[sl] - truth).max() <= 2.0 ** -6 * scale
        start += n


def test_a_querys_bits_do_not_depend_on_the_call_shape():
    """One sequence of 300 tokens, config-4 heads: the packed full pass, the same sequence among
    others, a chunked prefill, and prefill followed by one-token decode steps out of a KV cache."""
    from isoexec_amd.ops.attention.varlen_attn import KVCache, varlen_attention

    T, HQ, HKV = 300, 32, 4
    q, k, v = (t.to(DEV) for t in rand_qkv(T, HQ, HKV, seed=2))
    full = attn(q, k, v, [T])
    # among other sequences, at another place in the pack
    qo, ko, vo = (t.to(DEV) for t in rand_qkv(77, HQ, HKV, seed=3))
    mixed = attn(torch.cat([qo, q, qo[:5]]), torch.cat([ko, k, ko[:5]]), torch.cat([vo, v, vo[:5]]), [77, T, 5])
    assert same_bits(mixed[77 : 77 + T], full)
    # strided inputs: q, k, v as slices of one projection buffer
    buf = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], dim=1)
    qs = buf[:, : HQ * D].unflatten(1, (HQ, D))
    ks = buf[:, HQ * D : (HQ + HKV) * D].unflatten(1, (HKV, D))
    vs = buf[:, (HQ + HKV) * D :].unflatten(1, (HKV, D))
    assert same_bits(attn(qs, ks, vs, [T]), full)
    # chunked prefill and decode against a cache whose rows are not where the packed keys were
    cache = KVCache(rows=3, max_len=512, num_kv_heads=HKV, device=DEV)
    row = 2
    kf, vf = cache.flat()
    kv_start = torch.tensor([row * cache.max_len], dtype=torch.int64, device=DEV)
    done = 0
    for n in (64, 1, 100, 35):  # chunks of a chunked prefill
        idx = torch.arange(done, done + n, device=DEV) + row * cache.max_len
        cache.write(idx, k[done : done + n], v[done : done + n])
        cu = torch.tensor([0, n], dtype=torch.int32, device=DEV)
        pos0 = torch.tensor([done], dtype=torch.int32, device=DEV)
        o = varlen_attention(q[done : done + n], kf, vf, cu, n, kv_start=kv_start, q_pos0=pos0)
        assert same_bits(o, full[done : done + n]), (done, n)
        done += n
    cu1 = torch.tensor([0, 1], dtype=torch.int32, device=DEV)
    for t in range(done, T):  # one-token decode steps
        cache.write(torch.tensor([row * cache.max_len + t], device=DEV), k[t : t + 1], v[t : t + 1])
        o = varlen_attention(q[t : t + 1], kf, vf, cu1, 1, kv_start=kv_start, q_pos0=torch.tensor([t], dtype=torch.int32, device=DEV))
        assert same_bits(o, full[t : t + 1]), t


def test_batched_decode_with_null_lanes():
    """A decode batch: three live sequences at different context lengths and two padded lanes."""
    from isoexec_amd.ops.attention.varlen_attn import KVCache, varlen_attention

    HQ, HKV = 32, 4
    lens = [40, 129, 7]
    cache = KVCache(rows=4, max_len=256, num_kv_heads=HKV, device=DEV)
    kf, vf = cache.flat()
    fulls, qs = [], []
    for i, n in enumerate(lens):
        q, k, v = (t.to(DEV) for t in rand_qkv(n, HQ, HKV, seed=10 + i))
        cache.write(torch.arange(n, device=DEV) + (i + 1) * cache.max_len, k, v)
        fulls.append(attn(q, k, v, [n]))
        qs.append(q)
    junk = torch.randn(1, HQ, D, device=DEV).to(torch.bfloat16)
    qd = torch.cat([qs[0][-1:], junk, qs[1][-1:], qs[2][-1:], junk])
    kv_start = torch.tensor([1, 0, 2, 3, 0], dtype=torch.int64, device=DEV) * cache.max_len
    pos0 = torch.tensor([lens[0] - 1, -1, lens[1] - 1, lens[2] - 1, -1], dtype=torch.int32, device=DEV)
    cu = torch.arange(6, dtype=torch.int32, device=DEV)
    o = varlen_attention(qd, kf, vf, cu, 1, kv_start=kv_start, q_pos0=pos0)
    assert same_bits(o[0:1], fulls[0][-1:]) and same_bits(o[2:3], fulls[1][-1:]) and same_bits(o[3:4], fulls[2][-1:])
    assert not o[1].any() and not o[4].any()


def test_argument_checks():
    from isoexec_amd.ops.attention.varlen_attn import varlen_attention

    q, k, v = (t.to(DEV) for t in rand_qkv(8, 4, 2, seed=5))
    cu = torch.tensor([0, 8], dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="bf16 only"):
        varlen_attention(q.float(), k, v, cu, 8)
    with pytest.raises(RuntimeError, match="declined"):
        varlen_attention(q[..., :64].contiguous(), k[..., :64].contiguous(), v[..., :64].contiguous(), cu, 8)
    with pytest.raises(RuntimeError, match="declined"):
        varlen_attention(torch.cat([q, q[:, :2]], 1), k, v, cu, 8)  # 6 query heads over 2: group 3
    with pytest.raises(RuntimeError, match="int32"):
        varlen_attention(q, k, v, cu.long(), 8)
    for bad in (0.0, -0.125, float("inf"), float("nan")):  # the reference point lives on the unscaled scores
        with pytest.raises(RuntimeError):
            varlen_attention(q, k, v, cu, 8, scale=bad)
    empty = varlen_attention(q[:0], k, v, torch.zeros(1, dtype=torch.int32, device=DEV), 0)
    assert empty.shape == (0, 4, D)


def test_rope_bit_exact_in_place_on_a_strided_slice():
    from isoexec_amd.ops.rope.rope_hip import apply_rope_, rope_tables

    T, HQ, HKV, R = 50, 6, 2, 64
    g = cpu_gen(6)
    buf = torch.randn(T, (HQ + 2 * HKV) * D, generator=g).to(torch.bfloat16)
    buf[3, :D] = torch.tensor([0.0, -0.0] * (D // 2)).to(torch.bfloat16)  # signed zeros travel through
    pos = torch.randint(0, 4000, (T,), generator=g, dtype=torch.int32)
    cos_d, sin_d = rope_tables(4096, R, 1e6, device=DEV)
    cos_o, sin_o = o_attn.rope_tables(4096, R, 1e6)
    assert np.array_equal(np_bits(bf16_to_np(cos_d)), np_bits(cos_o)) and np.array_equal(np_bits(bf16_to_np(sin_d)), np_bits(sin_o))
    dbuf = buf.to(DEV)
    qv = dbuf[:, : HQ * D].unflatten(1, (HQ, D))
    kv = dbuf[:, HQ * D : (HQ + HKV) * D].unflatten(1, (HKV, D))
    apply_rope_(qv, cos_d, sin_d, pos.to(DEV))
    apply_rope_(kv, cos_d, sin_d, pos.to(DEV))
    host = bf16_to_np(buf)
    want_q = o_attn.rope(host[:, : HQ * D].reshape(T, HQ, D), cos_o, sin_o, pos.numpy())
    want_k = o_attn.rope(host[:, HQ * D : (HQ + HKV) * D].reshape(T, HKV, D), cos_o, sin_o, pos.numpy())
    got = bf16_to_np(dbuf)
    assert np.array_equal(np_bits(got[:, : HQ * D].reshape(T, HQ, D)), np_bits(want_q))
    assert np.array_equal(np_bits(got[:, HQ * D : (HQ + HKV) * D].reshape(T, HKV, D)), np_bits(want_k))
    assert np.array_equal(np_bits(got[:, (HQ + HKV) * D :]), np_bits(host[:, (HQ + HKV) * D :]))  # v untouched
    # full rotary width, and a row's bits do not depend on the other rows
    cos_f, sin_f = rope_tables(64, D, 1e4, device=DEV)
    x = torch.randn(9, 3, D, generator=g).to(torch.bfloat16).to(DEV)
    p = torch.arange(9, dtype=torch.int32, device=DEV)
    whole = apply_rope_(x.clone(), cos_f, sin_f, p)
    one = apply_rope_(x[4:5].clone(), cos_f, sin_f, p[4:5])
    assert same_bits(one, whole[4:5]) and same_bits(whole[0], x[0])


@pytest.mark.parametrize("R", [8, 40, 48, 128])
def test_rope_scalar_and_vector_kernels_give_the_oracle_bits(R):
    """R / 2 a multiple of 8 takes the kernel with 16-byte accesses (48, 128), any other even width the element kernel
    (8, 40): both are the oracle's expression element by element."""
    from isoexec_amd.ops.rope.rope_hip import apply_rope_, rope_tables

    g = cpu_gen(R)
    x = torch.randn(37, 5, 128, generator=g).to(torch.bfloat16)
    pos = torch.randint(0, 300, (37,), generator=g, dtype=torch.int32)
    cos, sin = rope_tables(300, R, 1e6, device=DEV)
    co, so = o_attn.rope_tables(300, R, 1e6)
    got = apply_rope_(x.clone().to(DEV), cos, sin, pos.to(DEV))
    want = o_attn.rope(bf16_to_np(x), co, so, pos.numpy())
    assert np.array_equal(np_bits(bf16_to_np(got)), np_bits(want))


def test_rope_vector_kernel_stores_the_element_kernels_bits_for_nans_and_infinities():
    """The 16-byte kernel rounds its products with the hardware convert and makes NaNs canonical at the store; the
    element kernel rounds with integer arithmetic throughout. Same values through both (a slice that starts 8 bytes
    into a row is not 16-byte aligned and takes the element kernel), NaNs with payloads and infinities included."""
    from isoexec_amd.ops.rope.rope_hip import apply_rope_, rope_tables

    g = cpu_gen(5)
    T, Hh, D = 33, 4, 128
    x = torch.randn(T, Hh * D, generator=g).to(torch.bfloat16)
    bits = x.view(torch.int16)
    bits[0, 3] = 0x7fa5
    bits[1, D + 70] = -1
    bits[2, 5] = 0x7f81
    x[3, 9] = float("inf")
    x[3, 9 + 64] = float("inf")
    x[4, 2 * D + 1] = float("-inf")
    x[5, :] = 3.0e38
    pos = torch.randint(0, 300, (T,), generator=g, dtype=torch.int32).to(DEV)
    cos, sin = rope_tables(300, D, 1e6, device=DEV)
    aligned = x.clone().to(DEV).view(T, Hh, D)
    wide = torch.zeros(T, Hh * D + 8, dtype=torch.bfloat16, device=DEV)
    wide[:, 4:4 + Hh * D] = x.to(DEV)
    shifted = wide[:, 4:4 + Hh * D].unflatten(1, (Hh, D))
    assert shifted.data_ptr() % 16 == 8
    a = apply_rope_(aligned, cos, sin, pos)
    b = apply_rope_(shifted, cos, sin, pos)
    assert not torch.isfinite(a.float()).all()
    assert torch.equal(a.contiguous().view(torch.int16), b.contiguous().view(torch.int16))


def test_rope_positions_outside_the_tables_read_nothing_and_give_nan():
    """The kernel bounds every position by the tables' row count: a position past the end (or negative) makes that
    token's rotated lanes NaN instead of reading beyond the tables; its neighbours are rotated as usual."""
    from isoexec_amd.ops.rope.rope_hip import apply_rope_, rope_tables
    from oracle import attention as o_attn

    g = cpu_gen(77)
    x = torch.randn(4, 3, 128, generator=g).to(torch.bfloat16)
    cos, sin = rope_tables(64, 128, 1e6, device=DEV)
    pos = torch.tensor([0, 63, 64, -1], dtype=torch.int32)
    got = apply_rope_(x.clone().to(DEV), cos, sin, pos.to(DEV)).float().cpu().numpy()
    co, so = o_attn.rope_tables(64, 128, 1e6)
    want = o_attn.rope(x[:2].float().numpy(), co, so, pos[:2].numpy())
    assert np.array_equal(got[:2], want)
    assert np.isnan(got[2:]).all()
