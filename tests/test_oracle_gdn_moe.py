"""CPU: pins for the oracle's GatedDeltaNet and MoE restatements (config 0 runs here in full)."""

import numpy as np
import torch

from oracle import gdn as o_gdn
from oracle import moe as o_moe
from oracle import prims as o_prims


def config0(seed=0, B=2, T=256, H=4, K=64, V=64):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, T, H, K, generator=g)
    k = torch.randn(B, T, H, K, generator=g)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6)
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    v = torch.randn(B, T, H, V, generator=g)
    beta = torch.sigmoid(torch.randn(B, T, H, generator=g))
    gate = -torch.nn.functional.softplus(torch.randn(B, T, H, generator=g))
    return [t.numpy() for t in (q, k, v, gate, beta)]


def test_config0_scan_against_fp64_recurrence_and_chunked_form():
    q, k, v, g, beta = config0()
    for b in range(2):
        st = np.zeros((4, 64, 64), np.float32)
        o = o_gdn.scan(q[b], k[b], v[b], g[b], beta[b], st)
        o64, s64 = o_gdn.scan_fp64(q[b], k[b], v[b], g[b], beta[b])
        assert np.abs(o - o64).max() <= 5e-6 and np.abs(st - s64).max() <= 5e-6
        for chunk in (16, 32, 64):  # the chunked WY algorithm of gdn_ops.py:261-315 in float64
            assert np.abs(o_gdn.chunk_fp64(q[b], k[b], v[b], g[b], beta[b], chunk) - o64).max() <= 1e-10


def test_config0_prefill_decode_splits_are_bitwise_equal():
    q, k, v, g, beta = config0()
    b = 1
    st = np.zeros((4, 64, 64), np.float32)
    whole = o_gdn.scan(q[b], k[b], v[b], g[b], beta[b], st)
    for split in (0, 1, 63, 64, 65, 127, 255):
        s2 = np.zeros((4, 64, 64), np.float32)
        parts = []
        if split:
            parts.append(o_gdn.scan(q[b, :split], k[b, :split], v[b, :split], g[b, :split], beta[b, :split], s2))
        for t in range(split, 256):
            parts.append(o_gdn.scan(q[b, t:t + 1], k[b, t:t + 1], v[b, t:t + 1], g[b, t:t + 1], beta[b, t:t + 1], s2))
        got = np.concatenate(parts)
        assert np.array_equal(got.view(np.uint32), whole.view(np.uint32))
        assert np.array_equal(s2.view(np.uint32), st.view(np.uint32))


def test_scan_closed_forms_and_gqa():
    T, K, V = 32, 64, 16
    k = np.eye(K, dtype=np.float32)[:T].reshape(T, 1, K)
    q = k * np.float32(K ** 0.5)
    rng = np.random.default_rng(1)
    v = rng.standard_normal((T, 1, V)).astype(np.float32)
    zeros, ones = np.zeros((T, 1), np.float32), np.ones((T, 1), np.float32)
    st = np.zeros((1, V, K), np.float32)
    assert np.array_equal(o_gdn.scan(q, k, v, zeros, ones, st), v)  # associative recall
    s0 = rng.standard_normal((1, V, K)).astype(np.float32)
    st = s0.copy()
    gg = -rng.random((T, 1)).astype(np.float32)
    o_gdn.scan(q, k, v, gg, zeros, st)  # beta = 0: pure decay
    assert np.abs(st - s0 * np.exp(gg.astype(np.float64).sum())).max() <= 1e-5
    # GQA: 2 value heads per key head == the expanded form
    q2 = rng.standard_normal((T, 2, K)).astype(np.float32)
    k2 = o_gdn.l2norm(rng.standard_normal((T, 2, K)).astype(np.float32), io_bf16=False)
    v4 = rng.standard_normal((T, 4, V)).astype(np.float32)
    g4 = -rng.random((T, 4)).astype(np.float32)
    b4 = rng.random((T, 4)).astype(np.float32)
    sa, sb = np.zeros((4, V, K), np.float32), np.zeros((4, V, K), np.float32)
    oa = o_gdn.scan(q2, k2, v4, g4, b4, sa)
    ob = o_gdn.scan(np.repeat(q2, 2, axis=1), np.repeat(k2, 2, axis=1), v4, g4, b4, sb)
    assert np.array_equal(oa, ob) and np.array_equal(sa, sb)


def test_l2norm_gate_and_conv_against_eager_expressions():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(40, 3, 128, generator=g)
    want = (x * torch.rsqrt((x * x).sum(-1, keepdim=True) + 1e-6)).numpy()
    assert np.abs(o_gdn.l2norm(x.numpy(), io_bf16=False) - want).max() <= 2e-7
    a, b = torch.randn(40, 4, generator=g) * 3, torch.randn(40, 4, generator=g)
    a[0, 0] = 25.0
    A_log, dt_bias = 0.2 * torch.randn(4, generator=g), 0.2 * torch.randn(4, generator=g)
    gg, bb = o_gdn.gate_and_beta(a.numpy(), b.numpy(), A_log.numpy(), dt_bias.numpy(), io_bf16=False)
    want_g = -A_log.exp() * torch.nn.functional.softplus(a + dt_bias)  # gdn_ops.py:1208
    assert np.abs(gg - want_g.numpy()).max() <= 1e-6 * np.abs(want_g.numpy()).max()
    assert np.abs(bb - torch.sigmoid(b).numpy()).max() <= 2e-7
    # a bf16 parameter: the eager expression takes exp() in bf16 (torch on the CPU is the library routine here)
    A16 = A_log.to(torch.bfloat16)
    gg16, _ = o_gdn.gate_and_beta(a.numpy(), b.numpy(), A16.float().numpy(), dt_bias.numpy(), io_bf16=False,
                                  exp_bf16=True)
    want16 = -A16.exp() * torch.nn.functional.softplus(a.float() + dt_bias.float())
    assert want16.dtype is torch.float32
    assert np.abs(gg16 - want16.numpy()).max() <= 1e-6 * np.abs(want16.numpy()).max()
    widened = -A16.float().exp() * torch.nn.functional.softplus(a + dt_bias)     # NOT the same function
    assert np.abs(gg16 - widened.numpy()).max() > 1e-4 * np.abs(widened.numpy()).max()
    # conv: brute-force loop over (t, d, tap) in float64, and the split-anywhere property
    T, D, W = 19, 6, 4
    xx = torch.randn(T, D, generator=g).to(torch.bfloat16).float().numpy()
    w = torch.randn(D, W, generator=g).to(torch.bfloat16).float().numpy()
    bias = torch.randn(D, generator=g).to(torch.bfloat16).float().numpy()
    y, fs = o_gdn.causal_conv(xx, w, bias)
    for t in range(T):
        for d in range(D):
            acc = sum(float(w[d, i]) * (float(xx[t - (W - 1) + i, d]) if t - (W - 1) + i >= 0 else 0.0)
                      for i in range(W)) + float(bias[d])
            ref = acc / (1.0 + np.exp(-acc))
            assert abs(float(y[t, d]) - ref) <= 2.0 ** -7 * abs(ref) + 1e-6
    assert np.array_equal(fs, xx[T - 3:].T)
    y1, s1 = o_gdn.causal_conv(xx[:2], w, bias)
    y2, s2 = o_gdn.causal_conv(xx[2:], w, bias, initial_state=s1)
    assert np.array_equal(np.concatenate([y1, y2]), y) and np.array_equal(s2, fs)


def test_router_against_torch_topk_softmax_and_tie_rules():
    g = torch.Generator().manual_seed(3)
    lg = 2 * torch.randn(50, 128, generator=g)
    idx, p = o_moe.router_topk(lg.numpy(), 8, mode=0)
    tv, ti = torch.topk(lg, 8, dim=1)
    assert np.array_equal(idx, ti.numpy()) and np.abs(p - torch.softmax(tv, -1).numpy()).max() <= 2e-7
    idx, p = o_moe.router_topk(lg.numpy(), 8, mode=1)  # HF form: softmax, top-k, renormalise
    pr = torch.softmax(lg, -1)
    tv, ti = torch.topk(pr, 8, dim=1)
    assert np.array_equal(idx, ti.numpy()) and np.abs(p - (tv / tv.sum(-1, keepdim=True)).numpy()).max() <= 2e-7
    tie = np.zeros((1, 16), np.float32)
    tie[0, 9] = np.nan
    idx, p = o_moe.router_topk(tie, 4, mode=0)
    assert idx[0].tolist() == [0, 1, 2, 3] and np.allclose(p, 0.25)  # lowest index wins; NaN is -inf
    idx, _ = o_moe.router_topk(np.full((1, 8), np.nan, np.float32), 2, mode=0)
    assert idx[0].tolist() == [0, 1]


def test_permutation_against_stable_argsort_and_combine_loop():
    rng = np.random.default_rng(4)
    T, E, k = 97, 16, 4
    lg = rng.standard_normal((T, E)).astype(np.float32)
    idx, prob = o_moe.router_topk(lg, k)
    counts, st, pp, cr = o_moe.permute(idx, prob, E)
    dp, dm = o_moe.dense_from_topk(idx, prob, E)
    # ref_permute_index (moe_router_o2_kernel.py:389-397) on the dense tensors
    rt = torch.from_numpy(dm).T.contiguous()
    flat = rt.reshape(-1).to(torch.int8).argsort(descending=True, stable=True)[: T * k]
    assert np.array_equal(st, (flat % T).numpy())
    assert np.array_equal(pp, torch.from_numpy(dp).T.contiguous().reshape(-1)[flat].numpy())
    assert np.array_equal(counts, dm.sum(0))
    eo = o_prims.round_bf16(rng.standard_normal((T * k, 8)).astype(np.float32))
    got = o_moe.combine(eo, cr)
    for t in (0, 50, 96):
        rows = sorted((int(st_e), r) for r, st_e in enumerate(np.repeat(np.arange(E), counts)) if st[r] == t)
        acc = eo[rows[0][1]]
        for _, r in rows[1:]:
            acc = o_prims.round_bf16(acc + eo[r])
        assert np.array_equal(got[t], acc)


def test_expert_chain_against_brute_force():
    rng = np.random.default_rng(5)
    T, H, E, F, k = 12, 32, 4, 16, 2
    bf = lambda a: o_prims.round_bf16(a.astype(np.float32))
    x, w1, w2 = bf(rng.standard_normal((T, H))), bf(0.3 * rng.standard_normal((E, 2 * F, H))), \
        bf(0.3 * rng.standard_normal((E, H, F)))
    wr = bf(rng.standard_normal((E, H)))
    out = o_moe.moe_ffn(x, wr, w1, w2, k)
    lg = x @ wr.T
    for t in range(T):
        top = np.argsort(-lg[t], kind="stable")[:k]
        p = np.exp(lg[t, top] - lg[t, top].max())
        p = p / p.sum()
        acc = np.zeros(H)
        for e, pe in sorted(zip(top, p)):
            h = x[t].astype(np.float64) @ w1[e].astype(np.float64).T
            a = h[:F] / (1 + np.exp(-h[:F])) * h[F:] * pe
            acc += a @ w2[e].astype(np.float64).T
        assert np.abs(out[t] - acc).max() <= 0.03 * np.abs(acc).max() + 1e-3
    one = o_moe.moe_ffn(x[3:4], wr, w1, w2, k)
    assert np.array_equal(one[0], out[3])


# ---- the boundary (cpr) form: reference ops/gdn/gdn_cpr.py:104-186, :288-319 ------------------------------------

def _cpr_inputs(lens, seed, H=2, HV=4, K=32, V=16, slow_decay=True):
    """Packed inputs on the bf16 grid. ``slow_decay`` keeps the state alive over many chunks (|g| ~ 0.02 per token),
    so that an error made at one boundary is still there at the next ones."""
    g = torch.Generator().manual_seed(seed)
    T = sum(lens)
    bf = lambda t: t.to(torch.bfloat16).float().numpy()
    q = bf(torch.nn.functional.normalize(torch.randn(T, H, K, generator=g), dim=-1))
    k = bf(torch.nn.functional.normalize(torch.randn(T, H, K, generator=g), dim=-1))
    v = bf(torch.randn(T, HV, V, generator=g))
    gate = -torch.nn.functional.softplus(torch.randn(T, HV, generator=g))
    gate = (gate * (0.02 if slow_decay else 1.0)).numpy().astype(np.float32)
    beta = bf(torch.sigmoid(torch.randn(T, HV, generator=g)))
    return q, k, v, gate, beta


def _bf16_half_ulp(x):
    """Half a bf16 unit in the last place at the magnitude of (float64) x."""
    e = np.floor(np.log2(np.maximum(np.abs(x), 2.0 ** -126)))
    return 2.0 ** (e - 8)


def _restarted_chain_snapshots(q, k, v, g, beta, length, chunk, HV, V, K):
    """The mistake the snapshot test must catch: the chain continues from the ROUNDED snapshot."""
    chain = np.zeros((HV, V, K), np.float32)
    snaps = []
    for c0 in range(0, length, chunk):
        chain = o_prims.round_bf16(chain)
        snaps.append(chain.copy())
        sl = slice(c0, min(c0 + chunk, length))
        o_gdn.scan(q[sl], k[sl], v[sl], g[sl], beta[sl], chain)
    return snaps


def test_cpr_snapshots_are_the_rounded_fp64_boundary_states():
    lens, chunk = [200, 37, 0, 130], 16           # 13 + 3 + 0 + 9 chunks
    q, k, v, g, beta = _cpr_inputs(lens, 31)
    HV, V, K = v.shape[1], v.shape[2], k.shape[2]
    _, snaps, finals = o_gdn.cpr_forward(q, k, v, g, beta, lens, chunk)
    assert len(snaps) == sum(-(-n // chunk) for n in lens) and len(finals) == len(lens)
    pos, at = 0, 0
    for n, length in enumerate(lens):
        sl = slice(pos, pos + length)
        if length == 0:
            assert not finals[n].any()
            continue
        entering, final = o_gdn.chunk_states_fp64(k[sl], v[sl], g[sl], beta[sl], chunk)
        # the chunk pass itself against the token recurrence (two algorithms, one mathematics)
        _, s_rec = o_gdn.scan_fp64(q[sl], k[sl], v[sl], g[sl], beta[sl])
        assert np.abs(final - s_rec).max() <= 1e-11
        nt = entering.shape[0]
        got = np.stack(snaps[at:at + nt]).astype(np.float64)
        # a correctly rounded value of a chain that is within ~1e-6 of the truth: half a unit + the chain's error
        slack = np.abs(got - entering) - _bf16_half_ulp(entering)
        assert slack.max() <= 2e-6, (n, slack.max())
        assert np.array_equal(o_prims.round_bf16(got.astype(np.float32)), got.astype(np.float32))  # on the bf16 grid
        assert np.abs(finals[n] - final).max() <= 2e-6                                     # fp32 chain, unrounded
        assert not np.array_equal(o_prims.round_bf16(finals[n]), finals[n])
        if nt >= 8:   # the same check refuses a chain restarted from its rounded snapshots
            bad = np.stack(_restarted_chain_snapshots(q[sl], k[sl], v[sl], g[sl], beta[sl], length, chunk, HV, V, K))
            bad_slack = np.abs(bad.astype(np.float64) - entering) - _bf16_half_ulp(entering)
            assert bad_slack.max() > 1e-3 and (bad_slack > 2e-6).mean() > 0.05
        at += nt
        pos += length
    assert at == len(snaps)


def test_cpr_entry_states_and_snapshot_placement():
    lens, chunk = [70, 5], 32
    q, k, v, g, beta = _cpr_inputs(lens, 32)
    HV, V, K = v.shape[1], v.shape[2], k.shape[2]
    init = np.random.default_rng(3).standard_normal((2, HV, V, K)).astype(np.float32)
    _, snaps, finals = o_gdn.cpr_forward(q, k, v, g, beta, lens, chunk, init=init)
    assert np.array_equal(snaps[0], o_prims.round_bf16(init[0]))       # chunk 0 enters with the caller's state
    assert np.array_equal(snaps[3], o_prims.round_bf16(init[1]))
    entering, final = o_gdn.chunk_states_fp64(k[:70], v[:70], g[:70], beta[:70], chunk, state0=init[0])
    for c in range(3):
        assert (np.abs(snaps[c] - entering[c]) - _bf16_half_ulp(entering[c])).max() <= 2e-5
    assert np.abs(finals[0] - final).max() <= 2e-5
    # "entering", not "leaving": the state after chunk c is the state entering chunk c + 1, far from entering[c]
    assert np.abs(entering[1] - entering[0]).max() > 0.1


def test_cpr_outputs_start_from_the_snapshot_not_from_the_chain():
    lens, chunk = [96], 32
    q, k, v, g, beta = _cpr_inputs(lens, 33)
    HV, V, K = v.shape[1], v.shape[2], k.shape[2]
    base = o_prims.round_bf16(np.random.default_rng(4).standard_normal((1, HV, V, K)).astype(np.float32))
    moved = (base * np.float32(1 + 0.4 * 2.0 ** -8)).astype(np.float32)   # same bf16 value, different fp32 chain
    assert np.array_equal(o_prims.round_bf16(moved), base) and not np.array_equal(moved, base)
    o_a, snaps_a, fin_a = o_gdn.cpr_forward(q, k, v, g, beta, lens, chunk, init=base)
    o_b, snaps_b, fin_b = o_gdn.cpr_forward(q, k, v, g, beta, lens, chunk, init=moved)
    assert np.array_equal(snaps_a[0], snaps_b[0])
    assert np.array_equal(o_a[:chunk], o_b[:chunk])                       # chunk 0 sees only the snapshot
    assert not np.array_equal(fin_a[0], fin_b[0])                        # the chain carries the difference on
    st = moved[0].copy()                                                  # the mistake: chunk 0 scanned from the chain
    from_chain = o_gdn.scan(q[:chunk], k[:chunk], v[:chunk], g[:chunk], beta[:chunk], st, io_bf16=True)
    assert not np.array_equal(from_chain, o_b[:chunk])
    # numerically: every chunk's outputs are the float64 recurrence started from that chunk's snapshot
    for c in range(3):
        sl = slice(c * chunk, (c + 1) * chunk)
        want, _ = o_gdn.scan_fp64(q[sl], k[sl], v[sl], g[sl], beta[sl], state0=snaps_b[c])
        assert (np.abs(o_b[sl] - want) - _bf16_half_ulp(want)).max() <= 2e-5


def test_cpr_structural_identities_on_the_oracle():
    lens = [5, 64, 33]
    q, k, v, g, beta = _cpr_inputs(lens, 34, slow_decay=False)
    HV, V, K = v.shape[1], v.shape[2], k.shape[2]

    def recurrent(io_bf16):
        outs, pos = [], 0
        for length in lens:
            sl = slice(pos, pos + length)
            st = np.zeros((HV, V, K), np.float32)
            outs.append(o_gdn.scan(q[sl], k[sl], v[sl], g[sl], beta[sl], st, io_bf16=io_bf16))
            pos += length
        return np.concatenate(outs)

    same = lambda a, b: np.array_equal(a.view(np.uint32), b.view(np.uint32))
    one, snaps, _ = o_gdn.cpr_forward(q, k, v, g, beta, lens, 64)        # one chunk per sequence
    assert len(snaps) == 3 and same(one, recurrent(True))
    for chunk in (16, 32):                                               # fp32 wire: no rounding at the boundaries
        got, _, _ = o_gdn.cpr_forward(q, k, v, g, beta, lens, chunk, wire="fp32")
        assert same(got, recurrent(False)), chunk
    small, _, _ = o_gdn.cpr_forward(q, k, v, g, beta, lens, 16)          # bf16 boundaries: a different function
    assert not same(small, recurrent(True)) and np.abs(small - recurrent(True)).max() <= 2 ** -5
