"""GPU parity: GatedDeltaNet scan, preparation and conv (configs 0 and 2, reduced where stated)."""

import numpy as np
import pytest
import torch

from _util import DevicePrims, bf16_to_np, cpu_gen, np_bits, np_to_bf16, same_bits
from oracle import gdn as o_gdn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def dprims():
    return DevicePrims(DEV)


def make_inputs(B, T, H, HV, K, V, seed, dtype=torch.float32):
    """Config-0 style inputs: q,k randn then L2-normalised per head, v randn, beta = sigmoid(randn),
    g = -softplus(randn)."""
    g = cpu_gen(seed)
    q = torch.randn(B, T, H, K, generator=g)
    k = torch.randn(B, T, H, K, generator=g)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6)
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    v = torch.randn(B, T, HV, V, generator=g)
    beta = torch.sigmoid(torch.randn(B, T, HV, generator=g))
    gate = -torch.nn.functional.softplus(torch.randn(B, T, HV, generator=g))
    return q.to(dtype), k.to(dtype), v.to(dtype), gate.float(), beta.to(dtype)


def oracle_scan(q, k, v, g, beta, prims, io_bf16, state=None):
    """Per-sequence oracle over a [B, T, ...] batch. Returns (o, final_states)."""
    B = q.shape[0]
    HV, V, K = v.shape[2], v.shape[3], q.shape[3]
    outs, finals = [], []
    for b in range(B):
        st = np.zeros((HV, V, K), np.float32) if state is None else state[b].copy()
        f = lambda t: t[b].float().numpy()
        outs.append(o_gdn.scan(f(q), f(k), f(v), f(g), f(beta), st, io_bf16=io_bf16, prims=prims))
        finals.append(st)
    return np.stack(outs), np.stack(finals)


def run_scan(q, k, v, g, beta, pool, idx, cu=None, time_tile=0):
    from isoexec_amd.ops.gdn.gdn_ops import gdn_recurrent_kernel

    return gdn_recurrent_kernel(q, k, v, g, beta, ssm_state=pool, state_indices=idx, cu_seqlens=cu,
                                time_tile=time_tile)


def test_config0_scan_bit_exact_and_chunk_invariant(dprims):
    """Config 0: B=2, T=256, 4 heads, d_k=d_v=64, fp32. Oracle bit-exact; bitwise equal across
    time tiles {16, 32, 64} and prefill/decode splits, state included."""
    B, T, H, K, V = 2, 256, 4, 64, 64
    q, k, v, g, beta = make_inputs(B, T, H, H, K, V, seed=0)
    want_o, want_s = oracle_scan(q, k, v, g, beta, dprims, io_bf16=False)
    d = lambda t: t.to(DEV)
    idx = torch.zeros(B, T, dtype=torch.int32)
    idx[:, 0] = torch.arange(1, B + 1)
    idx[:, T - 1] = torch.arange(1, B + 1)
    results = []
    for tt in (16, 32, 64):
        pool = torch.zeros(B + 1, H, V, K, device=DEV)
        o = run_scan(d(q), d(k), d(v), d(g), d(beta), pool, d(idx), time_tile=tt)
        results.append((o, pool))
    o0, p0 = results[0]
    assert np.array_equal(np_bits(o0.cpu().numpy()), np_bits(want_o))
    assert np.array_equal(np_bits(p0[1:].cpu().numpy()), np_bits(want_s))
    for o, p in results[1:]:
        assert same_bits(o, o0) and same_bits(p, p0)
    # tolerance against the textbook float64 recurrence
    o64, _ = o_gdn.scan_fp64(q[0].numpy(), k[0].numpy(), v[0].numpy(), g[0].numpy(), beta[0].numpy())
    assert np.abs(o0[0].cpu().numpy() - o64).max() <= 2e-5
    # prefill to t, then token-by-token decode: identical bits and identical final state
    for split in (0, 1, 63, 64, 65, 127, 255):
        pool = torch.zeros(B + 1, H, V, K, device=DEV)
        rows = torch.arange(1, B + 1, dtype=torch.int32, device=DEV)
        outs = []
        if split > 0:
            ip = torch.zeros(B, split, dtype=torch.int32)
            ip[:, 0] = torch.arange(1, B + 1)
            ip[:, split - 1] = torch.arange(1, B + 1)
            outs.append(run_scan(d(q[:, :split]), d(k[:, :split]), d(v[:, :split]), d(g[:, :split]),
                                 d(beta[:, :split]), pool, d(ip)))
        stop = min(T, split + 40)  # 40 decode steps are enough to expose any drift
        for t in range(split, stop):
            outs.append(run_scan(d(q[:, t:t + 1]), d(k[:, t:t + 1]), d(v[:, t:t + 1]), d(g[:, t:t + 1]),
                                 d(beta[:, t:t + 1]), pool, rows))
        got = torch.cat(outs, dim=1)
        assert same_bits(got, o0[:, :stop]), split


def test_scan_bf16_gqa_varlen_cross_sequence_and_null_lanes(dprims):
    """Config-2 head geometry (K=V=128, GQA 2 v-heads per k-head) at reduced head count, bf16 io,
    packed varlen with the reference's lengths [150, 37, 64, 201] (gdn_batch_invariant.py:141-215)."""
    H, HV, K, V = 2, 4, 128, 128
    lens = [150, 37, 64, 201]
    total = sum(lens)
    q, k, v, g, beta = make_inputs(1, total, H, HV, K, V, seed=2, dtype=torch.bfloat16)
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
    N = len(lens)
    idx = torch.zeros(N, max(lens), dtype=torch.int32)
    for n, L in enumerate(lens):
        idx[n, 0] = n + 1
        idx[n, L - 1] = n + 1
    d = lambda t: t.to(DEV)
    pool = torch.zeros(N + 1, HV, V, K, device=DEV)
    o = run_scan(d(q), d(k), d(v), d(g), d(beta), pool, d(idx), cu=d(cu))[0]
    # oracle per sequence
    for n, L in enumerate(lens):
        s, e = int(cu[n]), int(cu[n + 1])
        st = np.zeros((HV, V, K), np.float32)
        f = lambda t: t[0, s:e].float().numpy()
        want = o_gdn.scan(f(q), f(k), f(v), f(g), f(beta), st, io_bf16=True, prims=dprims)
        assert same_bits(o[s:e].cpu(), np_to_bf16(want)), n
        assert np.array_equal(np_bits(pool[n + 1].cpu().numpy()), np_bits(st)), n
    # each sequence alone == inside the packed batch (cross-sequence invariance)
    for n, L in enumerate(lens):
        s, e = int(cu[n]), int(cu[n + 1])
        p1 = torch.zeros(2, HV, V, K, device=DEV)
        i1 = torch.zeros(1, L, dtype=torch.int32)
        i1[0, 0] = 1
        alone = run_scan(d(q[:, s:e]), d(k[:, s:e]), d(v[:, s:e]), d(g[:, s:e]), d(beta[:, s:e]), p1, d(i1))[0]
        assert same_bits(alone, o[s:e])
    # null lane: sequence 1 mapped to row 0 is skipped: zero output, pool untouched
    idx2 = idx.clone()
    idx2[1] = 0
    pool2 = torch.zeros(N + 1, HV, V, K, device=DEV)
    o2 = run_scan(d(q), d(k), d(v), d(g), d(beta), pool2, d(idx2), cu=d(cu))[0]
    s, e = int(cu[1]), int(cu[2])
    assert float(o2[s:e].float().abs().max()) == 0.0 and float(pool2[2].abs().max()) == 0.0
    assert same_bits(o2[:s], o[:s]) and same_bits(o2[e:], o[e:])
    # mid-sequence store: a positive index at column t stores the state after token t
    idx3 = torch.zeros(1, 64, dtype=torch.int32)
    idx3[0, 0] = 1
    idx3[0, 9] = 2
    idx3[0, 63] = 1
    s, e = int(cu[2]), int(cu[3])
    pool3 = torch.zeros(3, HV, V, K, device=DEV)
    run_scan(d(q[:, s:e]), d(k[:, s:e]), d(v[:, s:e]), d(g[:, s:e]), d(beta[:, s:e]), pool3, d(idx3))
    st = np.zeros((HV, V, K), np.float32)
    f = lambda t: t[0, s:e].float().numpy()
    _, snap = o_gdn.scan(f(q), f(k), f(v), f(g), f(beta), st, io_bf16=True, prims=dprims, snapshots=True)
    assert np.array_equal(np_bits(pool3[2].cpu().numpy()), np_bits(snap[9]))
    assert np.array_equal(np_bits(pool3[1].cpu().numpy()), np_bits(snap[63]))


def test_scan_closed_forms():
    """beta = 0: pure decay S_T = exp(sum g) S_0 (o = S q). g = 0, beta = 1, orthonormal keys:
    the state is an associative memory and o_t = v_t for q_t = k_t * sqrt(K)."""
    H, K, V, T = 1, 64, 64, 48
    g = cpu_gen(3)
    eye = torch.eye(K)[:T]  # orthonormal keys
    k = eye.view(1, T, 1, K)
    q = k * (K ** 0.5)
    v = torch.randn(1, T, H, V, generator=g)
    zeros = torch.zeros(1, T, H)
    ones = torch.ones(1, T, H)
    d = lambda t: t.to(DEV)
    idx = torch.zeros(1, T, dtype=torch.int32)
    idx[0, 0] = 1
    pool = torch.zeros(2, H, V, K, device=DEV)
    o = run_scan(d(q), d(k), d(v), d(zeros), d(ones), pool, d(idx))
    assert torch.equal(o.cpu(), v)  # exact: products with 0/1 and a scale of 8 * 0.125
    s0 = torch.randn(H, V, K, generator=g)
    gg = -torch.rand(1, T, H, generator=g)
    pool = torch.zeros(2, H, V, K, device=DEV)
    pool[1] = s0.to(DEV)
    idx[0, T - 1] = 1
    run_scan(d(q), d(k), d(v), d(gg), d(zeros), pool, d(idx))
    want = s0.double() * torch.exp(gg.double().sum())
    assert (pool[1].cpu().double() - want).abs().max().item() <= 1e-5


def test_l2norm_and_gate_bit_exact(dprims):
    from isoexec_amd.ops.gdn.gdn_ops import gdn_gate_and_beta, gdn_l2norm

    g = cpu_gen(4)
    for dtype in (torch.bfloat16, torch.float32):
        proj = (2 * torch.randn(50, 2 * 2 * 128 + 4 * 128, generator=g)).to(dtype)
        x = proj[:, 256:512].view(50, 2, 128)  # a strided slice of the conv output
        want = o_gdn.l2norm(x.float().numpy(), io_bf16=dtype is torch.bfloat16)
        pd = proj.to(DEV)
        got = gdn_l2norm(pd[:, 256:512].view(50, 2, 128))
        assert np.array_equal(np_bits(got.float().cpu().numpy()), np_bits(want))
        a = (2 * torch.randn(50, 4, generator=g)).to(dtype)
        b = (2 * torch.randn(50, 4, generator=g)).to(dtype)
        a[0, 0] = 30.0  # softplus threshold branch
        A_log = 0.2 * torch.randn(4, generator=g)
        dt_bias = 0.2 * torch.randn(4, generator=g)
        wg, wb = o_gdn.gate_and_beta(a.float().numpy(), b.float().numpy(), A_log.numpy(), dt_bias.numpy(),
                                     io_bf16=dtype is torch.bfloat16, prims=dprims)
        gg, bb = gdn_gate_and_beta(a.to(DEV), b.to(DEV), A_log.to(DEV), dt_bias.to(DEV))
        # softplus is evaluated as one device primitive; exp(A_log) and the product are IEEE
        assert np.array_equal(np_bits(gg.cpu().numpy()), np_bits(wg))
        assert np.array_equal(np_bits(bb.float().cpu().numpy()), np_bits(wb))
        # a bf16 parameter under the eager name: exp() is rounded to bf16 before the product (gdn_ops.py:1197-1210)
        A16 = A_log.to(torch.bfloat16)
        wg16, _ = o_gdn.gate_and_beta(a.float().numpy(), b.float().numpy(), A16.float().numpy(), dt_bias.numpy(),
                                      io_bf16=dtype is torch.bfloat16, prims=dprims, exp_bf16=True)
        gg16, _ = gdn_gate_and_beta(a.to(DEV), b.to(DEV), A16.to(DEV), dt_bias.to(DEV))
        assert np.array_equal(np_bits(gg16.cpu().numpy()), np_bits(wg16))
        assert not np.array_equal(np_bits(gg16.cpu().numpy()), np_bits(wg))
        with pytest.raises(RuntimeError, match="fp32 and bf16 A_log"):
            gdn_gate_and_beta(a.to(DEV), b.to(DEV), A_log.half().to(DEV), dt_bias.to(DEV))


def test_conv_bit_exact_prefill_decode_and_state(dprims):
    from isoexec_amd.ops.gdn.gdn_ops import gdn_causal_conv, gdn_causal_conv_batched

    g = cpu_gen(5)
    T, D, W = 70, 384, 4
    x = torch.randn(T, D, generator=g).to(torch.bfloat16)
    w = (0.5 * torch.randn(D, W, generator=g)).to(torch.bfloat16)
    b = (0.1 * torch.randn(D, generator=g)).to(torch.bfloat16)
    for bias in (None, b):
        bn = None if bias is None else bf16_to_np(bias)
        want_y, want_s = o_gdn.causal_conv(bf16_to_np(x), bf16_to_np(w), bn, prims=dprims)
        y, s = gdn_causal_conv(x.to(DEV), w.to(DEV), None if bias is None else bias.to(DEV),
                               return_final_state=True)
        assert same_bits(y.cpu(), np_to_bf16(want_y)) and same_bits(s.cpu(), np_to_bf16(want_s))
    # split anywhere == unsplit, chained through the returned state (incl. a 2-token first chunk)
    for cut in (1, 2, 3, 33):
        y1, s1 = gdn_causal_conv(x[:cut].to(DEV), w.to(DEV), b.to(DEV), return_final_state=True)
        y2, s2 = gdn_causal_conv(x[cut:].to(DEV), w.to(DEV), b.to(DEV), initial_state=s1, return_final_state=True)
        assert same_bits(torch.cat([y1, y2]), y) and same_bits(s2, s)
    # token-by-token batched decode == prefill
    state = torch.zeros(1, D, W - 1, dtype=torch.bfloat16, device=DEV)
    outs = []
    for t in range(12):
        xt = x[t:t + 1].to(DEV)
        outs.append(gdn_causal_conv_batched(xt.view(1, 1, D), w.to(DEV), b.to(DEV), initial_state=state)[0])
        state = torch.cat([state[..., 1:], xt.view(1, D, 1)], dim=-1)
    assert same_bits(torch.cat(outs), y[:12])
    # The vector path (W = 4, D a multiple of 8) and the scalar path compute the same function: a width
    # the vector path does not take, and a channel count it cannot.
    for (D2, W2) in ((100, 4), (64, 3), (8, 2)):
        x2 = torch.randn(19, D2, generator=g).to(torch.bfloat16)
        w2 = (0.5 * torch.randn(D2, W2, generator=g)).to(torch.bfloat16)
        b2 = (0.1 * torch.randn(D2, generator=g)).to(torch.bfloat16)
        want_y, want_s = o_gdn.causal_conv(bf16_to_np(x2), bf16_to_np(w2), bf16_to_np(b2), prims=dprims)
        y2, s2 = gdn_causal_conv(x2.to(DEV), w2.to(DEV), b2.to(DEV), return_final_state=True)
        assert same_bits(y2.cpu(), np_to_bf16(want_y)) and same_bits(s2.cpu(), np_to_bf16(want_s)), (D2, W2)


@pytest.mark.parametrize("lens", [[333, 7, 64, 1, 257, 130, 80, 16, 90], [40, 3, 9, 1, 21, 33, 12, 2, 30]],
                         ids=["long", "short"])
@pytest.mark.parametrize("D,normed", [(2048, False), (6144, False), (2048, True), (4096, True)])
def test_packed_conv_in_the_run_order_against_the_oracle(D, normed, lens, dprims):
    """Channel counts that fill whole workgroups take the convolution's XCD-run order (consecutive token groups of a
    channel block on one XCD). Every sequence of a ragged packed batch against the oracle, stored windows in and out; the
    normalising form against the oracle's conv followed by its l2norm."""
    from isoexec_amd.ops.gdn.gdn_ops import conv_packed

    W, K = 4, 128
    g = cpu_gen(D + normed)
    T, n = sum(lens), len(lens)             # mean length 108 (16 or 8 tokens per thread) or 16 (4 per thread)
    wide = torch.randn(T, D + 72, generator=g).to(torch.bfloat16)
    x = wide[:, 8:8 + D]                                    # a column slice: row pitch D + 72, first column 8
    w = (0.5 * torch.randn(D, W, generator=g)).to(torch.bfloat16)
    b = (0.1 * torch.randn(D, generator=g)).to(torch.bfloat16)
    pool = torch.randn(n + 1, D, W - 1, generator=g).to(torch.bfloat16)
    rows_in = torch.tensor([0, 2, 0, 4, 5, 0, 7, 0, 9], dtype=torch.int32)
    rows_out = torch.arange(1, n + 1, dtype=torch.int32)
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
    pool_d = pool.to(DEV)
    qk = D // 2 if normed else 0
    y = conv_packed(wide.to(DEV)[:, 8:8 + D], w.to(DEV), b.to(DEV), cu_seqlens=cu.to(DEV), conv_state=pool_d,
                    rows_in=rows_in.to(DEV), rows_out=rows_out.to(DEV), l2norm_qk=qk, head_k_dim=K if normed else 0)
    for i, L in enumerate(lens):
        s0 = int(cu[i])
        init = bf16_to_np(pool[int(rows_in[i])]) if int(rows_in[i]) else None
        want_y, want_s = o_gdn.causal_conv(bf16_to_np(x[s0:s0 + L]), bf16_to_np(w), bf16_to_np(b), initial_state=init,
                                           prims=dprims)
        if normed:
            want_y[:, :qk] = o_gdn.l2norm(want_y[:, :qk].reshape(L, qk // K, K)).reshape(L, qk)
        assert same_bits(y[s0:s0 + L].cpu(), np_to_bf16(want_y)), (i, L)
        assert same_bits(pool_d[i + 1].cpu(), np_to_bf16(want_s)), (i, L)


def test_native_core_varlen_equals_decode_steps():
    """The fused-front composition (raw q/k, raw a/b): one varlen call == T sequential decode calls,
    state included (gdn_native_kernel_parity_test_gpu.py T1-T4)."""
    from isoexec_amd.ops.gdn.gdn_ops import gdn_native_core_kernel

    g = cpu_gen(6)
    T, H, HV, K, V = 24, 2, 4, 128, 128
    q = torch.randn(1, T, H, K, generator=g).to(torch.bfloat16).to(DEV)
    k = torch.randn(1, T, H, K, generator=g).to(torch.bfloat16).to(DEV)
    v = torch.randn(1, T, HV, V, generator=g).to(torch.bfloat16).to(DEV)
    a = torch.randn(T, HV, generator=g).to(torch.bfloat16).to(DEV)
    b = torch.randn(T, HV, generator=g).to(torch.bfloat16).to(DEV)
    A_log = (0.2 * torch.randn(HV, generator=g)).to(DEV)
    dt_bias = (0.2 * torch.randn(HV, generator=g)).to(DEV)
    idx = torch.zeros(1, T, dtype=torch.int32, device=DEV)
    idx[0, 0] = 1
    idx[0, T - 1] = 1
    pool = torch.zeros(2, HV, V, K, device=DEV)
    cu = torch.tensor([0, T], dtype=torch.int32, device=DEV)
    o = gdn_native_core_kernel(q, k, v, a, b, A_log, dt_bias, ssm_state=pool, state_indices=idx, cu_seqlens=cu)
    pool2 = torch.zeros(2, HV, V, K, device=DEV)
    one = torch.ones(1, dtype=torch.int32, device=DEV)
    outs = [gdn_native_core_kernel(q[:, t:t + 1], k[:, t:t + 1], v[:, t:t + 1], a[t:t + 1], b[t:t + 1], A_log,
                                   dt_bias, ssm_state=pool2, state_indices=one, cu_seqlens=None)
            for t in range(T)]
    assert same_bits(torch.cat(outs, dim=1), o) and same_bits(pool2, pool)


def test_fused_decode_prep_equals_the_three_launches_bit_for_bit():
    """``decode_prep`` (one launch: conv on the stored window slid in place, l2norm of q and k, gating) against
    ``conv_packed`` + ``gdn_l2norm`` + ``gate_and_beta_fp32``, each pinned against the oracle above: outputs AND the
    pool, over several steps, with a padded lane and operands that are column slices of one projection buffer."""
    from isoexec_amd.ops.gdn.gdn_ops import conv_packed, decode_prep, gate_and_beta_fp32, gdn_l2norm

    g = cpu_gen(41)
    N, H, K, HV, V, W = 5, 2, 128, 4, 128, 4
    D = 2 * H * K + HV * V
    rows = torch.tensor([3, 0, 1, 6, 2], dtype=torch.int32, device=DEV)       # lane 1 is padded
    cw = (0.5 * torch.randn(D, W, generator=g)).to(torch.bfloat16).to(DEV)
    cb = (0.1 * torch.randn(D, generator=g)).to(torch.bfloat16).to(DEV)
    A_log, dt_bias = (0.3 * torch.randn(HV, generator=g)).to(DEV), (0.3 * torch.randn(HV, generator=g)).to(DEV)
    pool0 = torch.randn(8, D, W - 1, generator=g).to(torch.bfloat16).to(DEV)
    cu = torch.arange(N + 1, dtype=torch.int32, device=DEV)
    for bias in (cb, None):
        pool_a, pool_b = pool0.clone(), pool0.clone()
        for step in range(4):
            proj = torch.randn(N, D + 2 * HV + 24, generator=g).to(torch.bfloat16).to(DEV)
            proj[0, :D] *= 30.0                                                # large activations, softplus branch
            x, b_in, a_in = proj[:, :D], proj[:, D:D + HV], proj[:, D + HV:D + 2 * HV]
            y = conv_packed(x, cw, bias, cu_seqlens=cu, conv_state=pool_a, rows_in=rows, rows_out=rows)
            want_qk = gdn_l2norm(y[:, :2 * H * K].unflatten(1, (2 * H, K)))
            want_g, want_beta = gate_and_beta_fp32(a_in, b_in, A_log, dt_bias)
            got = decode_prep(x, a_in, b_in, cw, bias, A_log, dt_bias, pool_b, rows, H=H, K=K, HV=HV, V=V)
            assert got is not None
            yy, gg, bb = got
            assert same_bits(yy[:, :2 * H * K].reshape(N, 2 * H, K), want_qk), step
            assert same_bits(yy[:, 2 * H * K:].contiguous(), y[:, 2 * H * K:].contiguous())
            assert same_bits(gg, want_g) and same_bits(bb, want_beta)
            assert same_bits(pool_a, pool_b)
        assert same_bits(pool_a[0], pool0[0]) and not same_bits(pool_a[3], pool0[3])
    # what the kernel does not serve is declined, not approximated
    assert decode_prep(x.float(), a_in, b_in, cw, cb, A_log, dt_bias, pool_b, rows, H=H, K=K, HV=HV, V=V) is None
    assert decode_prep(x[:, :2 * 2 * 64 + HV * V], a_in, b_in, cw[:2 * 2 * 64 + HV * V], None, A_log, dt_bias, pool_b, rows,
                       H=2, K=64, HV=HV, V=V) is None


@pytest.mark.parametrize("H,HV", [(2, 2), (16, 32)])
def test_conv_with_the_l2norm_folded_in_equals_the_two_launches(H, HV):
    """``conv_packed(..., l2norm_qk=...)``: q and k heads leave the convolution's launch normalised. Against the plain
    convolution followed by ``gdn_l2norm`` on those columns, bit for bit: long and very short sequences in one packed
    batch (both paths through the kernel), an input that is a column slice of a wider buffer, history rows in and out."""
    from isoexec_amd.ops.gdn.gdn_ops import conv_packed, gdn_l2norm, gdn_native_core, gdn_native_core_normed

    K = V = 128
    W = 4
    kd = H * K
    D = 2 * kd + HV * V
    g = cpu_gen(70 + H)
    lens = [300, 1, 2, 70, 3, 5, 129]
    T = sum(lens)
    wide = torch.randn(T, D + 64, generator=g).to(torch.bfloat16).to(DEV)
    x = wide[:, :D]
    weight = (torch.randn(D, W, generator=g) * 0.4).to(torch.bfloat16).to(DEV)
    bias = (torch.randn(D, generator=g) * 0.1).to(torch.bfloat16).to(DEV)
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32, device=DEV)
    n = len(lens)
    pools = [(torch.randn(n + 1, D, W - 1, generator=cpu_gen(9)).to(torch.bfloat16).to(DEV)) for _ in range(2)]
    rows_in = torch.tensor([1, 0, 3, 0, 5, 6, 0], dtype=torch.int32, device=DEV)   # some sequences continue a stored window
    rows_out = torch.arange(1, n + 1, dtype=torch.int32, device=DEV)
    plain = conv_packed(x, weight, bias, cu_seqlens=cu, conv_state=pools[0], rows_in=rows_in, rows_out=rows_out)
    fused = conv_packed(x, weight, bias, cu_seqlens=cu, conv_state=pools[1], rows_in=rows_in, rows_out=rows_out,
                        l2norm_qk=2 * kd, head_k_dim=K)
    assert fused is not None and same_bits(pools[0], pools[1])
    want_qk = gdn_l2norm(plain[:, :2 * kd].unflatten(1, (2 * H, K)))
    assert same_bits(fused[:, :2 * kd].unflatten(1, (2 * H, K)).contiguous(), want_qk)
    assert same_bits(fused[:, 2 * kd:].contiguous(), plain[:, 2 * kd:].contiguous())
    # the composition the trainer runs: raw heads through gdn_native_core == normalised heads through its _normed form
    a = torch.randn(T, HV, generator=g).to(torch.bfloat16).to(DEV)
    b = torch.randn(T, HV, generator=g).to(torch.bfloat16).to(DEV)
    A_log = (torch.randn(HV, generator=g) * 0.3).to(DEV)
    dt_bias = (torch.randn(HV, generator=g) * 0.3).to(DEV)
    split = lambda y: (y[:, :kd].unflatten(1, (H, K)).unsqueeze(0), y[:, kd:2 * kd].unflatten(1, (H, K)).unsqueeze(0),
                       y[:, 2 * kd:].unflatten(1, (HV, V)).unsqueeze(0))
    o_raw = gdn_native_core(*split(plain), a, b, A_log, dt_bias, cu_seqlens=cu)
    o_normed = gdn_native_core_normed(*split(fused), a, b, A_log, dt_bias, cu_seqlens=cu)
    assert same_bits(o_raw, o_normed)
    # a head that holds an infinity or a NaN takes the launch's other way out (canonical NaNs, zeros): same bits again
    spoiled = x.clone()
    spoiled[5, 3] = float("inf")            # long sequence, first q head
    spoiled[200, kd + 130] = float("nan")   # long sequence, a k head
    spoiled[300, 7] = float("-inf")         # the one-token sequence
    spoiled[T - 1, 2 * kd - 1] = float("nan")
    plain_s = conv_packed(spoiled, weight, bias, cu_seqlens=cu)
    fused_s = conv_packed(spoiled, weight, bias, cu_seqlens=cu, l2norm_qk=2 * kd, head_k_dim=K)
    want_s = gdn_l2norm(plain_s[:, :2 * kd].unflatten(1, (2 * H, K)))
    assert not torch.isfinite(want_s.float()).all()
    assert same_bits(fused_s[:, :2 * kd].unflatten(1, (2 * H, K)).contiguous(), want_s)
    assert same_bits(fused_s[:, 2 * kd:].contiguous(), plain_s[:, 2 * kd:].contiguous())
    # heads of another size are not served by the one-launch form: the wrapper makes the two calls itself
    y64 = conv_packed(x, weight, bias, cu_seqlens=cu, l2norm_qk=2 * kd, head_k_dim=64)
    plain64 = conv_packed(x, weight, bias, cu_seqlens=cu)
    assert same_bits(y64[:, :2 * kd].unflatten(1, (4 * H, 64)).contiguous(), gdn_l2norm(plain64[:, :2 * kd].unflatten(1, (4 * H, 64))))
    assert same_bits(y64[:, 2 * kd:].contiguous(), plain64[:, 2 * kd:].contiguous())


def test_scan_with_the_gated_output_norm_folded_in_equals_the_two_launches():
    """``gdn_recurrent_kernel(..., gated_norm=...)``: the lane-pair scan applies the layer's gated output norm to its own
    outputs. Against the scan followed by ``fused_gated_out_norm``: outputs and final states bit for bit, a packed batch
    with short, long and empty sequences, null lanes (state index 0) included, a gate that is a column slice of a wider
    buffer; where the lane-pair layout does not run the library declines the form before it touches the state and the
    wrapper makes the two calls."""
    from isoexec_amd.ops.gdn.gdn_ops import gdn_l2norm, gdn_recurrent_kernel
    from isoexec_amd.ops.norms.fused_outnorm import fused_gated_out_norm

    H, HV, K, V = 16, 32, 128, 128
    g = cpu_gen(91)
    lens = [70, 1, 0, 33, 16, 5, 129, 17, 2, 64, 48, 31, 7, 96, 3, 40, 12, 100]        # 18 sequences x 32 heads >= 512 pairs
    T, N = sum(lens), len(lens)
    bf = lambda t: t.to(torch.bfloat16).to(DEV)
    q = gdn_l2norm(bf(torch.randn(T, H, K, generator=g)))
    k = gdn_l2norm(bf(torch.randn(T, H, K, generator=g)))
    v = bf(torch.randn(T, HV, V, generator=g))
    gate = -torch.nn.functional.softplus(torch.randn(T, HV, generator=g)).to(DEV)
    beta = bf(torch.sigmoid(torch.randn(T, HV, generator=g)))
    wide = bf(torch.randn(T, HV * V + 64, generator=g))
    z = wide[:, :HV * V].unflatten(1, (HV, V))
    w = bf(torch.randn(V, generator=g) * 0.1)
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32, device=DEV)
    rows = torch.arange(1, N + 1, dtype=torch.int32, device=DEV)
    rows[4] = 0                                                                           # a null lane: outputs defined, no state
    pool0 = torch.randn(N + 1, HV, V, K, generator=g).to(DEV) * 0.1
    u = lambda t: t.unsqueeze(0)
    pa, pb = pool0.clone(), pool0.clone()
    o = gdn_recurrent_kernel(u(q), u(k), u(v), u(gate), u(beta), ssm_state=pa, state_indices=rows, cu_seqlens=cu)[0]
    want = fused_gated_out_norm(o, z, w, 1e-6).view(T, HV, V)
    got = gdn_recurrent_kernel(u(q), u(k), u(v), u(gate), u(beta), ssm_state=pb, state_indices=rows, cu_seqlens=cu,
                               gated_norm=(z, w, 1e-6, True))
    assert got is not None and same_bits(got[0], want) and same_bits(pa, pb)
    # NaNs and infinities in values, gate and weight: the folded norm rounds inside its chain with the hardware convert
    # and must still store what the two launches store (canonical NaNs, signed zeros, infinities)
    v2, wide2, w2 = v.clone(), wide.clone(), w.clone()
    v2[3, 1, 7] = float("nan")
    v2[80, 5, 100] = float("inf")
    v2.view(torch.int16)[200, 9, 3] = -1                      # 0xffff: a negative NaN with a full payload
    wide2[10, 2 * V + 5] = float("-inf")
    wide2[11, 3 * V + 6] = float("nan")
    wide2[12, 4 * V + 7] = -300.0                             # silu underflows to a signed zero
    w2[9] = float("inf")
    z2 = wide2[:, :HV * V].unflatten(1, (HV, V))
    pe, pf = pool0.clone(), pool0.clone()
    o2 = gdn_recurrent_kernel(u(q), u(k), u(v2), u(gate), u(beta), ssm_state=pe, state_indices=rows, cu_seqlens=cu)[0]
    want2 = fused_gated_out_norm(o2, z2, w2, 1e-6).view(T, HV, V)
    got_nf = gdn_recurrent_kernel(u(q), u(k), u(v2), u(gate), u(beta), ssm_state=pf, state_indices=rows, cu_seqlens=cu,
                                  gated_norm=(z2, w2, 1e-6, True))
    assert not torch.isfinite(want2.float()).all()
    assert got_nf is not None and same_bits(got_nf[0], want2) and same_bits(pe, pf)
    # fewer than 512 (sequence, head) pairs: the 16-lane layout runs; the library declines the fused form untouched ...
    from isoexec_amd import _lib

    pc = pool0.clone()
    few = torch.tensor([0, 70, 71], dtype=torch.int32, device=DEV)
    scratch = torch.empty(71, HV, V, dtype=torch.bfloat16, device=DEV)
    rc = _lib.lib().ix_gdn_scan_gated_norm(q.data_ptr(), k.data_ptr(), v.data_ptr(), gate.data_ptr(), beta.data_ptr(),
                                           scratch.data_ptr(), H * K, H * K, HV * V, pc.data_ptr(), few.data_ptr(),
                                           rows.data_ptr(), 2, H, HV, K, V, K ** -0.5, 0, z.data_ptr(), z.stride(0),
                                           w.data_ptr(), 1e-6, 1, _lib.current_stream(torch.device(DEV)))
    torch.cuda.synchronize()
    assert rc == _lib.IX_DECLINED and same_bits(pc, pool0)
    # ... and the wrapper makes the two calls: the same result
    pd = pool0.clone()
    got2 = gdn_recurrent_kernel(u(q[:71]), u(k[:71]), u(v[:71]), u(gate[:71]), u(beta[:71]), ssm_state=pd,
                                state_indices=rows[:2], cu_seqlens=few, gated_norm=(z[:71], w, 1e-6, True))
    assert same_bits(got2[0], want[:71]) and same_bits(pd[:3], pa[:3])
