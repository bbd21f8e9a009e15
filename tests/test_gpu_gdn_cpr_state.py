"""GPU parity of the boundary-form engine state (``CprGDN``; reference gdn_cpr_state.py:379-1245) with the
boundary-form forward (``gdn_cpr_fwd``): whatever way a request's tokens are cut into a packed prefill, resumed
prefill chunks and single-token decode steps, mixed with other requests and padded lanes, the layer's outputs equal
the one-pass forward's bit for bit, and its entry states, running states, buffers and positions are what the
definition says."""

import numpy as np
import pytest
import torch

from _util import cpu_gen, same_bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
H, K, HV, V, W = 2, 64, 4, 64, 4
KD = H * K
D = 2 * KD + HV * V
C = 16


def params():
    g = cpu_gen(11)
    bf = lambda t: t.to(torch.bfloat16)
    return dict(conv_weight=bf(torch.randn(D, W, generator=g) * 0.4).to(DEV), conv_bias=bf(torch.randn(D, generator=g) * 0.1).to(DEV),
                A_log=(torch.randn(HV, generator=g) * 0.3).to(DEV), dt_bias=(torch.randn(HV, generator=g) * 0.3).to(DEV))


def make_layer(capacity=6, chunk=C):
    from isoexec_amd.ops.gdn.gdn_cpr_state import CprGDN

    return CprGDN(capacity=capacity, chunk_size=chunk, num_k_heads=H, head_k_dim=K, num_v_heads=HV, head_v_dim=V,
                  device=DEV, **params())


def request(seed, n):
    g = cpu_gen(seed)
    bf = lambda t: t.to(torch.bfloat16).to(DEV)
    return bf(torch.randn(n, D, generator=g)), bf(torch.randn(n, HV, generator=g)), bf(torch.randn(n, HV, generator=g))


def one_pass(layer, x, a, b, chunk=C):
    """The forward over a whole request from nothing: conv, normalisation, gate, then gdn_cpr_fwd; also the chain
    state at the last boundary and the running state after the last token."""
    from isoexec_amd.ops.gdn.gdn_cpr import chunk_boundary_states, gdn_cpr_fwd
    from isoexec_amd.ops.gdn.gdn_ops import conv_packed, gdn_recurrent_kernel

    n = x.shape[0]
    cu = torch.tensor([0, n], dtype=torch.int32, device=DEV)
    y = conv_packed(x, layer.conv_weight, layer.conv_bias, cu_seqlens=cu)
    q, k, v = layer._split_qkv(y)
    g, beta = layer._gate_and_beta(a, b)
    u = lambda t: t.unsqueeze(0)
    o = gdn_cpr_fwd(u(q), u(k), u(v), u(g), u(beta), cu_seqlens=cu, chunk_size=chunk)[0]
    nfull = (n // chunk) * chunk
    entry = torch.zeros(HV, V, K, device=DEV)
    if nfull:
        cuf = torch.tensor([0, nfull], dtype=torch.int32, device=DEV)
        _, fin, _ = chunk_boundary_states(None, u(k[:nfull]), u(v[:nfull]), u(g[:nfull]), u(beta[:nfull]), cuf, chunk,
                                          output_final_state=True)
        entry = fin[0]
    running = entry.to(torch.bfloat16).float().unsqueeze(0).contiguous()
    pool = torch.cat([torch.zeros_like(running), running])
    if n > nfull:
        cut = torch.tensor([0, n - nfull], dtype=torch.int32, device=DEV)
        gdn_recurrent_kernel(u(q[nfull:]), u(k[nfull:]), u(v[nfull:]), u(g[nfull:]), u(beta[nfull:]), ssm_state=pool,
                             state_indices=torch.tensor([1], dtype=torch.int32, device=DEV), cu_seqlens=cut)
    return o, entry, pool[1], (k, v, g, beta)


def check_row(layer, slot, n, want):
    o_want, entry, running, (k, v, g, beta) = want
    row = layer.require_row(slot)
    assert int(layer.pos[row]) == n
    assert same_bits(layer.entry_state[row], entry)
    assert same_bits(layer.ssm_state[row], running)
    r = n % layer.chunk_size
    if r:
        assert same_bits(layer.k_buf[row, :r], k[n - r:n].contiguous()) and same_bits(layer.v_buf[row, :r], v[n - r:n].contiguous())
        assert same_bits(layer.g_buf[row, :r], g[n - r:n]) and same_bits(layer.b_buf[row, :r], beta[n - r:n])


@pytest.mark.parametrize("cuts", [
    {"prefill": [(0, 37), (1, 16), (2, 5)], "decode_to": 70},          # ends inside, on, and before a boundary
    {"prefill": [(0, 1), (1, 32), (2, 47)], "decode_to": 50},
])
def test_prefill_then_decode_equals_the_one_pass_forward(cuts):
    layer = make_layer()
    total = cuts["decode_to"]
    reqs = {s: request(100 + s, total) for s, _ in cuts["prefill"]}
    want = {s: one_pass(layer, *reqs[s]) for s in reqs}
    slots = [s for s, _ in cuts["prefill"]]
    lens = [n for _, n in cuts["prefill"]]
    x = torch.cat([reqs[s][0][:n] for s, n in cuts["prefill"]])
    a = torch.cat([reqs[s][1][:n] for s, n in cuts["prefill"]])
    b = torch.cat([reqs[s][2][:n] for s, n in cuts["prefill"]])
    qsl = [0] + list(np.cumsum(lens))
    o = layer.prefill(torch.tensor(slots, device=DEV), slots, x, a, b, qsl)
    at = 0
    for s, n in cuts["prefill"]:
        assert same_bits(o[at:at + n], want[s][0][:n]), (s, "prefill")
        at += n
    have = dict(cuts["prefill"])
    # decode: all live requests plus one padded lane (an unknown slot id -> the null row)
    st = torch.tensor(slots + [4000], dtype=torch.int64, device=DEV)
    step = 0
    while any(have[s] < total for s in slots):
        xs = torch.stack([reqs[s][0][min(have[s], total - 1)] for s in slots] + [reqs[slots[0]][0][0]])
        as_ = torch.stack([reqs[s][1][min(have[s], total - 1)] for s in slots] + [reqs[slots[0]][1][0]])
        bs = torch.stack([reqs[s][2][min(have[s], total - 1)] for s in slots] + [reqs[slots[0]][2][0]])
        live = [s for s in slots if have[s] < total]
        if len(live) < len(slots):  # finished requests drop out of the batch
            keep = [i for i, s in enumerate(slots) if s in live] + [len(slots)]
            xs, as_, bs = xs[keep], as_[keep], bs[keep]
            stt = st[keep]
        else:
            stt = st
        od = layer.decode(stt, xs.contiguous(), as_.contiguous(), bs.contiguous())
        for i, s in enumerate(live):
            assert same_bits(od[i], want[s][0][have[s]]), (s, have[s], "decode")
            have[s] += 1
        assert not od[len(live)].any()  # the padded lane returns zeros
        step += 1
    for s in slots:
        full = one_pass(layer, *(t[:total] for t in reqs[s]))
        check_row(layer, s, total, full)
    assert int(layer.pos[0]) == 0 and not layer._due.any()


def test_chunked_prefill_resumes_inside_and_on_boundaries(monkeypatch):
    monkeypatch.setenv("SKYRL_ISOEXEC_GDN_CHUNKED_PREFILL", "1")
    layer = make_layer()
    n = 75
    req = request(7, n)
    want = one_pass(layer, *req)
    slot = 3
    st = torch.tensor([slot], device=DEV)
    got = []
    for lo, hi in ((0, 9), (9, 16), (16, 17), (17, 60), (60, 64), (64, 75)):  # inside, onto, off, across, onto, off
        got.append(layer.prefill(st, [slot], req[0][lo:hi], req[1][lo:hi], req[2][lo:hi], [0, hi - lo],
                                 has_initial_state=[lo > 0]))
        part = one_pass(layer, *(t[:hi] for t in req))
        check_row(layer, slot, hi, part)
    assert same_bits(torch.cat(got), want[0])
    # a reissued slot starts from nothing
    layer.release_slot(slot)
    o2 = layer.prefill(st, [slot], req[0][:20], req[1][:20], req[2][:20], [0, 20])
    assert same_bits(o2, want[0][:20])


def test_cpr_state_refuses_engine_owned_tensors():
    from isoexec_amd.ops.gdn.gdn_cpr_state import CprGDN

    with pytest.raises(ValueError, match="owns its state pool"):
        CprGDN(capacity=2, chunk_size=16, num_k_heads=H, head_k_dim=K, num_v_heads=HV, head_v_dim=V, device=DEV,
               ssm_state=torch.zeros(3, HV, V, K, device=DEV), conv_state=torch.zeros(3, D, W - 1, device=DEV), **params())


def test_decode_step_replays_from_a_graph_across_boundaries():
    """The decode step reads nothing on the host (due rows are marked and consumed on the device), so it can be
    recorded once and replayed: 40 replayed steps, crossing chunk boundaries at different steps per request, against
    the same steps run eagerly on a twin layer. Every replay is compared, with host work between replays."""
    eager, graphed = make_layer(), make_layer()
    slots = [0, 1, 2]
    lens = [5, 14, 16]
    total = 60
    reqs = {s: request(300 + s, total) for s in slots}
    x = torch.cat([reqs[s][0][:n] for s, n in zip(slots, lens)])
    a = torch.cat([reqs[s][1][:n] for s, n in zip(slots, lens)])
    b = torch.cat([reqs[s][2][:n] for s, n in zip(slots, lens)])
    qsl = [0] + list(np.cumsum(lens))
    st = torch.tensor(slots, dtype=torch.int64, device=DEV)
    for layer in (eager, graphed):
        layer.prefill(st, slots, x, a, b, qsl)
    have = dict(zip(slots, lens))
    feed = lambda: tuple(torch.stack([reqs[s][j][have[s]] for s in slots]).contiguous() for j in range(3))
    # one eager step on both, so every kernel has been launched once before the capture
    xs, as_, bs = feed()
    assert same_bits(eager.decode(st, xs, as_, bs), graphed.decode(st, xs.clone(), as_.clone(), bs.clone()))
    for s in slots:
        have[s] += 1
    sx, sa, sb = (t.clone() for t in feed())
    graphed.flush_slot_map()
    graph = torch.cuda.CUDAGraph()
    keep = [t.clone() for t in (graphed.ssm_state, graphed.entry_state, graphed.conv_state, graphed.pos, graphed.k_buf,
                                graphed.v_buf, graphed.g_buf, graphed.b_buf, graphed.last_used, graphed._clock)]
    with torch.cuda.graph(graph):
        out = graphed.decode(st, sx, sa, sb)
    for t, k in zip((graphed.ssm_state, graphed.entry_state, graphed.conv_state, graphed.pos, graphed.k_buf, graphed.v_buf,
                     graphed.g_buf, graphed.b_buf, graphed.last_used, graphed._clock), keep):
        t.copy_(k)  # capture may have run nothing or something: start the replays from the saved state
    for step in range(40):
        xs, as_, bs = feed()
        sx.copy_(xs); sa.copy_(as_); sb.copy_(bs)
        graph.replay()
        want = eager.decode(st, xs, as_, bs)
        torch.cuda.synchronize()
        assert same_bits(out, want), step
        for s in slots:
            have[s] += 1
    for t, u in ((graphed.ssm_state, eager.ssm_state), (graphed.entry_state, eager.entry_state), (graphed.pos, eager.pos)):
        assert same_bits(t, u)


def test_wide_heads_take_the_lane_pair_scan_in_the_boundary_pass():
    """K = V = 128 and a pool of more than 128 rows: the state-only boundary scan over the buffer pool then runs in
    the lane-pair layout (every row that is not due a null lane). Same check as above: prefill, decode across
    boundaries, against the one-pass forward."""
    from isoexec_amd.ops.gdn.gdn_cpr import gdn_cpr_fwd
    from isoexec_amd.ops.gdn.gdn_cpr_state import CprGDN
    from isoexec_amd.ops.gdn.gdn_ops import conv_packed

    h, k_, hv, v_, w_, c_ = 2, 128, 4, 128, 4, 16
    d = 2 * h * k_ + hv * v_
    g = cpu_gen(41)
    bf = lambda t: t.to(torch.bfloat16).to(DEV)
    layer = CprGDN(capacity=140, chunk_size=c_, num_k_heads=h, head_k_dim=k_, num_v_heads=hv, head_v_dim=v_, device=DEV,
                   conv_weight=bf(torch.randn(d, w_, generator=g) * 0.4), conv_bias=bf(torch.randn(d, generator=g) * 0.1),
                   A_log=(torch.randn(hv, generator=g) * 0.3).to(DEV), dt_bias=(torch.randn(hv, generator=g) * 0.3).to(DEV))
    total, lens, slots = 40, [13, 16, 30], [5, 6, 7]
    reqs = [(bf(torch.randn(total, d, generator=g)), bf(torch.randn(total, hv, generator=g)), bf(torch.randn(total, hv, generator=g)))
            for _ in slots]
    want = []
    for x, a, b in reqs:
        cu = torch.tensor([0, total], dtype=torch.int32, device=DEV)
        y = conv_packed(x, layer.conv_weight, layer.conv_bias, cu_seqlens=cu)
        q, k, v = layer._split_qkv(y)
        gate, beta = layer._gate_and_beta(a, b)
        u = lambda t: t.unsqueeze(0)
        want.append(gdn_cpr_fwd(u(q), u(k), u(v), u(gate), u(beta), cu_seqlens=cu, chunk_size=c_)[0])
    st = torch.tensor(slots, dtype=torch.int64, device=DEV)
    cat = lambda j: torch.cat([r[j][:n] for r, n in zip(reqs, lens)])
    o = layer.prefill(st, slots, cat(0), cat(1), cat(2), [0] + list(np.cumsum(lens)))
    at = 0
    for i, n in enumerate(lens):
        assert same_bits(o[at:at + n], want[i][:n])
        at += n
    have = list(lens)
    while min(have) < total:
        live = [i for i in range(3) if have[i] < total]
        pick = lambda j: torch.stack([reqs[i][j][have[i]] for i in live]).contiguous()
        od = layer.decode(st[live], pick(0), pick(1), pick(2))
        for row, i in enumerate(live):
            assert same_bits(od[row], want[i][have[i]]), (i, have[i])
            have[i] += 1
    assert not layer._due.any()


def two_layers(monkeypatch, capacity=6):
    """Two layers with their own parameters (as two GDN layers of a model), checkpointing on."""
    from isoexec_amd.ops.gdn import gdn_cpr_state as cpr

    monkeypatch.setenv("SKYRL_ISOEXEC_GDN_CHUNKED_PREFILL", "1")
    monkeypatch.setenv("SKYRL_ISOEXEC_GDN_CPR_APC", "1")
    monkeypatch.setattr(cpr, "CPR_APC_STORE", cpr.CprBoundaryStore(64 << 20))
    layers = [make_layer(capacity), make_layer(capacity)]
    layers[1].conv_weight = (layers[1].conv_weight.float() * 0.9).to(torch.bfloat16)
    layers[1].A_log = layers[1].A_log * 0.8
    assert all(ly._apc for ly in layers)
    return cpr, layers


def test_adopted_prefix_continues_bit_for_bit_as_a_cold_prefill(monkeypatch):
    """A prompt of 75 tokens (C = 16) is prefilled cold by one request; its boundary checkpoints are published under
    prefix keys; two later requests with the same prefix adopt the checkpoints at 64 and at 48 and prefill only the
    rest -- outputs, states and the decode steps after are the cold request's, bit for bit, in both layers."""
    cpr, layers = two_layers(monkeypatch)
    n, total = 75, 84
    req = request(7, total)
    other = request(8, 40)                                         # a second sequence in the same packed call
    want = [one_pass(ly, *(t[:n] for t in req)) for ly in layers]
    st = torch.tensor([1, 2], device=DEV)
    xs, as_, bs = (torch.cat([req[j][:n], other[j]]) for j in range(3))
    for ly, w in zip(layers, want):
        o = ly.prefill(st, [1, 2], xs, as_, bs, [0, n, n + 40])
        assert same_bits(o[:n], w[0])
        # the last two boundaries closed by each sequence were stashed: 48 and 64 of the first, 16 and 32 of the second
        assert {row: [p for p, _, _ in v] for row, v in ly._apc_pending.items()} == \
            {ly.require_row(1): [48, 64], ly.require_row(2): [16, 32]}
    fresh = cpr.cpr_apc_publish(layers, [(1, 64, b"p64"), (1, 48, b"p48"), (2, 32, b"o32"), (1, 32, b"never-stashed")])
    assert fresh == [b"p64", b"p48", b"o32"] and all(not ly._apc_pending for ly in layers)
    pos, entry, conv = cpr.cpr_apc_store().get(b"p64")
    assert pos == 64 and entry.shape == (2, HV, V, K) and entry.dtype is torch.float32 and conv.shape == (2, D, W - 1)
    for j, ly in enumerate(layers):                                # the stored entry IS the chain at the boundary
        assert same_bits(entry[j], one_pass(ly, *(t[:64] for t in req))[1])

    rows = cpr.cpr_apc_adopt_many(layers, [(5, 64, b"p64"), (6, 48, b"p48")])
    assert rows is not None and all(ly.require_row(5) == rows[0] and ly.require_row(6) == rows[1] for ly in layers)
    st2 = torch.tensor([5, 6], device=DEV)
    xs, as_, bs = (torch.cat([req[j][64:n], req[j][48:n]]) for j in range(3))
    for ly, w in zip(layers, want):
        o = ly.prefill(st2, [5, 6], xs, as_, bs, [0, n - 64, n - 64 + n - 48], has_initial_state=[True, True])
        assert same_bits(o[:n - 64], w[0][64:]) and same_bits(o[n - 64:], w[0][48:])
        for slot in (5, 6):
            check_row(ly, slot, n, w)
            assert same_bits(ly.conv_state[ly.require_row(slot)], ly.conv_state[ly.require_row(1)])
    # and the three requests decode alike from here, across the boundary at 80
    st3 = torch.tensor([1, 5, 6], device=DEV)
    for t in range(n, total):
        step = [req[j][t].expand(3, -1).contiguous() for j in range(3)]
        for ly in layers:
            od = ly.decode(st3, *step)
            assert same_bits(od[0], od[1]) and same_bits(od[0], od[2]), t
    for ly in layers:
        full = one_pass(ly, *req)
        for slot in (1, 5, 6):
            check_row(ly, slot, total, full)
    assert cpr.cpr_apc_store().stats()["hits"] == 3


def test_boundaries_whose_window_is_not_inside_the_call_are_not_stashed(monkeypatch):
    cpr, layers = two_layers(monkeypatch)
    ly = layers[0]
    req = request(9, 40)
    st = torch.tensor([3], device=DEV)
    ly.prefill(st, [3], *(t[:14] for t in req), [0, 14])
    assert not ly._apc_pending                                     # no boundary closed
    ly.prefill(st, [3], *(t[14:18] for t in req), [0, 4], has_initial_state=[True])
    assert not ly._apc_pending                                     # 16 closed, but only 2 of its 3 window inputs are here
    ly.prefill(st, [3], *(t[18:40] for t in req), [0, 22], has_initial_state=[True])
    assert [p for p, _, _ in ly._apc_pending[ly.require_row(3)]] == [32]
    ly.release_slot(3)
    assert not ly._apc_pending                                     # a released row keeps no stash


def test_sleep_gives_the_state_back_and_wake_starts_from_nothing(monkeypatch):
    cpr, layers = two_layers(monkeypatch)
    req = request(7, 40)
    st = torch.tensor([1], device=DEV)
    cold = [ly.prefill(st, [1], *req, [0, 40]) for ly in layers]
    cpr.cpr_apc_publish(layers, [(1, 32, b"p32")])
    assert len(cpr.cpr_apc_store()) == 1
    size = cpr.cpr_arena_bytes(layers)
    rows = 7
    per_layer = 2 * rows * HV * V * K * 4 + rows * D * (W - 1) * 2 + rows * C * (KD + HV * V) * 2 + rows * C * HV * 6
    assert per_layer <= size // 2 < per_layer + 7 * 256            # seven views, each on a 256-byte boundary
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    before = torch.cuda.memory_reserved()
    assert cpr.cpr_sleep(layers) == size and all(ly.asleep and ly.ssm_state is None and ly.k_buf is None for ly in layers)
    assert len(cpr.cpr_apc_store()) == 0                           # nothing advertises what no layer could continue
    assert torch.cuda.memory_reserved() <= before - size + (4 << 20)
    with pytest.raises(RuntimeError, match="cpr_wake"):
        layers[0].prefill(st, [1], *req, [0, 40])
    with pytest.raises(RuntimeError, match="cpr_wake"):
        layers[0].decode(st, req[0][:1], req[1][:1], req[2][:1])
    assert cpr.cpr_sleep(layers) == 0                              # asleep already
    assert cpr.cpr_wake(layers) == size and cpr.cpr_wake(layers) == 0
    for ly, o in zip(layers, cold):
        assert not ly.asleep and len(ly.table) == 0 and not ly.ssm_state.any() and not ly.entry_state.any()
        assert not ly.pos.any() and not ly.conv_state.any()
        with pytest.raises(RuntimeError):
            ly.prefill(st, [1], *(t[32:] for t in req), [0, 8], has_initial_state=[True])   # nobody resumes over a sleep
        assert same_bits(ly.prefill(st, [1], *req, [0, 40]), o)    # the same request, cold, gives the same bits


def test_arena_keeps_its_address_and_a_captured_step_replays_after_the_wake(monkeypatch):
    """With SKYRL_ISOEXEC_GDN_CPR_SLEEP=1 the state lives in a reserved address range: sleep unmaps its memory (the
    device's free memory grows by the arena), wake maps fresh zeroed memory at the same addresses, and a decode step
    captured into a graph BEFORE the sleep replays AFTER the wake with the bits of an eager twin."""
    from isoexec_amd.ops.gdn import gdn_cpr_state as cpr

    monkeypatch.setenv("SKYRL_ISOEXEC_GDN_CPR_SLEEP", "1")
    monkeypatch.setattr(cpr, "CPR_APC_STORE", cpr.CprBoundaryStore(1 << 20))
    graphed = make_layer()
    monkeypatch.delenv("SKYRL_ISOEXEC_GDN_CPR_SLEEP")
    eager = make_layer()
    assert graphed._device_arena is not None and eager._device_arena is None
    names = ("ssm_state", "conv_state", "entry_state", "k_buf", "v_buf", "g_buf", "b_buf")
    where = {n: getattr(graphed, n).data_ptr() for n in names}
    assert where["ssm_state"] == graphed._device_arena.base and all(p % 256 == 0 for p in where.values())

    slots, lens, total = [0, 1, 2], [5, 14, 16], 40
    reqs = {s: request(500 + s, total) for s in slots}
    st = torch.tensor(slots, dtype=torch.int64, device=DEV)
    qsl = [0] + list(np.cumsum(lens))
    packed = [torch.cat([reqs[s][j][:n] for s, n in zip(slots, lens)]) for j in range(3)]

    def prefill(layer):
        return layer.prefill(st, slots, *packed, qsl)

    assert same_bits(prefill(graphed), prefill(eager))
    have = dict(zip(slots, lens))
    feed = lambda: tuple(torch.stack([reqs[s][j][have[s]] for s in slots]).contiguous() for j in range(3))
    xs, as_, bs = feed()
    assert same_bits(graphed.decode(st, xs.clone(), as_.clone(), bs.clone()), eager.decode(st, xs, as_, bs))  # warm
    for s in slots:
        have[s] += 1
    sx, sa, sb = (t.clone() for t in feed())
    graphed.flush_slot_map()
    keep = [getattr(graphed, n).clone() for n in names] + [graphed.pos.clone(), graphed.last_used.clone(), graphed._clock.clone()]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = graphed.decode(st, sx, sa, sb)
    for t, k in zip([getattr(graphed, n) for n in names] + [graphed.pos, graphed.last_used, graphed._clock], keep):
        t.copy_(k)

    def replay_steps(n):
        for step in range(n):
            xs, as_, bs = feed()
            sx.copy_(xs); sa.copy_(as_); sb.copy_(bs)
            graph.replay()
            want = eager.decode(st, xs, as_, bs)
            torch.cuda.synchronize()
            assert same_bits(out, want), step
            for s in slots:
                have[s] += 1

    replay_steps(6)
    # ---- sleep: the memory goes back to the device, the addresses stay
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    size = cpr.cpr_sleep([graphed])
    assert size > 0 and graphed.asleep and not graphed._device_arena.mapped
    assert torch.cuda.mem_get_info()[0] >= free_before + graphed._device_arena.nbytes - (2 << 20)
    with pytest.raises(RuntimeError, match="cpr_wake"):
        graphed.decode(st, sx, sa, sb)
    # ---- wake: zeroed state at the same addresses, every row released; the same requests start over on both layers
    assert cpr.cpr_wake([graphed]) == size and graphed._device_arena.mapped
    assert {n: getattr(graphed, n).data_ptr() for n in names} == where
    assert not graphed.ssm_state.any() and not graphed.k_buf.any() and len(graphed.table) == 0
    eager.reset()
    assert same_bits(prefill(graphed), prefill(eager))
    for s, n in zip(slots, lens):
        have[s] = n
    graphed.flush_slot_map()
    replay_steps(20)                                               # the graph captured before the sleep, across boundaries
    for t, u in ((graphed.ssm_state, eager.ssm_state), (graphed.entry_state, eager.entry_state), (graphed.pos, eager.pos)):
        assert same_bits(t, u)
    # ---- the arena ends with an explicit call (nothing may view it any more)
    arena = graphed._device_arena
    cpr.cpr_sleep([graphed])
    arena.destroy()
