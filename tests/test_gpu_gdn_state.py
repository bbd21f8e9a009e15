"""GPU parity of the GatedDeltaNet layer core with its state pools: prefill, decode, resume, eviction.

The oracle runs each request as ONE sequence from a zero state (conv -> l2norm -> gate -> scan); the
layer sees the same tokens cut into a packed prefill and single-token decode steps, mixed with other
requests and with padded lanes. Outputs and both state pools must match bit for bit.
"""

import numpy as np
import pytest
import torch

from _util import DevicePrims, bf16_to_np, cpu_gen, np_bits, np_to_bf16, same_bits
from oracle import gdn as o_gdn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
H, K, HV, V, W = 2, 64, 4, 64, 4
KD = H * K
D = 2 * KD + HV * V


@pytest.fixture(scope="module")
def dprims():
    return DevicePrims(DEV)


@pytest.fixture()
def params():
    g = cpu_gen(11)
    bf = lambda t: t.to(torch.bfloat16)
    return dict(
        conv_weight=bf(torch.randn(D, W, generator=g) * 0.4),
        conv_bias=bf(torch.randn(D, generator=g) * 0.1),
        A_log=torch.randn(HV, generator=g) * 0.3,
        dt_bias=torch.randn(HV, generator=g) * 0.3,
    )


def make_layer(params, capacity, **kw):
    from isoexec_amd.ops.gdn.gdn_recurrent_state import RecurrentGDN

    return RecurrentGDN(capacity=capacity, conv_weight=params["conv_weight"].to(DEV), conv_bias=params["conv_bias"].to(DEV),
                        A_log=params["A_log"].to(DEV), dt_bias=params["dt_bias"].to(DEV), num_k_heads=H, head_k_dim=K,
                        num_v_heads=HV, head_v_dim=V, device=DEV, **kw)


def request(seed, T):
    g = cpu_gen(seed)
    bf = lambda t: t.to(torch.bfloat16)
    return bf(torch.randn(T, D, generator=g)), bf(torch.randn(T, HV, generator=g)), bf(torch.randn(T, HV, generator=g))


def oracle_request(x, a, b, params, prims):
    """The whole request as one sequence. Returns (o [T,HV,V], conv history [D,W-1], state [HV,V,K])."""
    f = bf16_to_np
    y, conv = o_gdn.causal_conv(f(x), f(params["conv_weight"]), f(params["conv_bias"]), prims=prims)
    T = y.shape[0]
    q = o_gdn.l2norm(y[:, :KD].reshape(T, H, K))
    k = o_gdn.l2norm(y[:, KD : 2 * KD].reshape(T, H, K))
    v = y[:, 2 * KD :].reshape(T, HV, V)
    g, beta = o_gdn.gate_and_beta(f(a), f(b), params["A_log"].numpy(), params["dt_bias"].numpy(), prims=prims)
    state = np.zeros((HV, V, K), np.float32)
    o = o_gdn.scan(q, k, v, g, beta, state, io_bf16=True, prims=prims)
    return o, conv, state


def pack(reqs, lo, hi):
    """Tokens [lo_i, hi_i) of each request, packed. Returns (x, a, b, qsl)."""
    xs, as_, bs, qsl = [], [], [], [0]
    for (x, a, b), s, e in zip(reqs, lo, hi):
        xs.append(x[s:e]); as_.append(a[s:e]); bs.append(b[s:e]); qsl.append(qsl[-1] + e - s)
    d = lambda parts: torch.cat(parts).to(DEV)
    return d(xs), d(as_), d(bs), qsl


def eq_bits(dev_tensor, want_np):
    got = dev_tensor.float().cpu().numpy() if dev_tensor.dtype is torch.bfloat16 else dev_tensor.cpu().numpy()
    return np.array_equal(np_bits(got), np_bits(np.ascontiguousarray(want_np, dtype=np.float32)))


def test_prefill_then_decode_matches_one_sequence_per_request(params, dprims):
    lens, steps = [37, 1, 2, 70], 6
    slots = [901, 17, 40000, 5]
    reqs = [request(100 + i, n + steps) for i, n in enumerate(lens)]
    want = [oracle_request(*r, params, dprims) for r in reqs]
    layer = make_layer(params, capacity=6)
    x, a, b, qsl = pack(reqs, [0] * 4, lens)
    o = layer.prefill(torch.tensor(slots, device=DEV), slots, x, a, b, qsl)
    for i, n in enumerate(lens):
        assert eq_bits(o[qsl[i] : qsl[i + 1]], want[i][0][:n]), f"prefill request {i}"
    # Decode with two padded lanes: an id no request holds and one outside the map.
    lane_slots = torch.tensor([slots[0], 123, slots[1], slots[2], 10**9, slots[3]], device=DEV)
    lanes = [0, None, 1, 2, None, 3]
    pad = request(999, 1)
    for s in range(steps):
        parts = [tuple(t[lens[r] + s : lens[r] + s + 1] for t in reqs[r]) if r is not None else pad for r in lanes]
        xd, ad, bd = (torch.cat([p[j] for p in parts]).to(DEV) for j in range(3))
        od = layer.decode(lane_slots, xd, ad, bd)
        for lane, r in enumerate(lanes):
            if r is None:
                assert not od[lane].any(), f"padded lane {lane} must return zeros"
            else:
                assert eq_bits(od[lane], want[r][0][lens[r] + s]), f"decode step {s} request {r}"
    for r, slot in enumerate(slots):
        row = layer.require_row(slot)
        assert eq_bits(layer.ssm_state[row], want[r][2]), f"ssm state of request {r}"
        assert eq_bits(layer.conv_state[row], want[r][1]), f"conv state of request {r}"
    assert not layer.ssm_state[0].any() and not layer.conv_state[0].any(), "the null row is never written"
    used = layer.last_used.cpu().tolist()
    assert all(used[layer.require_row(s)] == 4 + steps for s in slots)


def test_chunked_prefill_resumes_bitwise(params, dprims, monkeypatch):
    monkeypatch.setenv("SKYRL_ISOEXEC_GDN_CHUNKED_PREFILL", "1")
    lens = [50, 9, 33]
    cuts = [[0, 20, 21, 50], [0, 9, 9, 9], [0, 1, 30, 33]]  # the second request finishes in the first chunk
    slots = [3, 4, 5]
    reqs = [request(200 + i, n) for i, n in enumerate(lens)]
    want = [oracle_request(*r, params, dprims) for r in reqs]
    whole = make_layer(params, capacity=4)
    x, a, b, qsl = pack(reqs, [0] * 3, lens)
    o_whole = whole.prefill(torch.tensor(slots, device=DEV), slots, x, a, b, qsl)
    chunked = make_layer(params, capacity=4)
    outs = [[] for _ in reqs]
    for c in range(3):
        live = [i for i in range(3) if cuts[i][c + 1] > cuts[i][c]]
        x, a, b, q2 = pack([reqs[i] for i in live], [cuts[i][c] for i in live], [cuts[i][c + 1] for i in live])
        sl = [slots[i] for i in live]
        o = chunked.prefill(torch.tensor(sl, device=DEV), sl, x, a, b, q2, has_initial_state=[c > 0] * len(live))
        for j, i in enumerate(live):
            outs[i].append(o[q2[j] : q2[j + 1]])
    for i in range(3):
        got = torch.cat(outs[i])
        assert same_bits(got, o_whole[qsl[i] : qsl[i + 1]]) and eq_bits(got, want[i][0])
        rw, rc = whole.require_row(slots[i]), chunked.require_row(slots[i])
        assert same_bits(whole.ssm_state[rw], chunked.ssm_state[rc]) and eq_bits(chunked.ssm_state[rc], want[i][2])
        assert same_bits(whole.conv_state[rw], chunked.conv_state[rc]) and eq_bits(chunked.conv_state[rc], want[i][1])
    # With resume off, a re-presented slot starts over from nothing.
    monkeypatch.setenv("SKYRL_ISOEXEC_GDN_CHUNKED_PREFILL", "0")
    x, a, b, q2 = pack(reqs[:1], [0], [lens[0]])
    again = chunked.prefill(torch.tensor(slots[:1], device=DEV), slots[:1], x, a, b, q2)
    assert eq_bits(again, want[0][0])


def test_eviction_and_release_give_the_newcomer_a_clean_row(params, dprims):
    layer = make_layer(params, capacity=2)
    reqs = [request(300 + i, 12) for i in range(4)]
    want = [oracle_request(*r, params, dprims) for r in reqs]

    def prefill(i, slot):
        x, a, b, qsl = pack([reqs[i]], [0], [12])
        return layer.prefill(torch.tensor([slot], device=DEV), [slot], x, a, b, qsl)

    assert eq_bits(prefill(0, 10), want[0][0]) and eq_bits(prefill(1, 11), want[1][0])
    # One decode step touches slot 10 only, so slot 11 becomes the least recently used.
    x, a, b = (t.to(DEV) for t in request(1, 1))
    layer.decode(torch.tensor([10], device=DEV), x, a, b)
    row11 = layer.require_row(11)
    assert eq_bits(prefill(2, 12), want[2][0]) and layer.require_row(12) == row11
    assert eq_bits(layer.ssm_state[row11], want[2][2]) and eq_bits(layer.conv_state[row11], want[2][1])
    with pytest.raises(RuntimeError, match="no mapped row"):
        layer.require_row(11)
    # The evicted request's lane now resolves to the null row.
    assert not layer.decode(torch.tensor([11], device=DEV), x, a, b).any()
    layer.release_slot(12)
    assert eq_bits(prefill(3, 13), want[3][0]) and layer.require_row(13) == row11
    from isoexec_amd.ops.gdn.gdn_recurrent_state import invalidate_all_states

    assert invalidate_all_states([layer]) == 2
    assert not layer.ssm_state.any() and not layer.conv_state.any()
    assert not layer.decode(torch.tensor([13], device=DEV), x, a, b).any()


def test_native_state_indexes_the_engines_tensors_by_block_id(params, dprims):
    ssm = torch.zeros(9, HV, V, K, device=DEV)
    conv = torch.zeros(9, D, W - 1, dtype=torch.bfloat16, device=DEV)
    layer = make_layer(params, capacity=8, ssm_state=ssm, conv_state=conv)
    reqs = [request(400 + i, 20) for i in range(2)]
    want = [oracle_request(*r, params, dprims) for r in reqs]
    blocks = [7, 3]
    ssm[7].fill_(5.0)  # a recycled block holds stale state; a fresh prefill must not see it
    x, a, b, qsl = pack(reqs, [0, 0], [16, 16])
    o = layer.prefill(torch.tensor(blocks, device=DEV), blocks, x, a, b, qsl)
    assert eq_bits(o[:16], want[0][0][:16]) and eq_bits(o[16:], want[1][0][:16])
    ids = torch.tensor([3, 0, 7, 99], device=DEV)  # block 0 and an out-of-range id are padding
    for s in range(16, 20):
        parts = [reqs[1], reqs[0], reqs[0], reqs[0]]
        xd, ad, bd = (torch.cat([p[j][s : s + 1] for p in parts]).to(DEV) for j in range(3))
        od = layer.decode(ids, xd, ad, bd)
        assert eq_bits(od[0], want[1][0][s]) and eq_bits(od[2], want[0][0][s])
        assert not od[1].any() and not od[3].any()
    assert eq_bits(ssm[7], want[0][2]) and eq_bits(conv[3], want[1][1]) and not ssm[0].any()
    with pytest.raises(RuntimeError, match="out of range"):
        layer.prefill(torch.tensor([9], device=DEV), [9], x[:16], a[:16], b[:16], [0, 16])


def test_compact_state_index_form_equals_the_full_map(dprims):
    """One row per sequence (loaded first, stored last) is the [N, Tmax] map with only those two
    columns set."""
    from isoexec_amd.ops.gdn.gdn_ops import gdn_recurrent_kernel

    g = cpu_gen(5)
    lens = [5, 1, 64, 33]
    T = sum(lens)
    bf = lambda t: t.to(torch.bfloat16).to(DEV)
    q = torch.nn.functional.normalize(torch.randn(1, T, H, K, generator=g), dim=-1)
    k = torch.nn.functional.normalize(torch.randn(1, T, H, K, generator=g), dim=-1)
    v = torch.randn(1, T, HV, V, generator=g)
    gate = -torch.nn.functional.softplus(torch.randn(1, T, HV, generator=g))
    beta = torch.sigmoid(torch.randn(1, T, HV, generator=g))
    cu = torch.tensor(np.cumsum([0] + lens), dtype=torch.int32, device=DEV)
    rows = torch.tensor([2, 0, 4, 1], dtype=torch.int32, device=DEV)  # the second sequence is a null lane
    full = torch.zeros(4, max(lens), dtype=torch.int32)
    for i, (r, n) in enumerate(zip(rows.tolist(), lens)):
        full[i, 0] = r
        full[i, n - 1] = r
    start = torch.randn(5, HV, V, K, generator=g)
    pools, outs = [], []
    for idx in (rows, full.to(DEV)):
        pool = start.clone().to(DEV)
        outs.append(gdn_recurrent_kernel(bf(q), bf(k), bf(v), gate.to(DEV), bf(beta), ssm_state=pool, state_indices=idx, cu_seqlens=cu))
        pools.append(pool)
    assert same_bits(outs[0], outs[1]) and same_bits(pools[0], pools[1])
    assert same_bits(pools[0][3], start[3].to(DEV)) and not same_bits(pools[0][4], start[4].to(DEV))
    # Rows held per lane group (1, 2, 4) and the time tile are staging choices: same bits.
    for rpl in (1, 2, 4):
        for tt in (16, 64):
            pool = start.clone().to(DEV)
            got = gdn_recurrent_kernel(bf(q), bf(k), bf(v), gate.to(DEV), bf(beta), ssm_state=pool, state_indices=rows,
                                       cu_seqlens=cu, time_tile=tt | (rpl << 8))
            assert same_bits(got, outs[0]) and same_bits(pool, pools[0]), (rpl, tt)


def test_lane_pair_layout_gives_the_same_bits():
    """K = 128: a state row may be held by a pair of lanes (64 elements each, code 16 in bits 8.. of time_tile)
    instead of 16 lanes with 8 each. Same slices, same chains, same tree -- outputs and final states must be
    bit-equal to the 16-lane layout for every time tile, ragged lengths and a null lane included."""
    from isoexec_amd.ops.gdn.gdn_ops import gdn_recurrent_kernel

    Hh, Kk, HVv, Vv = 2, 128, 4, 128
    g = cpu_gen(11)
    lens = [5, 1, 64, 33, 130]
    T = sum(lens)
    bf = lambda t: t.to(torch.bfloat16).to(DEV)
    q = torch.nn.functional.normalize(torch.randn(1, T, Hh, Kk, generator=g), dim=-1)
    k = torch.nn.functional.normalize(torch.randn(1, T, Hh, Kk, generator=g), dim=-1)
    v = torch.randn(1, T, HVv, Vv, generator=g)
    gate = -torch.nn.functional.softplus(torch.randn(1, T, HVv, generator=g))
    beta = torch.sigmoid(torch.randn(1, T, HVv, generator=g))
    cu = torch.tensor(np.cumsum([0] + lens), dtype=torch.int32, device=DEV)
    rows = torch.tensor([2, 0, 4, 1, 5], dtype=torch.int32, device=DEV)  # the second sequence is a null lane
    start = torch.randn(6, HVv, Vv, Kk, generator=g)
    ref_pool = start.clone().to(DEV)
    ref = gdn_recurrent_kernel(bf(q), bf(k), bf(v), gate.to(DEV), bf(beta), ssm_state=ref_pool, state_indices=rows,
                               cu_seqlens=cu, time_tile=16 | (1 << 8))
    for tt in (8, 16, 64):
        pool = start.clone().to(DEV)
        got = gdn_recurrent_kernel(bf(q), bf(k), bf(v), gate.to(DEV), bf(beta), ssm_state=pool, state_indices=rows,
                                   cu_seqlens=cu, time_tile=tt | (16 << 8))
        assert same_bits(got, ref) and same_bits(pool, ref_pool), tt
    assert same_bits(ref_pool[3], start[3].to(DEV)) and not same_bits(ref_pool[5], start[5].to(DEV))


def test_fused_row_resolver_equals_the_eager_chain():
    """Slot ids -> rows in one launch (reference gdn_cpr_rows.py) against the index expression it replaces
    (gdn_recurrent_state.py:271-284): clamped lookups for a private pool, identity with out-of-range ids on
    row 0 for the engine's own blocks, both id widths, and the use stamp of the decode step."""
    from isoexec_amd.ops.gdn.gdn_cpr_rows import cpr_resolve_rows, resolve_and_stamp

    g = cpu_gen(77)
    map_n, rows_n = 50, 9
    slot2row = torch.randint(0, rows_n, (map_n,), generator=g, dtype=torch.int64).to(DEV)
    ids = torch.tensor([3, 49, 50, 1000, -1, -7, 0, 3, 17], dtype=torch.int64)
    for dt in (torch.int64, torch.int32):
        slots = ids.to(dt).to(DEV)
        want = slot2row[slots.long().clamp(0, map_n - 1)]
        r64, r32 = cpr_resolve_rows(slots, slot2row)
        assert r64.dtype is torch.int64 and r32.dtype is torch.int32
        assert torch.equal(r64, want) and torch.equal(r32.long(), want)
        # the engine's block ids are the rows: ids outside [0, blocks) read the null row
        nat = resolve_and_stamp(slots, blocks=40)
        s = slots.long()
        assert torch.equal(nat.long(), torch.where(s < 40, s, torch.zeros_like(s)).clamp(min=0))
    # every slot vector a replayed decode step can present, through the pool's own seam
    from test_gdn_rows_host import make_pool, rows_eager, slot_vectors

    rg = make_pool()
    rg.slot2row = rg.slot2row.to(DEV)
    for sv in slot_vectors(rg.slot2row.numel()):
        rows, rows32 = rg._rows_pair(sv.to(DEV))
        want = rows_eager(rg.slot2row, sv.to(DEV))
        assert rows.dtype is torch.int64 and rows32.dtype is torch.int32
        assert torch.equal(rows, want) and torch.equal(rows32.long(), want)
    # the use stamp: clock += 1, last_used[rows] = clock, twice in a row, duplicates included
    last_used = torch.zeros(rows_n, dtype=torch.int64, device=DEV)
    clock = torch.full((), 41, dtype=torch.int64, device=DEV)
    want_used = last_used.clone()
    for step, sl in enumerate((ids[:4], ids[4:])):
        slots = sl.to(DEV)
        rows = slot2row[slots.clamp(0, map_n - 1)]
        want_used[rows] = 42 + step
        got = resolve_and_stamp(slots, slot2row=slot2row, last_used=last_used, clock=clock)
        assert torch.equal(got.long(), rows)
        assert int(clock) == 42 + step and torch.equal(last_used, want_used)
    # shapes the resolver does not serve hand the caller back to the eager chain
    assert cpr_resolve_rows(ids.view(3, 3).to(DEV), slot2row) is None
    assert cpr_resolve_rows(ids.to(DEV), slot2row.int()) is None
    assert cpr_resolve_rows(torch.empty(0, dtype=torch.int64, device=DEV), slot2row)[0].numel() == 0
