"""The boundary store and the adoption of stored checkpoints, on the host with stand-in layers (no GPU). The
contracts are the reference's (gdn_cpr_state.py:96-196 store, :222-287 adoption; its own CPU tests
ops/gdn/tests/test_cpr_apc_adopt_many_cpu.py: one assignment per layer per step, exact state, a miss touches
nothing, refusals of the one-request door)."""

from collections import OrderedDict

import pytest
import torch

from isoexec_amd.ops.gdn import gdn_cpr_state as cpr


class Layer:
    def __init__(self, capacity=8):
        self.chunk_size = 64
        self.ssm_state = torch.zeros(capacity + 1, 1, 2, 2)
        self.conv_state = torch.zeros(capacity + 1, 3, 2, dtype=torch.bfloat16)
        self.entry_state = torch.zeros_like(self.ssm_state)
        self.k_buf = torch.zeros(1, dtype=torch.bfloat16)
        self.pos = torch.zeros(capacity + 1, dtype=torch.long)
        self._apc_pending = {r: [(64, None, None)] for r in range(1, capacity + 1)}
        self._slot2row = OrderedDict()
        self._free = list(range(1, capacity + 1))
        self.assign_calls = 0

    def _assign_many(self, slots):
        self.assign_calls += 1
        rows = []
        for slot in slots:
            if int(slot) not in self._slot2row:
                self._slot2row[int(slot)] = self._free.pop()
            rows.append(self._slot2row[int(slot)])
        return rows


@pytest.fixture
def stocked(monkeypatch):
    layers = [Layer(), Layer()]
    store = cpr.CprBoundaryStore(1 << 20, say=lambda msg: None)
    g = torch.Generator().manual_seed(3)
    entries = {key: torch.randn(2, 1, 2, 2, generator=g) * 7 for key in (b"a", b"b")}     # not bf16-representable
    convs = {key: (torch.arange(12, dtype=torch.float32).reshape(2, 3, 2) + off).to(torch.bfloat16)
             for key, off in ((b"a", 0), (b"b", 20))}
    assert store.put(b"a", 64, entries[b"a"], convs[b"a"]) and store.put(b"b", 128, entries[b"b"], convs[b"b"])
    monkeypatch.setattr(cpr, "CPR_APC_STORE", store)
    return layers, entries, convs


def test_adoption_assigns_once_per_layer_and_installs_exact_state(stocked):
    layers, entries, convs = stocked
    items = [(101, 64, b"a"), (102, 128, b"b"), (103, 64, b"a")]
    rows = cpr.cpr_apc_adopt_many(layers, items)
    assert rows == [8, 7, 6] and [ly.assign_calls for ly in layers] == [1, 1]
    for j, ly in enumerate(layers):
        entry = torch.stack([entries[key][j] for _, _, key in items])
        assert torch.equal(ly.entry_state[rows], entry)                                     # the fp32 chain, unrounded
        assert torch.equal(ly.ssm_state[rows], entry.to(torch.bfloat16).to(torch.float32))  # the running state: its snapshot
        assert not torch.equal(ly.ssm_state[rows], entry)
        assert torch.equal(ly.conv_state[rows], torch.stack([convs[key][j] for _, _, key in items]))
        assert ly.pos[rows].tolist() == [64, 128, 64] and all(r not in ly._apc_pending for r in rows)


def test_a_miss_touches_nothing(stocked):
    layers, _, _ = stocked
    assert cpr.cpr_apc_adopt_many(layers, [(101, 64, b"a"), (102, 128, b"missing")]) is None
    assert [ly.assign_calls for ly in layers] == [0, 0] and not any(ly._slot2row for ly in layers)
    assert all(not ly.ssm_state.any() and not ly.entry_state.any() for ly in layers)


def test_refusals_of_the_one_request_door(stocked):
    layers, _, _ = stocked
    assert cpr.cpr_apc_adopt(layers, 101, 64, b"a")
    assert not cpr.cpr_apc_adopt(layers, 102, 65, b"a")         # not a boundary
    assert not cpr.cpr_apc_adopt(layers, 103, 128, b"a")        # stored at another position
    assert not cpr.cpr_apc_adopt(layers, 104, 64, b"missing")
    assert not cpr.cpr_apc_adopt(layers[:1], 105, 64, b"a")     # stored for two layers, asked for one
    assert cpr.cpr_apc_adopt_many(layers, []) == [] and cpr.cpr_apc_adopt_many([], [(1, 64, b"a")]) is None


def test_layers_out_of_step_are_an_error(stocked):
    layers, _, _ = stocked
    layers[1]._free.pop()                                        # the second pool hands out another row
    with pytest.raises(RuntimeError, match="out of step"):
        cpr.cpr_apc_adopt_many(layers, [(101, 64, b"a")])


def pair(nbytes_entry=4000, fill=0.0):
    return torch.full((1, nbytes_entry // 4), fill), torch.zeros(1, 48, dtype=torch.bfloat16)   # 4000 + 96 bytes


def test_store_evicts_least_recently_used_within_its_budget():
    said = []
    store = cpr.CprBoundaryStore(3 * 4096, say=said.append)
    for key in (b"k1", b"k2", b"k3"):
        assert store.put(key, 64, *pair())
    assert store.nbytes == 3 * 4096 and len(store) == 3
    assert not store.put(b"k1", 64, *pair(fill=9.0))             # a known key is refreshed, not replaced
    assert store.get(b"k1")[1][0, 0] == 0.0
    assert store.get(b"k2") is not None                          # order of use is now k3, k1, k2
    assert store.put(b"k4", 128, *pair())
    assert b"k3" not in store and b"k1" in store and b"k2" in store and store.nbytes == 3 * 4096
    assert store.get(b"k3") is None
    assert store.stats() == {"entries": 3, "MiB": 0.0, "hits": 2, "misses": 1, "stores": 4, "evictions": 1,
                             "full_refusals": 0, "oversize_refusals": 0}
    assert not store.put(b"huge", 64, *pair(nbytes_entry=16000)) and not store.put(b"huge2", 64, *pair(nbytes_entry=16000))
    assert len(said) == 1 and "nothing can be stored" in said[0] and len(store) == 3   # refused, said once, nothing evicted


def test_append_only_store_refuses_instead_of_evicting_and_clear_runs_the_hooks(monkeypatch):
    said = []
    store = cpr.CprBoundaryStore(2 * 4096, evict=False, say=said.append)
    assert store.put(b"k1", 64, *pair()) and store.put(b"k2", 64, *pair())
    assert not store.put(b"k3", 64, *pair()) and not store.put(b"k4", 64, *pair())
    assert store.full_refusals == 2 and len(said) == 1 and "append-only" in said[0]
    assert b"k1" in store and b"k2" in store
    calls = []
    monkeypatch.setattr(cpr, "CPR_APC_ON_CLEAR", [lambda: calls.append(len(store))])
    store.clear()
    assert calls == [0] and store.nbytes == 0 and store.put(b"k3", 64, *pair())   # the hook sees the store empty

    def failing():
        raise OSError("index not retracted")

    monkeypatch.setattr(cpr, "CPR_APC_ON_CLEAR", [failing])
    with pytest.raises(OSError):
        store.clear()                                            # a failed retraction is not swallowed


def test_environment_names_mode_and_budget(monkeypatch):
    monkeypatch.delenv("SKYRL_ISOEXEC_GDN_CPR_APC", raising=False)
    monkeypatch.delenv("SKYRL_ISOEXEC_GDN_CPR_APC_MB", raising=False)
    assert not cpr.cpr_apc_enabled() and not cpr.cpr_apc_shared_mode() and cpr.cpr_apc_budget_bytes() == 1 << 30
    monkeypatch.setenv("SKYRL_ISOEXEC_GDN_CPR_APC", "1")
    assert cpr.cpr_apc_enabled() and not cpr.cpr_apc_shared_mode()
    monkeypatch.setenv("SKYRL_ISOEXEC_GDN_CPR_APC", "shm")
    monkeypatch.setenv("SKYRL_ISOEXEC_GDN_CPR_APC_MB", "0.5")
    assert cpr.cpr_apc_enabled() and cpr.cpr_apc_shared_mode() and cpr.cpr_apc_budget_bytes() == 1 << 19
    monkeypatch.setattr(cpr, "CPR_APC_STORE", None)
    store = cpr.cpr_apc_store()
    assert store is cpr.cpr_apc_store() and not store.evict and store.budget == 1 << 19
    store.put(b"k", 64, *pair())
    cpr.cpr_apc_store_invalidate()
    assert len(store) == 0


def test_publish_takes_what_every_layer_stashed(monkeypatch):
    monkeypatch.setattr(cpr, "CPR_APC_STORE", cpr.CprBoundaryStore(1 << 20))
    layers = [Layer(), Layer()]
    for ly in layers:
        ly._slot2row.update({11: 3, 12: 4})
        ly._apc_pending = {3: [(64, torch.full((1, 2, 2), 1.0), torch.zeros(3, 2)), (128, torch.full((1, 2, 2), 2.0), torch.ones(3, 2))],
                           4: [(64, torch.full((1, 2, 2), 3.0), torch.zeros(3, 2))]}
    del layers[1]._apc_pending[4]                                # the second layer stashed nothing for slot 12
    fresh = cpr.cpr_apc_publish(layers, [(11, 128, b"p128"), (11, 192, b"p192"), (12, 64, b"q64"), (99, 64, b"nobody")])
    assert fresh == [b"p128"]
    pos, entry, conv = cpr.cpr_apc_store().get(b"p128")
    assert pos == 128 and entry.shape == (2, 1, 2, 2) and conv.shape == (2, 3, 2) and bool((entry == 2.0).all())
    assert all(not ly._apc_pending for ly in layers)             # a stash lives for one step
    assert cpr.cpr_apc_publish(layers, [(11, 128, b"p128")]) == []
