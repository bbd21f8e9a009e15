"""Host bookkeeping of the GatedDeltaNet state pool (no device needed).

Follows the lifecycle cases the reference tests for ``RecurrentGDN`` (isoexec/ops/gdn/
gdn_recurrent_state.py:301-598): row 0 is never handed out, a batch's evictions come from one LRU
snapshot with rows claimed by the batch excluded, exhaustion never leaves a half-edited table, and
every edit reaches the device-map outbox.
"""

import numpy as np
import pytest
import torch

from isoexec_amd.ops.gdn.gdn_recurrent_state import (
    RecurrentGDN,
    SlotTable,
    chunked_prefill_enabled,
    flush_slot_maps,
    invalidate_all_states,
)


def test_rows_come_from_the_free_list_and_never_include_the_null_row():
    t = SlotTable(capacity=4, map_size=100)
    rows = t.assign_many([10, 20, 30, 40])
    assert sorted(rows) == [1, 2, 3, 4] and 0 not in rows and rows == [4, 3, 2, 1]
    assert t.assign_many([]) == []
    assert t.assign_many([20]) == [3]  # a slot that holds a row keeps it
    assert list(t.row_of) == [10, 30, 40, 20]  # and becomes the most recent
    assert t.require_row(30) == 2 and t.holds(30) and not t.holds(31) and len(t) == 4
    with pytest.raises(RuntimeError, match="LIVE state slot 31 has no mapped row"):
        t.require_row(31)
    with pytest.raises(RuntimeError, match="exceeds the slot map"):
        t.assign_many([100])
    with pytest.raises(RuntimeError, match="exceeds the slot map"):
        t.assign_many([-1])


def test_eviction_uses_one_snapshot_and_skips_rows_claimed_by_the_batch():
    t = SlotTable(capacity=3, map_size=100)
    assert t.assign_many([1, 2, 3]) == [3, 2, 1]
    calls = []

    def snapshot():
        calls.append(1)
        return [0, 7, 5, 9]  # last_used per row; row 0 is ignored

    # Slot 3 keeps row 1 (claimed); newcomers take the LRU rows 2 (tick 5) then 3 (tick 9), never row 1.
    rows = t.assign_many([3, 8, 9], lru_snapshot=snapshot)
    assert rows == [1, 2, 3] and len(calls) == 1
    assert dict(t.row_of) == {3: 1, 8: 2, 9: 3}
    keys, vals = t.drain_outbox()
    edits = dict(zip(keys.tolist(), vals.tolist()))
    assert edits[2] == 0 and edits[1] == 0 and edits[8] == 2 and edits[9] == 3 and edits[3] == 1
    assert t.drain_outbox() is None
    # Ties break toward the lower row, like a first-minimum argmin.
    assert t.assign_many([50], lru_snapshot=lambda: [0, 4, 4, 4]) == [1]
    with pytest.raises(RuntimeError, match="exceeds the 3 evictable state rows"):
        t.assign_many([60, 61, 62, 63], lru_snapshot=lambda: [0, 1, 2, 3])
    full = SlotTable(capacity=1, map_size=10)
    full.assign_many([1])
    with pytest.raises(RuntimeError, match="no eviction order"):
        full.assign_many([2])


def test_driver_managed_pool_refuses_before_editing_anything():
    t = SlotTable(capacity=2, map_size=100, driver_managed=True)
    t.assign_many([1, 2])
    before = (dict(t.row_of), list(t.free), dict(t.outbox))
    with pytest.raises(RuntimeError, match="driver-managed state pool exhausted"):
        t.assign_many([2, 3], lru_snapshot=lambda: [0, 0, 0])
    assert (dict(t.row_of), list(t.free), dict(t.outbox)) == before
    assert t.release(1) == 2
    assert t.assign_many([2, 3]) == [1, 2]


def test_release_and_rebind():
    t = SlotTable(capacity=3, map_size=100)
    t.assign_many([5, 6])
    t.drain_outbox()
    assert t.release(7) is None
    assert t.release(5) == 3 and t.free[-1] == 3 and not t.holds(5)
    assert t.outbox == {5: 0}
    assert t.assign_many([9]) == [3]  # the freed row is reused first
    # rebind: the row keeps its state, only the name moves; whatever the new name held is released.
    assert t.rebind(6, 6) is None and t.rebind(77, 78) is None
    assert t.rebind(6, 9) == 3
    assert dict(t.row_of) == {9: 2} and sorted(t.free) == [1, 3]
    keys, vals = t.drain_outbox()
    assert dict(zip(keys.tolist(), vals.tolist())) == {5: 0, 9: 2, 6: 0}
    with pytest.raises(RuntimeError, match="outside the slot map"):
        t.rebind(9, 1000)
    assert t.release_all() == [2] and len(t) == 0 and sorted(t.free) == [1, 2, 3]


def test_tampering_is_detected():
    t = SlotTable(capacity=3, map_size=100)
    t.assign_many([1, 2])
    t.row_of[9] = t.row_of[1]  # a second slot naming the same row, behind the table's back
    with pytest.raises(RuntimeError, match="also mapped by a second slot"):
        t.assign_many([3])
    t = SlotTable(capacity=3, map_size=100)
    t.free.append(1)
    with pytest.raises(RuntimeError, match="free-list rows contain a duplicate"):
        t.assign_many([3])
    t = SlotTable(capacity=2, map_size=100)
    t.assign_many([1])
    t.slot_of[t.row_of[1]] = 4
    with pytest.raises(RuntimeError, match="owned by slot 4"):
        t.release(1)
    with pytest.raises(ValueError):
        SlotTable(capacity=0, map_size=4)


def make_layer(capacity=3, **kw):
    H, K, HV, V, W = 2, 32, 4, 32, 4
    D = 2 * H * K + HV * V
    return RecurrentGDN(capacity=capacity, conv_weight=torch.zeros(D, W, dtype=torch.bfloat16), conv_bias=None,
                        A_log=torch.zeros(HV), dt_bias=torch.zeros(HV), num_k_heads=H, head_k_dim=K,
                        num_v_heads=HV, head_v_dim=V, device="cpu", **kw)


def test_layer_mirrors_the_table_on_the_device_map(monkeypatch):
    monkeypatch.setenv("SKYRL_ISOEXEC_GDN_SLOT_MAP_SIZE", "64")
    layer = make_layer()
    assert layer.ssm_state.shape == (4, 4, 32, 32) and layer.ssm_state.dtype is torch.float32
    assert layer.conv_state.shape == (4, 2 * 2 * 32 + 4 * 32, 3) and layer.slot2row.numel() == 64
    rows = layer._assign_many([7, 9])
    assert rows == [3, 2] and layer.slot2row[7] == 3 and layer.slot2row[9] == 2
    assert layer.last_used.tolist() == [0, 0, 2, 1] and int(layer._clock) == 2
    # Padding ids outside the map are clamped into it; unknown ids read the null row.
    got = layer._rows(torch.tensor([7, 9, 8, -5, 1000]))
    assert got.tolist() == [3, 2, 0, 0, 0]
    assert layer._assign(11) == 1
    # Pool full: the next newcomer evicts the least recently used row (slot 7's row 3, tick 1).
    assert layer._assign(12) == 3
    assert layer.slot2row[7] == 0 and layer.slot2row[12] == 3 and not layer.table.holds(7)
    assert layer.release_slot(9) == 2 and layer.flush_slot_map() == 1 and layer.slot2row[9] == 0
    layer.rebind_slot(12, 13)
    assert flush_slot_maps([layer]) == 2 and layer.slot2row[13] == 3 and layer.slot2row[12] == 0
    assert layer.require_row(13) == 3
    layer.ssm_state.fill_(1.0)
    layer.conv_state.fill_(1.0)
    assert invalidate_all_states([layer]) == 2
    assert not layer.ssm_state.any() and not layer.conv_state.any() and not layer.slot2row.any()
    assert len(layer.table) == 0 and int(layer._clock) == 0


def test_continuation_mask(monkeypatch):
    layer = make_layer()
    layer._assign_many([4])
    monkeypatch.delenv("SKYRL_ISOEXEC_GDN_CHUNKED_PREFILL", raising=False)
    assert not chunked_prefill_enabled()
    assert layer._continuation_mask([4, 5], None) == [False, False]
    monkeypatch.setenv("SKYRL_ISOEXEC_GDN_CHUNKED_PREFILL", "1")
    assert layer._continuation_mask([4, 5], None) == [True, False]
    assert layer._continuation_mask([4, 5], [False, False]) == [False, False]  # a reissued slot id starts fresh
    assert layer._continuation_mask([4, 5], torch.tensor([True, False])) == [True, False]
    with pytest.raises(RuntimeError, match="prefix-cache hit"):
        layer._continuation_mask([4, 5], [True, True])


def test_native_state_is_validated():
    H, K, HV, V, W = 2, 32, 4, 32, 4
    D = 2 * H * K + HV * V
    kw = dict(capacity=2, conv_weight=torch.zeros(D, W, dtype=torch.bfloat16), conv_bias=None, A_log=torch.zeros(HV),
              dt_bias=torch.zeros(HV), num_k_heads=H, head_k_dim=K, num_v_heads=HV, head_v_dim=V, device="cpu")
    ssm = torch.zeros(8, HV, V, K)
    conv = torch.zeros(8, D, W - 1, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="BOTH"):
        RecurrentGDN(ssm_state=ssm, **kw)
    with pytest.raises(RuntimeError, match="not float32"):
        RecurrentGDN(ssm_state=ssm.bfloat16(), conv_state=conv, **kw)
    with pytest.raises(RuntimeError, match="orientation is wrong"):
        RecurrentGDN(ssm_state=ssm, conv_state=conv.transpose(1, 2).contiguous(), **kw)
    layer = RecurrentGDN(ssm_state=ssm, conv_state=conv, **kw)
    assert layer._rows(torch.tensor([3, 8, -1, 0])).tolist() == [3, 0, 0, 0]
    assert layer.release_slot(3) is None and layer.flush_slot_map() == 0 and layer.require_row(5) == 5
    with pytest.raises(ValueError, match="multiple of num_k_heads"):
        RecurrentGDN(**{**kw, "num_v_heads": 3})
