"""Host-side tests of the slot -> row resolution seam (``gdn_cpr_rows`` + ``RecurrentGDN._rows_pair``), after the
reference's ops/gdn/tests/test_cpr_rows_cpu.py: without a device the fused launch is never attempted and the
answer is the eager index chain; the kill switch, the engine-block form and the decline predicates are host logic."""

import pytest
import torch

from isoexec_amd.ops.gdn import gdn_cpr_rows
from isoexec_amd.ops.gdn.gdn_recurrent_state import RecurrentGDN


def rows_eager(slot2row, slots):
    """The index chain the fused launch replaces (gdn_recurrent_state.py:283-284 of the reference)."""
    return slot2row[slots.long().clamp_(0, slot2row.numel() - 1)]


def make_pool(map_size=4096, rows=64):
    rg = RecurrentGDN.__new__(RecurrentGDN)  # only the fields _rows_pair touches
    rg._native = False
    g = torch.Generator().manual_seed(1234)
    rg.slot2row = torch.randint(0, rows, (map_size,), dtype=torch.int64, generator=g)
    return rg


def slot_vectors(map_size):
    """Every slot vector a replayed decode step can present (test_cpr_rows_cpu.py:37-48)."""
    return [
        torch.tensor([0, 1, 2, 3], dtype=torch.int32),
        torch.tensor([-1, -1, -1, -1], dtype=torch.int32),  # null-block padding
        torch.tensor([map_size - 1, map_size, map_size + 7, 1 << 20], dtype=torch.int32),
        torch.tensor([5, 5, 5, 5], dtype=torch.int32),  # duplicates -> one row
        torch.tensor([-3, 0, map_size, 17, -1, 9], dtype=torch.int32),
        torch.arange(512, dtype=torch.int32),  # production decode width
        torch.tensor([], dtype=torch.int32),
        torch.tensor([0, 1], dtype=torch.int64),
    ]


def test_rows_pair_is_the_eager_chain_without_a_device():
    rg = make_pool()
    for slots in slot_vectors(rg.slot2row.numel()):
        rows, rows32 = rg._rows_pair(slots)
        want = rows_eager(rg.slot2row, slots)
        assert rows.dtype is torch.int64 and rows32.dtype is torch.int32
        assert torch.equal(rows, want) and torch.equal(rows32, want.to(torch.int32))


def test_kill_switch_takes_the_eager_chain(monkeypatch):
    monkeypatch.setenv("SKYRL_ISOEXEC_GDN_CPR_FUSED_ROWS", "0")
    assert not gdn_cpr_rows.fused_rows_enabled()
    served = gdn_cpr_rows._served
    rg = make_pool()
    slots = torch.arange(64, dtype=torch.int32)
    rows, _ = rg._rows_pair(slots)
    assert torch.equal(rows, rows_eager(rg.slot2row, slots))
    assert gdn_cpr_rows._served == served
    monkeypatch.setenv("SKYRL_ISOEXEC_GDN_CPR_FUSED_ROWS", "1")
    assert gdn_cpr_rows.fused_rows_enabled()


def test_engine_block_ids_keep_their_own_clamp():
    """With the engine's own state tensors a slot id IS the row; ids past the tensor and negative ids read row 0."""
    rg = make_pool()
    rg._native = True
    rg.ssm_state = torch.zeros(16, 1)
    slots = torch.tensor([-1, 0, 15, 16, 999], dtype=torch.int32)
    rows, rows32 = rg._rows_pair(slots)
    s = slots.long()
    want = torch.where(s < 16, s, torch.zeros_like(s)).clamp_(min=0)
    assert torch.equal(rows, want) and torch.equal(rows32, want.to(torch.int32))


@pytest.mark.parametrize("slots, smap, why", [
    (torch.zeros(4, 2, dtype=torch.int32), torch.zeros(8, dtype=torch.int64), "2-D slots"),
    (torch.zeros(4, dtype=torch.int32), torch.zeros(8, 2, dtype=torch.int64), "2-D map"),
    (torch.zeros(4, dtype=torch.int32), torch.zeros(8, dtype=torch.int32), "int32 map"),
    (torch.zeros(4, dtype=torch.float32), torch.zeros(8, dtype=torch.int64), "float slots"),
])
def test_declines_rather_than_guesses(slots, smap, why):
    before = gdn_cpr_rows._declined
    assert gdn_cpr_rows.cpr_resolve_rows(slots, smap) is None, why
    assert gdn_cpr_rows._declined == before + 1
    assert "expected 1-D slots" in gdn_cpr_rows._decline_reason


def test_kernel_arithmetic_equals_the_eager_chain():
    """min(max(s, 0), n - 1) (the kernel's form) equals clamp_(0, n - 1) on every slot vector."""
    smap = torch.arange(97, dtype=torch.int64) * 3
    for slots in slot_vectors(smap.numel()):
        s = slots.long()
        kernel_form = smap[torch.minimum(torch.maximum(s, torch.zeros_like(s)), torch.full_like(s, smap.numel() - 1))]
        assert torch.equal(kernel_form, rows_eager(smap, slots))
