"""Host-side behaviour of the slot -> pool-row seam (``gdn_cpr_rows`` and ``RecurrentGDN._rows_pair``).

What the reference pins in ops/gdn/tests/test_cpr_rows_cpu.py, restated for this package: without a device the
one-launch resolver is never tried and the answer is the eager index chain; an environment switch turns the
resolver off; engine-owned block ids keep their own range rule; unusual shapes and dtypes are declined (and
counted) instead of guessed at; and the clamp the kernel writes as min(max(.)) is the chain's clamp."""

import pytest
import torch

from isoexec_amd.ops.gdn import gdn_cpr_rows
from isoexec_amd.ops.gdn.gdn_recurrent_state import RecurrentGDN

MAP = 4096


def rows_eager(slot2row, slots):
    return slot2row[slots.long().clamp_(0, slot2row.numel() - 1)]


def make_pool(map_size=MAP, rows=64):
    """A layer object carrying only what the seam reads: the slot map and the ownership flag."""
    layer = object.__new__(RecurrentGDN)
    layer._native = False
    layer.slot2row = torch.randint(0, rows, (map_size,), dtype=torch.int64, generator=torch.Generator().manual_seed(1234))
    return layer


def slot_vectors(map_size):
    """Slot vectors a replayed decode step can present: plain, null-block padding, ids past the map, duplicates,
    a mixture, the widest production batch, an empty half, and ids that are already 64-bit."""
    i32 = lambda v: torch.tensor(v, dtype=torch.int32)
    return [i32([0, 1, 2, 3]), i32([-1] * 4), i32([map_size - 1, map_size, map_size + 7, 1 << 20]), i32([5] * 4),
            i32([-3, 0, map_size, 17, -1, 9]), torch.arange(512, dtype=torch.int32), i32([]),
            torch.tensor([0, 1], dtype=torch.int64)]


@pytest.mark.parametrize("case", range(8))
def test_rows_pair_is_the_eager_chain_without_a_device(case):
    layer = make_pool()
    slots = slot_vectors(MAP)[case]
    wide, narrow = layer._rows_pair(slots)
    want = rows_eager(layer.slot2row, slots)
    assert (wide.dtype, narrow.dtype) == (torch.int64, torch.int32)
    assert torch.equal(wide, want) and torch.equal(narrow.long(), want)


@pytest.mark.parametrize("case", range(8))
def test_kernel_clamp_is_the_chains_clamp(case):
    table = torch.arange(97, dtype=torch.int64) * 3
    s = slot_vectors(97)[case].long()
    as_kernel = table[torch.minimum(torch.maximum(s, torch.zeros_like(s)), torch.full_like(s, 96))]
    assert torch.equal(as_kernel, rows_eager(table, s))


def test_switch_turns_the_resolver_off(monkeypatch):
    layer = make_pool()
    slots = torch.arange(64, dtype=torch.int32)
    for value, enabled in (("0", False), ("false", False), ("", False), ("1", True)):
        monkeypatch.setenv("SKYRL_ISOEXEC_GDN_CPR_FUSED_ROWS", value)
        assert gdn_cpr_rows.fused_rows_enabled() is enabled
        served = gdn_cpr_rows._served
        assert torch.equal(layer._rows_pair(slots)[0], rows_eager(layer.slot2row, slots))
        assert gdn_cpr_rows._served == served  # host tensors never reach the launch either way
    monkeypatch.delenv("SKYRL_ISOEXEC_GDN_CPR_FUSED_ROWS")
    assert gdn_cpr_rows.fused_rows_enabled()


def test_engine_block_ids_keep_their_own_range_rule():
    layer = make_pool()
    layer._native, layer.ssm_state = True, torch.zeros(16, 1)
    slots = torch.tensor([-1, 0, 15, 16, 999], dtype=torch.int32)
    wide, narrow = layer._rows_pair(slots)
    assert wide.tolist() == [0, 0, 15, 0, 0] and narrow.tolist() == [0, 0, 15, 0, 0]


@pytest.mark.parametrize("slots, table", [
    (torch.zeros(4, 2, dtype=torch.int32), torch.zeros(8, dtype=torch.int64)),     # slots not a vector
    (torch.zeros(4, dtype=torch.int32), torch.zeros(8, 2, dtype=torch.int64)),     # map not a vector
    (torch.zeros(4, dtype=torch.int32), torch.zeros(8, dtype=torch.int32)),        # map not 64-bit
    (torch.zeros(4, dtype=torch.float32), torch.zeros(8, dtype=torch.int64)),      # slots not integers
])
def test_unusual_arguments_are_declined_and_counted(slots, table):
    before = gdn_cpr_rows._declined
    assert gdn_cpr_rows.cpr_resolve_rows(slots, table) is None
    assert gdn_cpr_rows._declined == before + 1 and "expected 1-D slots" in gdn_cpr_rows._decline_reason
