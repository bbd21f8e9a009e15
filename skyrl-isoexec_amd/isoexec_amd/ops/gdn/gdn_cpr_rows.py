"""One-launch slot -> row resolution for the decode step (reference: ops/gdn/gdn_cpr_rows.py:1-80).

Host-free and shape-static, so it records into a HIP graph. ``SKYRL_ISOEXEC_GDN_CPR_FUSED_ROWS=0`` (or an
unexpected shape/dtype) hands the caller back to the eager chain ``slot2row[slots.long().clamp(0, n - 1)]``.
"""
from __future__ import annotations

import os

import torch

from ... import _lib

_ENV = "SKYRL_ISOEXEC_GDN_CPR_FUSED_ROWS"

# served / declined call counts and the last decline's reason (gdn_cpr_rows.py:18-21)
_served = 0
_declined = 0
_decline_reason = ""


def fused_rows_enabled() -> bool:
    """Default on; the environment variable is a kill switch (gdn_cpr_rows.py:24-26)."""
    return os.environ.get(_ENV, "1").lower() not in ("", "0", "false", "no")


def _resolve(slots, slot2row, blocks, last_used, clock, want64):
    n = slots.numel()
    dev = slots.device
    rows64 = torch.empty(n, dtype=torch.int64, device=dev) if want64 else None
    rows32 = torch.empty(n, dtype=torch.int32, device=dev)
    global _served
    _served += 1
    _lib.check(
        _lib.lib().ix_gdn_resolve_rows(slots.data_ptr(), int(slots.dtype is torch.int64), n, _lib.ptr(slot2row),
                                       0 if slot2row is None else slot2row.numel(), int(blocks),
                                       _lib.ptr(rows64), rows32.data_ptr(), _lib.ptr(last_used), _lib.ptr(clock),
                                       _lib.current_stream(dev)), "ix_gdn_resolve_rows")
    return rows64, rows32


def _servable(slots, slot2row) -> bool:
    global _declined, _decline_reason
    ok = slots.dim() == 1 and slots.dtype in (torch.int32, torch.int64) and slots.is_contiguous()
    if ok and slot2row is not None:
        ok = slot2row.dim() == 1 and slot2row.dtype is torch.int64 and slot2row.is_contiguous()
    if not ok:
        _declined += 1
        _decline_reason = (
            f"slots.dim={slots.dim()} slots.dtype={slots.dtype} "
            + ("" if slot2row is None else f"map.dim={slot2row.dim()} map.dtype={slot2row.dtype} ")
            + "(expected 1-D slots, 1-D int64 map)")
    return ok


def cpr_resolve_rows(slots: torch.Tensor, slot2row: torch.Tensor):
    """``(rows_int64, rows_int32)`` for a decode batch's engine slot ids; ``None`` to request the eager chain
    (gdn_cpr_rows.py:49-80)."""
    if slot2row is None or not _servable(slots, slot2row):
        return None
    _lib.require_device(slots, slot2row)
    return _resolve(slots, slot2row, 0, None, None, True)


def resolve_and_stamp(slots: torch.Tensor, *, slot2row=None, blocks: int = 0, last_used=None, clock=None):
    """The decode step's form: int32 rows, and when ``last_used``/``clock`` are given the same launch advances the
    clock and stamps the rows (``clock += 1; last_used[rows] = clock``). ``slot2row=None`` maps engine block ids
    onto themselves, ids outside ``[0, blocks)`` onto row 0 (gdn_recurrent_state.py:277-282). ``None`` when the
    arguments are not servable."""
    if not _servable(slots, slot2row):
        return None
    if (last_used is None) != (clock is None):
        raise ValueError("last_used and clock go together")
    if last_used is not None and (last_used.dtype is not torch.int64 or clock.dtype is not torch.int64):
        return None
    _lib.require_device(slots, slot2row, last_used, clock)
    return _resolve(slots, slot2row, blocks, last_used, clock, False)[1]
