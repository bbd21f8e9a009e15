"""GPU: the device self-check (``ix_arch_selfcheck``; reference ops/collectives/pik_bootstrap.py:82-93) passes on this
device, each of its comparisons sees a single flipped bit, and the host side files the verdict and switches the library
off on a failure."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _run(inject):
    from isoexec_amd import _lib

    L = _lib.lib()
    need = int(L.ix_arch_selfcheck_workspace_bytes())
    assert 4 << 20 <= need <= 16 << 20
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    mask = ctypes.c_uint(0xFFFF)
    stream = torch.cuda.current_stream().cuda_stream
    if inject is None:
        rc = L.ix_arch_selfcheck(ws.data_ptr(), need, ctypes.byref(mask), stream)
    else:
        rc = L.ix_arch_selfcheck_probe(ws.data_ptr(), need, inject, ctypes.byref(mask), stream)
    return rc, mask.value


def test_selfcheck_passes_and_every_comparison_has_teeth():
    assert _run(None) == (0, 0)
    assert _run(0) == (0, 0)
    for inject in (1, 2, 4, 5, 7):
        assert _run(inject) == (1, inject), inject      # IX_DECLINED, exactly the checks whose reference was touched
    assert _run(None) == (0, 0)                          # nothing is left behind in the library


def test_selfcheck_refuses_bad_scratch_without_launching():
    from isoexec_amd import _lib

    L = _lib.lib()
    need = int(L.ix_arch_selfcheck_workspace_bytes())
    ws = torch.empty(need + 256, dtype=torch.uint8, device=DEV)
    assert L.ix_arch_selfcheck(None, need, None, None) == -1
    assert L.ix_arch_selfcheck(ws.data_ptr(), need - 1, None, None) == -3
    assert L.ix_arch_selfcheck(ws.data_ptr() + 8, need, None, None) == -1     # not 256-byte aligned


def test_host_side_files_the_verdict(monkeypatch):
    from isoexec_amd.core import arch, enforce

    enforce._reset_for_tests()
    monkeypatch.setattr(arch, "_SELFCHECK", None)
    assert arch.arch_selfcheck(verbose=False) is True
    records = enforce.ledger().by_id(arch.SELFCHECK_OBLIGATION)
    assert [(r.phase, r.result) for r in records] == [(enforce.INSTALL, enforce.OK)] and "gfx950" in records[0].evidence
    assert arch.arch_selfcheck(verbose=False) is True and len(enforce.ledger().by_id(arch.SELFCHECK_OBLIGATION)) == 1
    enforce._reset_for_tests()
