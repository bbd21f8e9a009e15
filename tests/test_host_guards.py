"""Host-side refusals that protect the kernels' addressing (no GPU: every case raises before anything is launched).

The rotary tables hold ``max_positions`` rows and the kernel indexes them by position; the packed attention form
addresses keys from the queries' offsets. Lengths that would leave those ranges are refused on the host."""

import pytest
import torch

from isoexec_amd.ops.attention.varlen_attn import varlen_attention
from isoexec_amd.ops.rope.rope_hip import apply_rope_
from isoexec_amd.runtimes import hybrid


def test_sequences_longer_than_the_rotary_tables_are_refused():
    cfg = hybrid.HybridConfig(max_positions=64)
    hybrid.check_lengths(cfg, [64, 3], "x")
    with pytest.raises(ValueError, match="max_positions"):
        hybrid.check_lengths(cfg, [65], "x")
    with pytest.raises(ValueError, match="max_positions"):
        hybrid.RolloutEngine(cfg, None, max_num_seqs=1, max_len=65)       # refused before any weight is touched
    trainer = hybrid.TrainerModel.__new__(hybrid.TrainerModel)
    trainer.cfg, trainer.blocks = cfg, None
    with pytest.raises(ValueError, match="trainer pass"):
        trainer.hidden_states(torch.zeros(70, dtype=torch.int64), [70])
    engine = hybrid.RolloutEngine.__new__(hybrid.RolloutEngine)
    engine.cfg, engine.blocks, engine.max_len = cfg, None, 32
    with pytest.raises(ValueError, match="prefill"):
        engine.prefill([0], torch.zeros(70, dtype=torch.int64), [70])
    with pytest.raises(ValueError, match="cache length"):
        engine.prefill([0], torch.zeros(40, dtype=torch.int64), [40])


def test_packed_attention_needs_a_key_for_every_query():
    q = torch.zeros(10, 8, 128, dtype=torch.bfloat16)
    k = torch.zeros(6, 2, 128, dtype=torch.bfloat16)
    cu = torch.tensor([0, 10], dtype=torch.int32)
    with pytest.raises(RuntimeError, match="packed keys hold 6 tokens for 10 queries"):
        varlen_attention(q, k, k, cu, 10)
    with pytest.raises(RuntimeError, match="needs kv_start"):
        varlen_attention(q, q[:, :2], q[:, :2], cu, 10, q_pos0=torch.zeros(1, dtype=torch.int32))


def test_rope_table_shape_is_checked_before_the_device():
    x = torch.zeros(4, 2, 128, dtype=torch.bfloat16)
    pos = torch.zeros(4, dtype=torch.int32)
    bad = torch.zeros(16, 130, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="even R <= D"):
        apply_rope_(x, bad, bad, pos)


def test_a_declined_logprob_kernel_is_not_ignored(monkeypatch):
    blocks = hybrid._Blocks.__new__(hybrid._Blocks)
    monkeypatch.setattr(hybrid._Blocks, "logits", lambda self, x, want_row_max=False: (torch.zeros(2, 10), torch.zeros(2)))
    monkeypatch.setattr(hybrid, "sampled_forward", lambda *a, **k: None)
    with pytest.raises(RuntimeError, match="declined"):
        blocks.sampled_logprobs(torch.zeros(2, 4), torch.zeros(2, dtype=torch.int64))


def test_failed_selfcheck_switches_the_library_off_and_is_a_ledger_violation(monkeypatch):
    """The failure path of ``arch_selfcheck`` on a stand-in library (no device needed): the verdict is a violation at the
    install phase, and every later ``lib()`` of the process raises."""
    import ctypes
    import sys
    import types

    import pytest

    from isoexec_amd import _lib
    from isoexec_amd.core import arch, enforce

    class FakeLib:
        def ix_arch_selfcheck_workspace_bytes(self):
            return 1024

        def ix_arch_selfcheck(self, ws, nbytes, mask, stream):
            ctypes.cast(mask, ctypes.POINTER(ctypes.c_uint))[0] = 0b0101
            return _lib.IX_DECLINED

    class FakeTensor:
        def data_ptr(self):
            return 4096

    class FakeCtx:
        def __enter__(self):
            return self

        def __exit__(self, *a):
            return False

    fake_torch = types.SimpleNamespace(
        device=lambda *a: "cuda:0", uint8="u8", empty=lambda *a, **k: FakeTensor(),
        cuda=types.SimpleNamespace(current_device=lambda: 0, device=lambda d: FakeCtx()))
    enforce._reset_for_tests()
    monkeypatch.setattr(arch, "_SELFCHECK", None)
    monkeypatch.setattr(_lib, "_DISABLED", None)
    monkeypatch.setattr(_lib, "lib", lambda: FakeLib())
    monkeypatch.setattr(_lib, "current_stream", lambda dev=None: 0)
    monkeypatch.setitem(sys.modules, "torch", fake_torch)
    assert arch.arch_selfcheck(verbose=False) is False
    record, = enforce.ledger().by_id(arch.SELFCHECK_OBLIGATION)
    assert (record.phase, record.result) == (enforce.INSTALL, enforce.VIOLATION)
    assert "seeded product differs" in record.evidence and "log-softmax launch shapes differ" in record.evidence
    assert "integer product" not in record.evidence
    assert _lib.disabled_reason().startswith("arch self-check failed")
    monkeypatch.undo()
    # the real loader now refuses, until the process-wide latch is cleared again (here: by hand, for the other tests)
    monkeypatch.setattr(_lib, "_DISABLED", "arch self-check failed: test")
    with pytest.raises(_lib.IsoExecLibraryError, match="switched off"):
        _lib.lib()
    monkeypatch.undo()
    assert _lib.disabled_reason() is None
    enforce._reset_for_tests()
