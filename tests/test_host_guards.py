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
