"""GPU parity of the caller protocol: the trainer's chunk walk, the engine's hooks, and that the two
runtimes produce the same bits for the same row."""

import numpy as np
import pytest
import torch

from _util import DevicePrims, bf16_to_np, cpu_gen, np_bits, same_bits
from oracle import logprobs as o_lp

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
B, S, V = 2, 37, 8192 + 4096  # three blocks per row, ragged against the chunk sizes below


@pytest.fixture()
def callers(monkeypatch):
    from isoexec_amd.ops.logprobs import rowinv
    from isoexec_amd.runtimes import logprob_callers

    monkeypatch.setenv("SKYRL_ISOEXEC", "1")
    monkeypatch.setenv("SKYRL_ISOEXEC_PIK_LEAVES", "4")
    rowinv._reset_for_test()
    yield logprob_callers
    rowinv._reset_for_test()


def make(seed=0):
    g = cpu_gen(seed)
    logits = (torch.randn(B, S, V, generator=g) * 3).to(torch.bfloat16)
    target = torch.randint(0, V, (B, S), generator=g)
    return logits, target


def test_trainer_walk_is_bit_exact_chunk_invariant_and_differentiable(callers):
    from isoexec_amd.ops.logprobs import rowinv

    logits, target = make()
    want, _ = o_lp.rowinv_sampled(bf16_to_np(logits).reshape(B * S, V), target.numpy().reshape(-1), 4, prims=DevicePrims(DEV))
    xd, td = logits.to(DEV), target.to(DEV)
    whole = callers._ix_logprobs_apply(xd, td, 0, V, None, True, None)
    assert np.array_equal(np_bits(whole.cpu().numpy().reshape(-1)), np_bits(want))
    for chunk in (1, 5, 16, 36, 37, 100):
        walked = callers._ix_logprobs_apply(xd, td, 0, V, None, True, chunk)
        assert same_bits(walked, whole), chunk
    st = rowinv.stats()
    assert st["served"] > 0 and st["agreed"] is True and st["declined"] == 0
    # The first call probed against the incumbent; the two are different functions that agree closely.
    inc = callers.incumbent_logprobs(xd, td, 0, V)
    assert float((inc - whole).abs().max()) < 1e-4
    # Training: gradient of sum(logprob) is onehot - softmax, through the chunk walk.
    xg = xd.clone().requires_grad_(True)
    out = callers._ix_logprobs_apply(xg, td, 0, V, None, False, 8)
    assert out.requires_grad and same_bits(out.detach(), whole)
    out.sum().backward()
    ref = -torch.softmax(xd.float(), -1)
    ref.scatter_add_(-1, td.unsqueeze(-1), torch.ones(B, S, 1, device=DEV))
    assert float((xg.grad.float() - ref).abs().max()) <= 2 ** -8  # the gradient is rounded to bf16
    # A shape the kernel does not serve hands the whole call to the incumbent.
    odd = xd[..., : V - 2].contiguous()
    t_odd = td.clamp(max=V - 3)
    got = callers._ix_logprobs_apply(odd, t_odd, 0, V - 2, None, True, 8)
    # The incumbent's own bits move with the chunking (its reduction order follows the shape), so the
    # comparison is against the incumbent walked the same way.
    kept = same_bits(got, callers._incumbent_apply(odd, t_odd, 0, V - 2, True, 8))
    assert kept
    assert rowinv.stats()["declined"] > 0


def test_engine_rows_equal_trainer_rows_bitwise(callers):
    """The trainer scores [B, S, V] in chunks; the engine sees a few sampled rows in another order
    and asks for the full row. The sampled entries must be the same bits."""
    logits, target = make(seed=4)
    xd, td = logits.to(DEV), target.to(DEV)
    trainer = callers._ix_logprobs_apply(xd, td, 0, V, None, True, 16).reshape(-1)
    hook = callers.make_engine_compute_logprobs()
    pick = torch.tensor([70, 3, 36, 37, 0, 11], device=DEV)
    rows = xd.reshape(B * S, V).index_select(0, pick)
    full = hook(rows)
    assert full.shape == (6, V) and full.dtype is torch.float32
    want_full = o_lp.rowinv_full(bf16_to_np(rows), 4, prims=DevicePrims(DEV))
    assert np.array_equal(np_bits(full.cpu().numpy()), np_bits(want_full))
    sampled = full.gather(1, td.reshape(-1)[pick].unsqueeze(1)).squeeze(1)
    assert same_bits(sampled, trainer[pick])
    one = hook(rows[2:3])
    assert same_bits(one[0], full[2])
    census = callers.engine_logprob_census()
    assert census["rowinv_owned"] >= 2 and census["incumbent"] == 0


def test_sampled_rows_head_equals_slicing_the_full_logits(callers):
    from isoexec_amd.ops.mm.mm_hip import linear_nt

    g = cpu_gen(9)
    hidden = (torch.randn(300, 1024, generator=g)).to(torch.bfloat16).to(DEV)
    weight = (torch.randn(4096, 1024, generator=g) * 0.05).to(torch.bfloat16).to(DEV)
    head = callers.SampledRowsHead(weight)
    everything = linear_nt(hidden, weight)
    pick = torch.tensor([299, 0, 128, 129, 7], device=DEV)
    assert same_bits(head.compute_logits(hidden, pick), everything.index_select(0, pick))
    assert same_bits(head.compute_logits(hidden[5:6]), everything[5:6])
    assert same_bits(head.compute_logits(hidden.float(), pick), everything.index_select(0, pick))
    scaled = callers.SampledRowsHead(weight, logit_scale=0.5).compute_logits(hidden, pick)
    assert same_bits(scaled, everything.index_select(0, pick) * 0.5)
