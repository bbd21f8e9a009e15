"""GPU: the composed model against the CPU oracle composition (oracle/hybrid.py), end to end.

Every op is compared with its oracle bit for bit elsewhere, and trainer == rollout is checked HIP against HIP; this
test catches what those cannot: a wiring mistake common to both runtimes (a wrong slice of a projection, a norm weight
from the wrong layer, a missing residual). The device's own top-k expert choices are handed to the oracle, so the
discrete decisions are like for like and only arithmetic differs: the oracle's matmuls accumulate in numpy's order, the
device's in the matrix instruction's, and each bf16 round of an activation may land one step apart.
Tolerance on a response token's logprob: 0.1 absolute, 0.03 on average (a wiring mistake moves logprobs by units)."""

import numpy as np
import pytest
import torch

from _util import DevicePrims, cpu_gen
from oracle import hybrid as o_hybrid

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("kernel", ["recurrent"])
def test_trainer_logprobs_match_the_oracle_composition(kernel):
    from isoexec_amd.runtimes.hybrid import HybridConfig, HybridWeights, TrainerModel

    cfg = HybridConfig(hidden=256, vocab=8192, layers=4, attention_every=2, gdn_k_heads=2, gdn_v_heads=4,
                       gdn_head_dim=64, q_heads=8, kv_heads=2, head_dim=128, max_positions=512, experts=8, topk=2,
                       expert_inter=64, gdn_kernel=kernel)
    w = HybridWeights.make(cfg, seed=5, device=DEV)
    lens, plens = [14, 9], [6, 2]
    tokens = torch.randint(0, cfg.vocab, (sum(lens),), generator=cpu_gen(6))
    trainer = TrainerModel(cfg, w)
    trainer.blocks.routing_log = []
    got = [t.cpu().numpy() for t in trainer.response_logprobs(tokens.to(DEV), lens, plens)]
    routing = [r.cpu().numpy() for r in trainer.blocks.routing_log]
    assert len(routing) == cfg.layers and routing[0].shape == (sum(lens), cfg.topk)

    oracle = o_hybrid.HybridOracle(cfg, o_hybrid.weights_from_torch(w), prims=DevicePrims(DEV), routing=routing)
    want = oracle.response_logprobs(tokens.numpy(), lens, plens)
    worst, total, count = 0.0, 0.0, 0
    for g, e in zip(got, want):
        assert g.shape == e.shape
        d = np.abs(g - e)
        worst, total, count = max(worst, float(d.max())), total + float(d.sum()), count + d.size
    assert worst < 0.1, worst
    assert total / count < 0.03, total / count
    assert float(np.std(np.concatenate(want))) > 0.2   # a model that discriminates: the comparison says something

    # the oracle with its OWN routing agrees with the device's choices almost everywhere (near-ties may flip)
    own = o_hybrid.HybridOracle(cfg, o_hybrid.weights_from_torch(w), prims=DevicePrims(DEV))
    own_lp = own.response_logprobs(tokens.numpy(), lens, plens)
    assert max(float(np.abs(a - b).max()) for a, b in zip(own_lp, want)) < 0.5
