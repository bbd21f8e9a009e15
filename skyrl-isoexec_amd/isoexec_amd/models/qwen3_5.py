"""Qwen3.5-35B-A3B: the hybrid GatedDeltaNet + mixture-of-experts model the token-logprob path serves.

Reference: isoexec/models/qwen3_5.py:19-201. Widths are the checkpoint's; the composition is the
single-device one (no tensor parallelism, so no collective entries).
"""

from __future__ import annotations

from .policy import build_selections
from .profile import (
    ATTN_GQA,
    ATTN_NONE,
    SCORE_SOFTMAX,
    ModelProfile,
    RouterProfile,
    StateFact,
    ToleranceFact,
    TopologyAxisFact,
)

MODEL = "qwen3.5-35b-a3b"

# Widths of the checkpoint, before any sharding.
HIDDEN, VOCAB = 2048, 248320
LAYERS, GDN_LAYERS, ATTN_LAYERS = 40, 30, 10
GDN_HEADS_QK, GDN_HEADS_V, GDN_HEAD_DIM = 16, 32, 128
CONV_WIDTH = 4
NUM_EXPERTS, TOPK, MOE_FFN = 256, 8, 512

_ONE_DEVICE = tuple(TopologyAxisFact(axis=a, kind="pinned", degree=1, collective_plan="none") for a in ("TP", "PP", "CP"))

_GDN_STATE = StateFact(state_id="gdn_recurrent_state", invalidated_by=("weight_sync", "sleep_wake"), replay_safe=True,
                       ref="ops/gdn/gdn_recurrent_state.py::invalidate_all_states")

# Trainer scoring and engine decode run the same kernels, so the accepted difference between them is zero.
_SCORE_VS_DECODE = ToleranceFact(case_pair=("engine_decode", "trainer_score"),
                                 bounds=(("abs_diff_max_max", "0.0"), ("abs_diff_mean_max", "0.0")))

PROFILE = ModelProfile(
    model=MODEL,
    architectures=("Qwen3_5MoeForCausalLM", "Qwen3_5MoeForConditionalGeneration", "Qwen3NextForCausalLM"),
    name_patterns=("qwen3.5", "qwen3_5", "a3b", "qwen3-next"),
    attention=ATTN_GQA, has_gdn=True, has_moe=True, zero_centered_norms=True, tensor_parallel=False,
    router=RouterProfile(score_function=SCORE_SOFTMAX, expert_bias=False, topk=TOPK, num_experts=NUM_EXPERTS),
    gdn_kernel="recurrent", ssm_cache_dtype="float32",
    topology=_ONE_DEVICE, states=(_GDN_STATE,), tolerances=(_SCORE_VS_DECODE,),
    notes="hybrid GDN+MoE on one device; trainer and engine share every kernel",
)

# The same model with the attention layers left out of the composition: what the non-attention
# token-logprob path covers on its own.
PATH_PROFILE = PROFILE.with_overrides(model=MODEL + "/logprob-path", attention=ATTN_NONE, name_patterns=())

EXCEPTIONS: dict = {}


def build(registry, *, arch=None, profile=None):
    """The model's ExecutionContract against ``registry``; ``profile`` selects a variant explicitly."""
    from ..core.arch import ARCH
    from ..core.contract_build import build_execution_contract

    chosen = PROFILE if profile is None else profile
    evidence = dict(topology=chosen.topology, states=chosen.states, tolerances=chosen.tolerances)
    return build_execution_contract(registry, build_selections(chosen, EXCEPTIONS), arch=arch or ARCH,
                                    model=chosen.model, profile=chosen, **evidence)
