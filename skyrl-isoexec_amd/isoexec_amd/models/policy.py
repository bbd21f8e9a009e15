"""``ModelProfile`` -> ``{(op, site): Selection}``. Independent of any one model.

Reference: isoexec/models/policy.py:19-260. On this architecture every op has one implementation
that serves all of its sites (the kernels are row- and batch-invariant, so trainer and engine can
share them), which makes the composition symmetric: no entry needs an equivalence discharge.
An op the architecture does not run gets no key; absence means "no such site", never "default".
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Optional, Tuple

from ..core.contract_build import DEPLOYMENT, FUNCTION, ContractBuildError
from .profile import ATTN_NONE, ModelProfile

Key = Tuple[str, str]

TRAINER = ("trainer_fwd", "trainer_score")
ENGINE = ("engine_prefill", "engine_decode")
ALL_SITES = TRAINER + ENGINE

# The per-leaf block of the Kahan exp sum; must equal what the logprob kernel compiles with.
ROWINV_BLOCK = 4096

# Sentinel: an exception that deletes a derived key.
DROP = object()


@dataclass(frozen=True)
class Selection:
    """One resolved (op, site) choice. ``pinned_constants`` move bits and are hashed into the function
    half; ``neutrality_proof`` is mandatory for, and exclusive to, a DEPLOYMENT selection."""

    impl_id: str
    version: int = 1
    pinned_constants: Dict[str, object] = field(default_factory=dict)
    classification: str = FUNCTION
    neutrality_proof: Optional[str] = None

    def __post_init__(self) -> None:
        if self.classification not in (FUNCTION, DEPLOYMENT):
            raise ContractBuildError(
                f"unknown classification {self.classification!r}; must be one of ['{DEPLOYMENT}', '{FUNCTION}']"
            )
        if (self.classification == DEPLOYMENT) != bool(self.neutrality_proof):
            raise ContractBuildError(
                "a deployment selection requires a neutrality_proof and a function selection must not carry one"
            )


def entry(impl: str, version: int = 1, pinned: Optional[dict] = None, cls: str = FUNCTION, proof=None) -> Selection:
    """Spell one Selection; model files write their exceptions with it."""
    return Selection(impl, version, dict(pinned or {}), cls, proof)


def derive_selections(profile: ModelProfile) -> Dict[Key, Selection]:
    out: Dict[Key, Selection] = {}

    def put(op: str, sites, **kw) -> None:
        for site in sites:
            out[(op, site)] = entry(**kw)

    put("mm", ALL_SITES, impl="hip_mfma_batch_invariant")

    if profile.attention != ATTN_NONE:
        # One split is the contract: splitting the KV walk is what makes decode differ from prefill.
        put("attention.varlen", ALL_SITES, impl="hip_varlen_ns1", pinned={"num_splits": 1})
        put("rope.rope", ALL_SITES, impl="hip_rope")

    if not profile.zero_centered_norms:
        raise ContractBuildError(
            f"{profile.model!r}: only the zero-centred RMS norm has an implementation on this architecture"
        )
    put("norms.rms", ALL_SITES, impl="hip_fused")

    put(
        "logprobs.log_softmax",
        ALL_SITES,
        impl="hip_rowinv_leaftree",
        pinned={"leaves": profile.pik_leaves, "block": ROWINV_BLOCK, "accum": "kahan_fp32"},
    )
    # The trainer scores every position; only the engine slices to the sampled rows.
    put("logprobs.lm_head_slice", ENGINE, impl="sampled_rows")

    if profile.has_gdn:
        # The fused core absorbs gdn.l2norm and gdn.gating, so those get no entry of their own.
        put("gdn.core", ALL_SITES, impl="hip_fused_recurrent", pinned={"kernel": profile.gdn_kernel})
        put("gdn.conv", ALL_SITES, impl="hip_causal_conv")
        put("gdn.state", ENGINE, impl="hip_private_pool", pinned={"ssm_cache_dtype": profile.ssm_cache_dtype})
        put("norms.gated_out", ALL_SITES, impl="hip_fused")

    if profile.has_moe:
        r = profile.router
        if r.score_function != "softmax" or r.expert_bias:
            raise ContractBuildError(
                f"{profile.model!r}: router {r.score_function!r} (expert_bias={r.expert_bias}) has no "
                f"implementation on this architecture; only the bias-free softmax router does"
            )
        put("moe.router", ALL_SITES, impl="hip_fused_topk", pinned={"topk": r.topk, "experts": r.num_experts, "score": r.order})
        put("moe.dispatch", ALL_SITES, impl="hip_bitmask_index")
        put("moe.experts", ALL_SITES, impl="hip_grouped_mfma")
        put("moe.combine", ALL_SITES, impl="hip_fixed_order", pinned={"leaf_dtype": profile.moe_combine_dtype})

    if profile.tensor_parallel:
        raise ContractBuildError(
            f"{profile.model!r}: tensor_parallel=True needs the collectives family, which this single-device "
            f"composition does not register"
        )
    return out


def apply_exceptions(selections: Dict[Key, Selection], exceptions: Optional[dict]) -> Dict[Key, Selection]:
    """Overlay a model's exceptions. A key is ``(op, site)`` or ``(op, "*")``, a value a Selection or
    ``DROP``. An exception may only override or drop what the derivation produced."""
    if not exceptions:
        return selections
    out = dict(selections)
    for (op, site), value in exceptions.items():
        hits = [k for k in out if k[0] == op and site in ("*", k[1])]
        if not hits:
            raise ValueError(
                f"exception names ({op!r}, {site!r}) but the derivation produced no such key; if the model "
                f"needs a key policy does not derive, the profile is wrong, not the contract"
            )
        for k in hits:
            if value is DROP:
                del out[k]
            else:
                out[k] = value
    return out


def build_selections(profile: ModelProfile, exceptions: Optional[dict] = None) -> Dict[Key, Selection]:
    return apply_exceptions(derive_selections(profile), exceptions)


def policy_matches_registry_capabilities(profile: ModelProfile, registry) -> list:
    """Where the derived selections disagree with the registry: an unregistered op or impl, or an op
    whose trainer and engine impls differ without a claim that licenses the difference."""
    problems = []
    sel = derive_selections(profile)
    for op in sorted({op for op, _ in sel}):
        if not registry.has_op(op):
            problems.append(f"{op}: selected but not registered")
            continue
        spec = registry.get_op(op)
        trainer = {sel[(op, s)].impl_id for s in TRAINER if (op, s) in sel}
        engine = {sel[(op, s)].impl_id for s in ENGINE if (op, s) in sel}
        problems += [f"{op}: selects unregistered impl {i!r}" for i in sorted(trainer | engine) if i not in spec.impls]
        if not trainer or not engine or trainer == engine:
            continue
        engine_sel = [sel[(op, s)] for s in ENGINE if (op, s) in sel]
        if all(e.classification == DEPLOYMENT for e in engine_sel):
            continue
        caps = [spec.impls[i].capabilities for i in engine if i in spec.impls]
        if not any(c.get("bitwise_equal_to") in trainer or c.get("equivalence_proof") for c in caps):
            problems.append(
                f"{op}: sites resolve to different impls (trainer={sorted(trainer)} engine={sorted(engine)}) "
                f"with no bitwise_equal_to / equivalence_proof capability and no deployment classification"
            )
    return problems
