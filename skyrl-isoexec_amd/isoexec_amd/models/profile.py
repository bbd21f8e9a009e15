"""``ModelProfile``: the structural facts of one architecture, with no implementation choice in it.

Reference: isoexec/models/profile.py:16-215. Facts that cannot be checked against code (a topology
envelope, a state's lifecycle, a tolerance) carry the reference that grounds them.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field, replace
from typing import Optional, Tuple

from ..contract import STATE_EVENTS

ATTN_GQA = "gqa"
ATTN_NONE = "none"  # the composition covers the non-attention path only
_ATTENTIONS = frozenset({ATTN_GQA, ATTN_NONE})

SCORE_SOFTMAX = "softmax"
SCORE_SIGMOID = "sigmoid"
_SCORES = (SCORE_SOFTMAX, SCORE_SIGMOID, "sqrtsoftplus")


class ProfileError(ValueError):
    pass


@dataclass(frozen=True)
class TopologyAxisFact:
    """One parallelism axis: ``pinned`` to a degree with its collective plan, or ``invariant`` over a
    proven domain of at least two degrees with the gate that proved it."""

    axis: str
    kind: str
    degree: Optional[int] = None
    collective_plan: Optional[str] = None
    domain: Tuple[int, ...] = ()
    proof: Optional[str] = None

    def __post_init__(self) -> None:
        who = f"topology axis {self.axis!r}"
        if self.kind not in ("pinned", "invariant"):
            raise ProfileError(f"{who}: unknown kind {self.kind!r}")
        if self.proof is not None and not self.proof.strip():
            raise ProfileError(f"{who}: empty proof ref names no gate")
        if self.kind == "pinned":
            if self.degree is None or self.collective_plan is None:
                raise ProfileError(f"{who}: pinned requires degree and collective_plan")
            if self.degree < 1:
                raise ProfileError(f"{who}: pinned degree {self.degree} is not a deployable degree (>= 1)")
        elif not self.domain or not self.proof:
            raise ProfileError(f"{who}: invariant requires a non-empty proven domain and a proof ref")
        elif len(set(self.domain)) < 2:
            raise ProfileError(f"{who}: invariance over the single degree {sorted(set(self.domain))} is a tautology; pin it")


@dataclass(frozen=True)
class StateFact:
    """An engine-side state pool: what invalidates it and the hook (``"path.py::symbol"``) that does."""

    state_id: str
    invalidated_by: Tuple[str, ...]
    replay_safe: bool
    ref: str

    def __post_init__(self) -> None:
        if not self.state_id or not self.invalidated_by or not self.ref:
            raise ProfileError(f"state fact {self.state_id!r}: requires a non-empty invalidated_by and a ref naming the hook")
        stray = sorted(set(self.invalidated_by) - STATE_EVENTS)
        if stray:
            raise ProfileError(
                f"state fact {self.state_id!r}: unknown lifecycle event(s) {stray}; the vocabulary is {sorted(STATE_EVENTS)}"
            )


@dataclass(frozen=True)
class ToleranceFact:
    """An accepted numeric envelope between two cases. Bounds are decimal strings, hashed as written."""

    case_pair: Tuple[str, str]
    bounds: Tuple[Tuple[str, str], ...]
    attributed_to: Tuple[str, ...] = ()

    def __post_init__(self) -> None:
        if len(self.case_pair) != 2 or not self.bounds:
            raise ProfileError(f"tolerance fact {self.case_pair!r}: requires a 2-case pair and bounds")
        for name, text in self.bounds:
            try:
                ok = math.isfinite(float(text))
            except (TypeError, ValueError):
                raise ProfileError(f"tolerance fact {self.case_pair!r}: bound {name}={text!r} is not a decimal string")
            if not ok:  # "nan" and "inf" parse, and a gate comparing against them admits everything
                raise ProfileError(f"tolerance fact {self.case_pair!r}: bound {name}={text!r} is not a finite threshold")


@dataclass(frozen=True)
class RouterProfile:
    score_function: str = SCORE_SOFTMAX
    expert_bias: bool = False
    topk: Optional[int] = None
    num_experts: Optional[int] = None
    scaling_factor: Optional[float] = None
    group_topk: Optional[int] = None
    eps: Optional[float] = None
    # "softmax_then_topk" scores all experts and keeps k; "topk_then_softmax" normalises the kept k.
    order: str = "softmax_then_topk"

    def __post_init__(self) -> None:
        if self.score_function not in _SCORES:
            raise ProfileError(f"unknown router score_function {self.score_function!r}")


@dataclass(frozen=True)
class ModelProfile:
    model: str
    architectures: Tuple[str, ...] = ()
    name_patterns: Tuple[str, ...] = ()
    arch_discriminator: Optional[object] = field(default=None, compare=False)
    attention: str = ATTN_GQA
    has_gdn: bool = False
    has_moe: bool = False
    zero_centered_norms: bool = True
    tensor_parallel: bool = False
    router: Optional[RouterProfile] = None
    gdn_kernel: str = "recurrent"
    gdn_chunk_size: int = 64
    ssm_cache_dtype: str = "float32"
    pik_leaves: int = 8
    pik_leaf_dtype: str = "bf16"
    # Evidence rather than structure, so excluded from equality.
    topology: Tuple[TopologyAxisFact, ...] = field(default=(), compare=False)
    states: Tuple[StateFact, ...] = field(default=(), compare=False)
    tolerances: Tuple[ToleranceFact, ...] = field(default=(), compare=False)
    notes: str = ""
    source: str = "declared"

    def __post_init__(self) -> None:
        if self.attention not in _ATTENTIONS:
            raise ProfileError(f"unknown attention family {self.attention!r}; expected one of {sorted(_ATTENTIONS)}")
        if self.has_moe and self.router is None:
            raise ProfileError(f"{self.model!r}: has_moe=True requires a RouterProfile")
        if not self.has_moe and self.router is not None:
            raise ProfileError(f"{self.model!r}: router declared but has_moe=False")
        axes = [t.axis for t in self.topology]
        if len(axes) != len(set(axes)):
            raise ProfileError(f"{self.model!r}: duplicate topology axis declaration")

    def op_families(self) -> frozenset:
        fams = {"mm", "norms", "logprobs"}
        if self.attention != ATTN_NONE:
            fams |= {"attention", "rope"}
        if self.has_gdn:
            fams.add("gdn")
        if self.has_moe:
            fams.add("moe")
        if self.tensor_parallel:
            fams.add("collectives")
        return frozenset(fams)

    def with_overrides(self, **kw) -> "ModelProfile":
        return replace(self, **kw)
