"""What a model declaration states: facts about an architecture, and no choice of implementation.

A fact that cannot be checked by looking at code -- how far a parallelism axis may vary, what invalidates a carried
state, how far two cases may differ -- comes with the reference that justifies it, and is refused when it is
malformed in a way that would make it vacuous. (Reference: isoexec/models/profile.py:16-215.)
"""

from __future__ import annotations

import dataclasses
import math
from dataclasses import dataclass, field

from ..contract import STATE_EVENTS

# attention families
ATTN_GQA = "gqa"
ATTN_NONE = "none"   # the declaration covers the path without attention only
_ATTENTIONS = frozenset((ATTN_GQA, ATTN_NONE))
# router score functions
SCORE_SOFTMAX = "softmax"
SCORE_SIGMOID = "sigmoid"
_SCORES = (SCORE_SOFTMAX, SCORE_SIGMOID, "sqrtsoftplus")


class ProfileError(ValueError):
    pass


def _refuse(subject: str, problem: str):
    raise ProfileError(f"{subject}: {problem}")


@dataclass(frozen=True)
class TopologyAxisFact:
    """A parallelism axis. Either ``pinned`` (a degree and the collective plan that goes with it) or ``invariant``
    (a domain of at least two degrees over which a named gate has shown the results do not move)."""

    axis: str
    kind: str
    degree: "int | None" = None
    collective_plan: "str | None" = None
    domain: tuple = ()
    proof: "str | None" = None

    def __post_init__(self) -> None:
        subject = f"topology axis {self.axis!r}"
        if self.proof is not None and self.proof.strip() == "":
            _refuse(subject, "empty proof ref names no gate")
        if self.kind == "pinned":
            if None in (self.degree, self.collective_plan):
                _refuse(subject, "pinned requires degree and collective_plan")
            if self.degree < 1:
                _refuse(subject, f"pinned degree {self.degree} is not a deployable degree (>= 1)")
        elif self.kind == "invariant":
            if not (self.domain and self.proof):
                _refuse(subject, "invariant requires a non-empty proven domain and a proof ref")
            distinct = sorted(set(self.domain))
            if len(distinct) < 2:
                _refuse(subject, f"invariance over the single degree {distinct} is a tautology; pin it")
        else:
            _refuse(subject, f"unknown kind {self.kind!r}")


@dataclass(frozen=True)
class StateFact:
    """A pool of state an engine carries: the lifecycle events that invalidate it, whether replaying a captured
    graph over it is safe, and the hook (``"path.py::symbol"``) that performs the invalidation."""

    state_id: str
    invalidated_by: tuple
    replay_safe: bool
    ref: str

    def __post_init__(self) -> None:
        subject = f"state fact {self.state_id!r}"
        if not (self.state_id and self.invalidated_by and self.ref):
            _refuse(subject, "requires a non-empty invalidated_by and a ref naming the hook")
        unknown = sorted(set(self.invalidated_by).difference(STATE_EVENTS))
        if unknown:
            _refuse(subject, f"unknown lifecycle event(s) {unknown}; the vocabulary is {sorted(STATE_EVENTS)}")


def _threshold_problem(text):
    """Why ``text`` cannot serve as a numeric threshold, or None. "nan" and "inf" do parse as numbers, and a
    comparison against them lets everything through."""
    try:
        number = float(text)
    except (TypeError, ValueError):
        return "is not a decimal string"
    return None if math.isfinite(number) else "is not a finite threshold"


@dataclass(frozen=True)
class ToleranceFact:
    """How far two cases may differ: named bounds, written as decimal strings and hashed exactly as written."""

    case_pair: tuple
    bounds: tuple
    attributed_to: tuple = ()

    def __post_init__(self) -> None:
        subject = f"tolerance fact {self.case_pair!r}"
        if len(self.case_pair) != 2 or len(self.bounds) == 0:
            _refuse(subject, "requires a 2-case pair and bounds")
        for name, text in self.bounds:
            problem = _threshold_problem(text)
            if problem:
                _refuse(subject, f"bound {name}={text!r} {problem}")


@dataclass(frozen=True)
class RouterProfile:
    """The router of a mixture-of-experts model. ``order``: "softmax_then_topk" scores every expert and keeps k,
    "topk_then_softmax" keeps k and normalises those."""

    score_function: str = SCORE_SOFTMAX
    expert_bias: bool = False
    topk: "int | None" = None
    num_experts: "int | None" = None
    scaling_factor: "float | None" = None
    group_topk: "int | None" = None
    eps: "float | None" = None
    order: str = "softmax_then_topk"

    def __post_init__(self) -> None:
        if self.score_function not in _SCORES:
            raise ProfileError(f"unknown router score_function {self.score_function!r}")


@dataclass(frozen=True)
class ModelProfile:
    """Structure first (these fields decide equality), then evidence (topology, states, tolerances: compared by
    nobody, carried into the contract's claims)."""

    model: str
    architectures: tuple = ()
    name_patterns: tuple = ()
    arch_discriminator: object = field(default=None, compare=False)
    attention: str = ATTN_GQA
    has_gdn: bool = False
    has_moe: bool = False
    zero_centered_norms: bool = True
    tensor_parallel: bool = False
    router: "RouterProfile | None" = None
    gdn_kernel: str = "recurrent"
    gdn_chunk_size: int = 64
    ssm_cache_dtype: str = "float32"
    pik_leaves: int = 8
    pik_leaf_dtype: str = "bf16"
    moe_combine_dtype: str = "fp32"   # what a token's k expert rows are summed in: "fp32" (one rounding) or "bf16" (one per add)
    topology: tuple = field(default=(), compare=False)
    states: tuple = field(default=(), compare=False)
    tolerances: tuple = field(default=(), compare=False)
    notes: str = ""
    source: str = "declared"

    def __post_init__(self) -> None:
        me = repr(self.model)
        if self.attention not in _ATTENTIONS:
            raise ProfileError(f"unknown attention family {self.attention!r}; expected one of {sorted(_ATTENTIONS)}")
        if self.moe_combine_dtype not in ("fp32", "bf16"):
            _refuse(me, f"unknown moe_combine_dtype {self.moe_combine_dtype!r}")
        if self.has_moe != (self.router is not None):
            _refuse(me, "has_moe=True requires a RouterProfile" if self.has_moe else "router declared but has_moe=False")
        declared_axes = [fact.axis for fact in self.topology]
        if len(declared_axes) > len(set(declared_axes)):
            _refuse(me, "duplicate topology axis declaration")

    def op_families(self) -> frozenset:
        """The op families a model of this shape needs implementations from."""
        optional = {
            "attention": self.attention != ATTN_NONE,
            "rope": self.attention != ATTN_NONE,
            "gdn": self.has_gdn,
            "moe": self.has_moe,
            "collectives": self.tensor_parallel,
        }
        return frozenset({"mm", "norms", "logprobs"} | {name for name, needed in optional.items() if needed})

    def with_overrides(self, **changes) -> "ModelProfile":
        return dataclasses.replace(self, **changes)
