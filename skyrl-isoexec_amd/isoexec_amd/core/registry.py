"""Ops, implementations and their rounding schedules: the table a model's selections resolve against.

Reference: isoexec/core/registry.py:14-247. An op's identity is its rounding schedule. Sites and
hazards come from closed vocabularies; there is no layer dimension (an op resolves identically at
every layer).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Sequence

# Execution sites. A site an op does not list does not exist for it; there is no default.
_BASE_SITES = frozenset({"trainer_fwd", "trainer_score", "engine_prefill", "engine_decode"})

# What a parity test may claim to exercise (and must then show it did).
HAZARDS = frozenset(
    {
        "null_lanes",        # padded / inert lanes under graph replay
        "t_zero",            # an empty sequence
        "non_contiguous",    # strided inputs
        "e_mismatch",        # expert count differs from the expected one
        "profiling_shapes",  # shapes the engine profiles at start-up
        "tie_boundaries",    # ties in top-k
        "subnormals",        # denormal inputs on flush-to-zero paths
        "signed_zero",       # +0.0 versus -0.0
    }
)

_ROUTES = frozenset({"reference_preserving", "composition_defining", "protected", "canonical"})


class RegistryError(ValueError):
    pass


class _PerModel:
    """Marks a schedule key whose value is a fact of the model, supplied by the pin itself."""

    __slots__ = ()

    def __repr__(self) -> str:
        return "PER_MODEL"


PER_MODEL = _PerModel()


def pin_values_equal(a, b) -> bool:
    """Equality between a declared schedule value and a pin: a list equals the same tuple (JSON turns
    one into the other), and a bool never equals an int."""
    if isinstance(a, bool) != isinstance(b, bool):
        return False
    seq = (list, tuple)
    if isinstance(a, seq) and isinstance(b, seq):
        return len(a) == len(b) and all(map(pin_values_equal, a, b))
    if isinstance(a, dict) and isinstance(b, dict):
        return a.keys() == b.keys() and all(pin_values_equal(a[k], b[k]) for k in a)
    return a == b


class OneOf:
    """A schedule value restricted to an enumerated set."""

    __slots__ = ("values",)

    def __init__(self, *values) -> None:
        self.values = tuple(values)

    def __contains__(self, candidate) -> bool:
        return any(pin_values_equal(v, candidate) for v in self.values)

    def __repr__(self) -> str:
        return f"OneOf{self.values!r}"


@dataclass(frozen=True)
class RoundingSchedule:
    """What an impl computes, as data. ``machine_assertable`` holds literals, ``PER_MODEL`` or
    ``OneOf``; its keys are exactly the pins the impl accepts. Changing either half is a new version."""

    machine_assertable: Dict[str, object] = field(default_factory=dict)
    documentary: str = ""

    def check_pin(self, key: str, value) -> Optional[str]:
        """None when the pin is consistent with the schedule, else the reason it is not. A key the
        schedule never declared refuses: such a pin would hash and match while constraining nothing."""
        if key not in self.machine_assertable:
            known = sorted(str(k) for k in self.machine_assertable)
            return (
                f"the impl's machine_assertable rounding schedule declares no such key (declared: {known}). "
                "A pin the impl never declared constrains nothing -- declare it (a literal, PER_MODEL, "
                "or OneOf(...)) or drop the pin."
            )
        declared = self.machine_assertable[key]
        if declared is PER_MODEL:
            return None
        fits = (value in declared) if isinstance(declared, OneOf) else pin_values_equal(declared, value)
        return None if fits else f"the impl declares {key}={declared!r}"


@dataclass(frozen=True)
class StateInvalidation:
    """When a stateful op's state must be rebound; ``hook(state, ctx) -> bool`` is the host-only
    check (True while the state is still valid)."""

    condition: str
    hook: Optional[Callable[..., bool]] = None


@dataclass(frozen=True)
class ImplSpec:
    """One implementation of an op at a pinned version. ``subsumes`` lists the ops it absorbs;
    ``hazards`` is the floor its parity tests exercise."""

    impl_id: str
    version: int
    supported_archs: frozenset
    rounding: RoundingSchedule = field(default_factory=RoundingSchedule)
    capabilities: Dict[str, object] = field(default_factory=dict)
    subsumes: Sequence[str] = ()
    state_invalidation: Optional[StateInvalidation] = None
    hazards: Sequence[str] = ()
    route: str = "protected"

    def __post_init__(self) -> None:
        if self.route not in _ROUTES:
            raise RegistryError(f"impl {self.impl_id!r} declares unknown route {self.route!r}")
        stray = set(self.hazards) - HAZARDS
        if stray:
            raise RegistryError(
                f"impl {self.impl_id!r} declares unknown hazard(s) {sorted(stray)}; the hazard "
                f"vocabulary is {sorted(HAZARDS)}"
            )
        if not self.supported_archs:
            raise RegistryError(f"impl {self.impl_id!r} must declare at least one supported arch")


@dataclass
class OpSpec:
    name: str
    sites: List[str]
    impls: Dict[str, ImplSpec] = field(default_factory=dict)
    per_layer_uniform: bool = True

    def add_impl(self, impl: ImplSpec) -> "OpSpec":
        if impl.impl_id in self.impls:
            raise RegistryError(f"op {self.name!r} already has impl {impl.impl_id!r}")
        self.impls[impl.impl_id] = impl
        return self


class Registry:
    def __init__(self) -> None:
        self._sites = set(_BASE_SITES)
        self._ops: Dict[str, OpSpec] = {}

    @property
    def sites(self) -> frozenset:
        return frozenset(self._sites)

    @property
    def ops(self) -> Dict[str, OpSpec]:
        return dict(self._ops)

    def register_site(self, name: str) -> None:
        if not name or not name.replace("_", "").isalnum():
            raise RegistryError(f"invalid site name {name!r}: must be a non-empty identifier")
        self._sites.add(name)

    def register_op(self, op: OpSpec) -> OpSpec:
        if op.name in self._ops:
            raise RegistryError(f"op {op.name!r} already registered")
        stray = set(op.sites) - self._sites
        if stray:
            raise RegistryError(
                f"op {op.name!r} declares unknown site(s) {sorted(stray)}; register them first via "
                f"register_site(). Known sites: {sorted(self._sites)}"
            )
        self._ops[op.name] = op
        return op

    def has_op(self, name: str) -> bool:
        return name in self._ops

    def get_op(self, name: str) -> OpSpec:
        try:
            return self._ops[name]
        except KeyError:
            raise RegistryError(f"unknown op {name!r}") from None

    def installed_keys(self) -> frozenset:
        return frozenset((op.name, site) for op in self._ops.values() for site in op.sites)

    def assert_subsumption_closed(self) -> None:
        for op in self._ops.values():
            for impl in op.impls.values():
                for absorbed in impl.subsumes:
                    if absorbed not in self._ops:
                        raise RegistryError(
                            f"impl {op.name}:{impl.impl_id} subsumes unregistered op {absorbed!r}; "
                            f"its passthrough cannot be derived"
                        )
