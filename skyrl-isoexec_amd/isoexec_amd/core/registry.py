"""The table of ops and their implementations that a model's selections are resolved against.

An implementation is identified by WHAT IT COMPUTES, written down as a rounding schedule; an op lists the execution
sites it exists at (a site it does not list does not exist for it -- nothing is defaulted); hazards are the
situations an implementation's parity tests promise to exercise. Sites, hazards and routes are closed vocabularies.
There is no per-layer dimension: an op resolves the same way at every layer.
(Reference: isoexec/core/registry.py:14-247.)
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Sequence


class RegistryError(ValueError):
    pass


# ---- vocabularies --------------------------------------------------------------------------------------------
_BASE_SITES = frozenset(("trainer_fwd", "trainer_score", "engine_prefill", "engine_decode"))
_ROUTES = frozenset(("reference_preserving", "composition_defining", "protected", "canonical"))
_HAZARD_NOTES = {
    "null_lanes": "padded lanes that must stay inert when a graph is replayed",
    "t_zero": "a sequence with no tokens",
    "non_contiguous": "inputs that are strided views",
    "e_mismatch": "an expert count other than the expected one",
    "profiling_shapes": "the shapes an engine probes at start-up",
    "tie_boundaries": "equal scores in a top-k",
    "subnormals": "denormal inputs where a path flushes to zero",
    "signed_zero": "the sign of a zero",
}
HAZARDS = frozenset(_HAZARD_NOTES)


# ---- values a schedule may hold ------------------------------------------------------------------------------
class _PerModel:
    """Placeholder for a schedule value that is a fact of the model: the pin supplies it."""

    __slots__ = ()

    def __repr__(self) -> str:
        return "PER_MODEL"


PER_MODEL = _PerModel()


def pin_values_equal(a, b) -> bool:
    """Do a declared value and a pinned value agree? Lists and tuples compare by content (a round trip through
    JSON turns one into the other), mappings key by key, and True is not 1."""
    if isinstance(a, bool) or isinstance(b, bool):
        return isinstance(a, bool) and isinstance(b, bool) and a == b
    if isinstance(a, (list, tuple)) and isinstance(b, (list, tuple)):
        return len(a) == len(b) and all(pin_values_equal(x, y) for x, y in zip(a, b))
    if isinstance(a, dict) and isinstance(b, dict):
        return set(a) == set(b) and all(pin_values_equal(a[k], b[k]) for k in a)
    return a == b


class OneOf:
    """A schedule value that may be any one of the listed alternatives."""

    __slots__ = ("values",)

    def __init__(self, *values) -> None:
        self.values = tuple(values)

    def __contains__(self, candidate) -> bool:
        for allowed in self.values:
            if pin_values_equal(allowed, candidate):
                return True
        return False

    def __repr__(self) -> str:
        return "OneOf" + repr(self.values)


@dataclass(frozen=True)
class RoundingSchedule:
    """What an implementation computes. ``machine_assertable`` maps a key to a literal, ``PER_MODEL`` or a
    ``OneOf``; these keys are also the only pins the implementation accepts. ``documentary`` is prose. A change to
    either is a new version of the implementation."""

    machine_assertable: "dict[str, object]" = field(default_factory=dict)
    documentary: str = ""           # prose; hashed with the rest

    def check_pin(self, key: str, value) -> Optional[str]:
        """Why pinning ``key`` to ``value`` contradicts this schedule, or None if it does not. Pinning a key the
        schedule does not have is refused too: it would be hashed and compared while constraining nothing."""
        try:
            declared = self.machine_assertable[key]
        except KeyError:
            have = sorted(map(str, self.machine_assertable))
            return (f"the impl's machine_assertable rounding schedule declares no such key (declared: {have}). "
                    "A pin the impl never declared constrains nothing -- declare it (a literal, PER_MODEL, or "
                    "OneOf(...)) or drop the pin.")
        if declared is PER_MODEL:
            return None
        if isinstance(declared, OneOf):
            agrees = value in declared
        else:
            agrees = pin_values_equal(declared, value)
        return None if agrees else f"the impl declares {key}={declared!r}"


@dataclass(frozen=True)
class StateInvalidation:
    """For an op that keeps state: the condition under which the state has to be rebound, and optionally a
    host-side ``hook(state, ctx) -> bool`` that is True while the state is still good."""

    condition: str                                  # in words
    hook: "Callable[..., bool] | None" = None       # host-side check, optional


@dataclass(frozen=True)
class ImplSpec:
    """An implementation of an op at one version. ``subsumes``: ops it absorbs (they then install nothing of their
    own). ``hazards``: the least its parity tests exercise."""

    impl_id: str                    # unique within its op
    version: int                    # bumped whenever the rounding schedule changes
    supported_archs: frozenset      # architecture tags the bits were established on
    rounding: "RoundingSchedule" = field(default_factory=lambda: RoundingSchedule())
    capabilities: "dict[str, object]" = field(default_factory=dict)
    subsumes: "tuple[str, ...]" = ()
    state_invalidation: "StateInvalidation | None" = None
    hazards: "tuple[str, ...]" = ()
    route: str = "protected"        # one of _ROUTES

    def __post_init__(self) -> None:
        me = f"impl {self.impl_id!r}"
        if self.route not in _ROUTES:
            raise RegistryError(f"{me} declares unknown route {self.route!r}")
        unknown = sorted(set(self.hazards).difference(HAZARDS))
        if unknown:
            raise RegistryError(f"{me} declares unknown hazard(s) {unknown}; the hazard vocabulary is {sorted(HAZARDS)}")
        if len(self.supported_archs) == 0:
            raise RegistryError(f"{me} must declare at least one supported arch")


@dataclass
class OpSpec:
    name: str                                   # "family.op"
    sites: "list[str]"                          # where the op exists
    impls: "dict[str, ImplSpec]" = field(default_factory=dict)
    per_layer_uniform: bool = True              # resolved once, for every layer

    def add_impl(self, impl: ImplSpec) -> "OpSpec":
        """Chainable. One impl id, one impl."""
        if self.impls.setdefault(impl.impl_id, impl) is not impl:
            raise RegistryError(f"op {self.name!r} already has impl {impl.impl_id!r}")
        return self


class Registry:
    """Ops by name, plus the site vocabulary (which a deployment may extend before registering ops)."""

    def __init__(self) -> None:
        self._ops: "dict[str, OpSpec]" = dict()
        self._sites = set(_BASE_SITES)

    # -- sites
    @property
    def sites(self) -> frozenset:
        return frozenset(self._sites)

    def register_site(self, name: str) -> None:
        looks_like_identifier = bool(name) and name.replace("_", "").isalnum()
        if not looks_like_identifier:
            raise RegistryError(f"invalid site name {name!r}: must be a non-empty identifier")
        self._sites.add(name)

    # -- ops
    @property
    def ops(self) -> "dict[str, OpSpec]":
        """A copy: registering goes through ``register_op``."""
        return {name: op for name, op in self._ops.items()}

    def has_op(self, name: str) -> bool:
        return name in self._ops

    def get_op(self, name: str) -> OpSpec:
        if name not in self._ops:
            raise RegistryError(f"unknown op {name!r}")
        return self._ops[name]

    def register_op(self, op: OpSpec) -> OpSpec:
        if self.has_op(op.name):
            raise RegistryError(f"op {op.name!r} already registered")
        unknown = sorted(set(op.sites).difference(self._sites))
        if unknown:
            raise RegistryError(f"op {op.name!r} declares unknown site(s) {unknown}; register them first via "
                                f"register_site(). Known sites: {sorted(self._sites)}")
        self._ops[op.name] = op
        return op

    def installed_keys(self) -> frozenset:
        """Every (op, site) pair that exists."""
        return frozenset((name, site) for name, op in self._ops.items() for site in op.sites)

    def assert_subsumption_closed(self) -> None:
        """An absorbed op must itself be registered, or nothing can say what was absorbed."""
        for name, op in self._ops.items():
            for impl_id, impl in op.impls.items():
                missing = [a for a in impl.subsumes if a not in self._ops]
                if missing:
                    raise RegistryError(f"impl {name}:{impl_id} subsumes unregistered op {missing[0]!r}; its "
                                        f"passthrough cannot be derived")
