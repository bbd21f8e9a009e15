"""The ExecutionContract record types: immutable data, no I/O, no registry access.

Field names and their order are the wire format (reference: isoexec/contract/types.py:1-132), so a
contract frozen by the reference decodes here and hashes to the same three identities. Each field
carries a ``wire`` tag that the codec in ``serialize.py`` interprets; that table is the single description
of the format, used for encoding, strict decoding and the identity projections alike.

Wire tags:
    "val"        a JSON scalar (str / int / bool / None), stored as is
    "strs"       a tuple of scalars, written as a JSON list
    "map"        sorted (key, value) pairs, written as a JSON object; a BitPattern value is an object
    "pair"       exactly two strings, written as a two-element list
    <class>      a nested record
    [<class>]    a tuple of nested records
    ?<class>     a nested record or None (spelled ("opt", <class>))
"""

from __future__ import annotations

from collections.abc import Mapping
from dataclasses import dataclass, field

# Closed vocabularies (reference: contract/types.py:6-14).
ROUTES = frozenset({"reference_preserving", "composition_defining", "protected", "canonical"})
DISCHARGE_KINDS = frozenset({"bitwise_equal_to", "equivalence_proof", "neutrality_proof"})
COVERAGE_KINDS = frozenset({"enumerated_shapes", "symbolic_domain"})
HALVES = frozenset({"function", "deployment"})
TOPOLOGY_KINDS = frozenset({"pinned", "invariant"})
# Only lifecycle events that some boundary observes; anything else would be hashed prose.
STATE_EVENTS = frozenset({"weight_sync", "sleep_wake"})


def _w(tag, **kw):
    return field(metadata={"wire": tag}, **kw)


def sorted_pairs(m) -> tuple:
    """A Mapping or an iterable of pairs -> a tuple of (str key, value) pairs in key order."""
    items = m.items() if isinstance(m, Mapping) else tuple(m)
    return tuple(sorted((str(k), v) for k, v in items))


@dataclass(frozen=True)
class BitPattern:
    """The only carrier a floating-point constant may travel in: hex bits plus the dtype name."""

    bits: str = _w("val")
    dtype: str = _w("val")


@dataclass(frozen=True)
class ImplRef:
    id: str = _w("val")
    version: int = _w("val")
    arch: str = _w("val")


@dataclass(frozen=True)
class EquivalenceProof:
    kind: str = _w("val")
    ref: str = _w("val")


@dataclass(frozen=True)
class Coverage:
    kind: str = _w("val")
    description: str = _w("val")


@dataclass(frozen=True)
class ModelRef:
    family: str = _w("val")
    architectures: tuple = _w("strs")
    profile_ref: str = _w("val")


@dataclass(frozen=True)
class Identities:
    semantic: str = _w("val")
    numerical_policy: str = _w("val")
    deployment: str = _w("val")


@dataclass(frozen=True)
class ExecutionCase:
    id: str = _w("val")
    runtime_role: str = _w("val")
    grad_mode: str = _w("val")
    state_mode: str = _w("val")
    shape_domain: str = _w("val")
    constraints: tuple = _w("strs", default=())


@dataclass(frozen=True)
class CompositionEntry:
    """One partition unit: a sorted group of logical ops run by one impl under a set of cases."""

    region: tuple = _w("strs")
    cases: tuple = _w("strs")
    impl: ImplRef = _w(ImplRef)
    route: str = _w("val")
    constants: tuple = _w("map", default=())
    artifact: str | None = _w("val", default=None)
    reference: ImplRef | None = _w(("opt", ImplRef), default=None)
    coverage: Coverage | None = _w(("opt", Coverage), default=None)
    discharge: EquivalenceProof | None = _w(("opt", EquivalenceProof), default=None)
    half: str = _w("val", default="function")

    def __post_init__(self):
        object.__setattr__(self, "constants", sorted_pairs(self.constants))


@dataclass(frozen=True)
class TopologyClaim:
    axis: str = _w("val")
    kind: str = _w("val")
    degree: int | None = _w("val", default=None)
    collective_plan: str | None = _w("val", default=None)
    domain: tuple = _w("strs", default=())
    proof: str | None = _w("val", default=None)


@dataclass(frozen=True)
class StateClaim:
    state_id: str = _w("val")
    invalidated_by: tuple = _w("strs")
    replay_safe: bool = _w("val")
    ref: str = _w("val")


@dataclass(frozen=True)
class ToleranceClaim:
    case_pair: tuple = _w("pair")
    bounds: tuple = _w("map", default=())  # values are decimal strings, hashed as written
    attributed_to: tuple = _w("strs", default=())

    def __post_init__(self):
        object.__setattr__(self, "bounds", sorted_pairs(self.bounds))


@dataclass(frozen=True)
class Claims:
    topology: tuple = _w([TopologyClaim], default=())
    state: tuple = _w([StateClaim], default=())
    tolerances: tuple = _w([ToleranceClaim], default=())


@dataclass(frozen=True)
class ExecutionContract:
    schema_version: str = _w("val")
    model: ModelRef = _w(ModelRef)
    identities: Identities = _w(Identities)
    cases: tuple = _w([ExecutionCase])
    composition: tuple = _w([CompositionEntry])
    claims: Claims = _w(Claims, default_factory=Claims)
