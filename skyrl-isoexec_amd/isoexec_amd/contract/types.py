"""The records an ExecutionContract is made of: immutable data, no I/O, no registry access.

The records are GENERATED from the schema table below. A record's field names and their order are the wire format
of the reference (isoexec/contract/types.py:1-132), so a contract frozen there decodes here and hashes to the same
three identities; the table adds to every field the ``wire`` tag that ``serialize.py`` encodes, strictly decodes and
projects identities by, which makes the table the one description of the format.

Wire tags: ``"val"`` a JSON scalar (str, int, bool, None) stored as is; ``"strs"`` a tuple of scalars, a JSON list;
``"map"`` (key, value) pairs in key order, a JSON object whose values may be BitPattern objects; ``"pair"`` exactly
two strings; a record class = a nested record; ``[cls]`` = a tuple of records; ``("opt", cls)`` = a record or None.
"""

from __future__ import annotations

import dataclasses
from collections.abc import Mapping

# Closed vocabularies (reference: contract/types.py:6-14).
ROUTES = frozenset(("canonical", "composition_defining", "protected", "reference_preserving"))
HALVES = frozenset(("deployment", "function"))
DISCHARGE_KINDS = frozenset(("bitwise_equal_to", "equivalence_proof", "neutrality_proof"))
COVERAGE_KINDS = frozenset(("enumerated_shapes", "symbolic_domain"))
TOPOLOGY_KINDS = frozenset(("invariant", "pinned"))
# A lifecycle event belongs here only if some boundary of the system observes it; anything else would be prose
# that gets hashed.
STATE_EVENTS = frozenset(("sleep_wake", "weight_sync"))

_REQUIRED = object()


def sorted_pairs(m) -> tuple:
    """A mapping, or any iterable of pairs, as a tuple of (str key, value) pairs ordered by key."""
    pairs = m.items() if isinstance(m, Mapping) else m
    return tuple(sorted(((str(k), v) for k, v in pairs), key=lambda kv: kv[0]))


def _record(name: str, doc: str, columns, normalise=()):
    """A frozen dataclass ``name`` with one field per (field name, wire tag, default) column. ``normalise`` names the
    "map" fields that are put into key order on construction."""
    specs = []
    for column in columns:
        field_name, tag = column[0], column[1]
        default = column[2] if len(column) > 2 else _REQUIRED
        options = {"metadata": {"wire": tag}}
        if default is dataclasses.MISSING or default is _REQUIRED:
            pass
        elif callable(default):
            options["default_factory"] = default
        else:
            options["default"] = default
        specs.append((field_name, object, dataclasses.field(**options)))
    namespace = {"__doc__": doc}
    if normalise:
        def __post_init__(self, _fields=tuple(normalise)):
            for f in _fields:
                object.__setattr__(self, f, sorted_pairs(getattr(self, f)))
        namespace["__post_init__"] = __post_init__
    cls = dataclasses.make_dataclass(name, specs, frozen=True, namespace=namespace)
    cls.__module__ = __name__
    return cls


BitPattern = _record("BitPattern", "The only way a floating-point constant travels: its bits in hex and the dtype's name.",
                     [("bits", "val"), ("dtype", "val")])

ImplRef = _record("ImplRef", "An implementation by id, version and the architecture it was resolved for.",
                  [("id", "val"), ("version", "val"), ("arch", "val")])

EquivalenceProof = _record("EquivalenceProof", "A discharge: what kind of argument, and where it lives.",
                           [("kind", "val"), ("ref", "val")])

Coverage = _record("Coverage", "What an entry's claim ranges over.", [("kind", "val"), ("description", "val")])

ModelRef = _record("ModelRef", "The model the contract was derived for.",
                   [("family", "val"), ("architectures", "strs"), ("profile_ref", "val")])

Identities = _record("Identities", "The three hashes of a contract.",
                     [("semantic", "val"), ("numerical_policy", "val"), ("deployment", "val")])

ExecutionCase = _record("ExecutionCase", "A situation the model runs in (who, with or without gradients, which state, which shapes).",
                        [("id", "val"), ("runtime_role", "val"), ("grad_mode", "val"), ("state_mode", "val"),
                         ("shape_domain", "val"), ("constraints", "strs", ())])

CompositionEntry = _record(
    "CompositionEntry", "One unit of the partition: a sorted group of logical ops that one impl runs under a set of cases.",
    [("region", "strs"), ("cases", "strs"), ("impl", ImplRef), ("route", "val"), ("constants", "map", ()),
     ("artifact", "val", None), ("reference", ("opt", ImplRef), None), ("coverage", ("opt", Coverage), None),
     ("discharge", ("opt", EquivalenceProof), None), ("half", "val", "function")],
    normalise=("constants",))

TopologyClaim = _record("TopologyClaim", "A parallelism axis, either pinned to a degree or claimed invariant over a domain.",
                        [("axis", "val"), ("kind", "val"), ("degree", "val", None), ("collective_plan", "val", None),
                         ("domain", "strs", ()), ("proof", "val", None)])

StateClaim = _record("StateClaim", "A piece of carried state and the events that invalidate it.",
                     [("state_id", "val"), ("invalidated_by", "strs"), ("replay_safe", "val"), ("ref", "val")])

ToleranceClaim = _record("ToleranceClaim", "An accepted envelope between two cases; bounds are decimal strings, hashed as written.",
                         [("case_pair", "pair"), ("bounds", "map", ()), ("attributed_to", "strs", ())],
                         normalise=("bounds",))

Claims = _record("Claims", "Everything a contract claims beyond its composition.",
                 [("topology", [TopologyClaim], ()), ("state", [StateClaim], ()), ("tolerances", [ToleranceClaim], ())])

ExecutionContract = _record(
    "ExecutionContract", "The frozen contract.",
    [("schema_version", "val"), ("model", ModelRef), ("identities", Identities), ("cases", [ExecutionCase]),
     ("composition", [CompositionEntry]), ("claims", Claims, Claims)])
