"""Structural invariants of a frozen contract, checked at build time and in CI.

Each rule is a generator of human-readable violations; ``validate`` runs all of them and returns the
list (empty = valid). The rule set follows the reference's (isoexec/contract/validate.py:38-167).
"""

from __future__ import annotations

import math
import re
from collections.abc import Mapping

from .identity import compute_identities
from .serialize import SUPPORTED_SCHEMA_VERSIONS, SerializationError
from .types import (
    COVERAGE_KINDS,
    DISCHARGE_KINDS,
    HALVES,
    ROUTES,
    STATE_EVENTS,
    TOPOLOGY_KINDS,
    BitPattern,
    ExecutionContract,
)

_HEX_BITS = re.compile(r"^0x[0-9a-fA-F]+$")


class ValidationError(Exception):
    pass


def _finite_decimal(text) -> bool:
    # "nan" and "inf" parse as floats and would make a threshold comparison admit everything.
    try:
        return math.isfinite(float(text))
    except (TypeError, ValueError):
        return False


def _label(entry) -> str:
    return f"entry {entry.region}@{entry.impl.id}"


def _rule_header(c, case_ids, required):
    if c.schema_version not in SUPPORTED_SCHEMA_VERSIONS:
        yield f"unsupported schema_version {c.schema_version!r}"
    if len(case_ids) != len(c.cases):
        yield "duplicate case ids"
    if not c.composition:
        yield (
            "empty composition: a contract naming no entry claims nothing, and two processes that both "
            "failed to derive a composition would agree perfectly"
        )


def _rule_entries(c, case_ids, required):
    claimed = set()
    for e in c.composition:
        who = _label(e)
        if not e.region:
            yield f"{who}: empty region"
        if tuple(sorted(e.region)) != tuple(e.region):
            yield f"{who}: region tuple must be sorted"
        if e.route not in ROUTES:
            yield f"{who}: unknown route {e.route!r}"
        if e.half not in HALVES:
            yield f"{who}: unknown half {e.half!r}"
        if e.discharge is not None:
            if e.discharge.kind not in DISCHARGE_KINDS:
                yield f"{who}: unknown discharge kind {e.discharge.kind!r}"
            if not e.discharge.ref.strip():
                yield f"{who}: {e.discharge.kind} discharge with an empty ref"
        if e.coverage is not None and e.coverage.kind not in COVERAGE_KINDS:
            yield f"{who}: unknown coverage kind {e.coverage.kind!r}"
        for cid in e.cases:
            if cid not in case_ids:
                yield f"{who}: unknown case {cid!r}"
            if (e.region, cid) in claimed:
                yield f"{who}: duplicate (region, case) claim for {cid!r}"
            claimed.add((e.region, cid))
        if e.route == "composition_defining" and e.artifact is None:
            yield f"{who}: composition_defining requires an artifact"
        if e.route == "reference_preserving" and e.reference is None:
            yield f"{who}: reference_preserving requires a reference"
        if e.half == "deployment" and (e.discharge is None or e.discharge.kind != "neutrality_proof"):
            yield f"{who}: deployment-half entry requires a neutrality_proof discharge"
        for key, const in e.constants:
            if isinstance(const, float):
                yield f"{who}: constant {key!r} is a raw float"
            if isinstance(const, BitPattern) and not _HEX_BITS.match(const.bits):
                yield f"{who}: constant {key!r} has invalid bit pattern {const.bits!r}"


def _rule_ownership(c, case_ids, required):
    # Within one case a logical op belongs to at most one region; required ops must all be owned.
    for cid in case_ids:
        owner = {}
        for e in c.composition:
            if cid not in e.cases:
                continue
            for op in e.region:
                if op in owner and owner[op] != e.region:
                    yield f"case {cid!r}: op {op!r} owned by both {owner[op]} and {e.region}"
                owner[op] = e.region
        if required is not None and cid in required:
            uncovered = required[cid] - set(owner)
            if uncovered:
                yield f"case {cid!r}: uncovered required op(s) {sorted(uncovered)}"


def _rule_asymmetry(c, case_ids, required):
    # One region run by different impls under different cases: every such entry carries its proof.
    impls_of = {}
    for e in c.composition:
        impls_of.setdefault(e.region, []).append(e)
    for region, group in impls_of.items():
        if len({e.impl.id for e in group}) > 1:
            for e in group:
                if e.discharge is None:
                    yield f"entry {region}@{e.impl.id}: asymmetric region requires a discharge"


def _rule_tolerances(c, case_ids, required):
    for t in c.claims.tolerances:
        for cid in t.case_pair:
            if cid not in case_ids:
                yield f"tolerance {t.case_pair}: unknown case {cid!r}"
        if not t.bounds:
            yield f"tolerance {t.case_pair}: no bounds (an envelope with no threshold admits everything)"
        for key, bound in t.bounds:
            if not _finite_decimal(bound):
                yield f"tolerance {t.case_pair}: bound {key}={bound!r} is not a finite threshold"


def _rule_state(c, case_ids, required):
    for s in c.claims.state:
        if not s.ref.strip():
            yield f"state {s.state_id!r}: empty ref (the claim names no implementing hook)"
        if not s.invalidated_by:
            yield f"state {s.state_id!r}: empty invalidated_by (a state invalidated by nothing is not a claim)"
        stray = sorted(set(s.invalidated_by) - STATE_EVENTS)
        if stray:
            yield (
                f"state {s.state_id!r}: unknown lifecycle event(s) {stray}; the vocabulary is "
                f"{sorted(STATE_EVENTS)} -- an event no boundary observes cannot be enforced"
            )


def _rule_topology(c, case_ids, required):
    axes = [t.axis for t in c.claims.topology]
    if len(axes) != len(set(axes)):
        yield "duplicate topology axes"
    for t in c.claims.topology:
        if t.proof is not None and not t.proof.strip():
            yield f"topology {t.axis!r}: empty proof ref (a proof that names nothing is not a proof)"
        if t.kind not in TOPOLOGY_KINDS:
            yield f"topology {t.axis!r}: unknown kind {t.kind!r}"
        elif t.kind == "pinned":
            if t.degree is None or t.collective_plan is None:
                yield f"topology {t.axis!r}: pinned requires degree and collective_plan"
            elif t.degree < 1:
                yield f"topology {t.axis!r}: pinned degree {t.degree} is not a deployable degree (>= 1)"
        elif not t.domain or not t.proof:
            yield f"topology {t.axis!r}: invariant requires a non-empty domain and a proof"
        elif len(set(t.domain)) < 2:
            yield (
                f"topology {t.axis!r}: invariant over the single degree {sorted(set(t.domain))} is a "
                f"tautology, not an invariance claim; pin the axis instead"
            )


def _rule_identities(c, case_ids, required):
    try:
        fresh = compute_identities(c)
    except SerializationError as exc:
        yield f"identity recomputation failed: {exc}"
        return
    if c.identities != fresh:
        yield "stored identities do not match recomputed identities"


_RULES = (
    _rule_header,
    _rule_entries,
    _rule_ownership,
    _rule_asymmetry,
    _rule_tolerances,
    _rule_state,
    _rule_topology,
    _rule_identities,
)


def validate(contract: ExecutionContract, required_ops: Mapping | None = None) -> list:
    """Every violation of the structural rules, as text. ``required_ops`` maps a case id to the set
    of logical ops that case must have an owner for."""
    case_ids = {c.id for c in contract.cases}
    found = []
    for rule in _RULES:
        found.extend(rule(contract, case_ids, required_ops))
    return found


def validate_or_raise(contract: ExecutionContract, required_ops: Mapping | None = None) -> None:
    problems = validate(contract, required_ops)
    if problems:
        raise ValidationError("; ".join(problems))
