"""Structural checks on a frozen contract (build time and CI).

``validate`` returns every complaint as text, an empty list meaning the contract is well formed. The checks are
grouped by what they look at -- the header, each entry on its own, who owns which op inside a case, regions served
by several impls, and the three claim families -- and the rule set is the reference's
(isoexec/contract/validate.py:35-175).
"""

from __future__ import annotations

import math
import re
from collections import defaultdict
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


class ValidationError(Exception):
    pass


class _Complaints(list):
    """Collects complaints; ``unless(ok, text)`` records ``text`` when ``ok`` does not hold."""

    def unless(self, ok, text: str) -> bool:
        if not ok:
            self.append(text)
        return bool(ok)


def _is_hex_word(text: str) -> bool:
    return re.fullmatch(r"0x[0-9a-fA-F]+", text) is not None


def _is_finite_number(text) -> bool:
    """A threshold must compare: "nan" and "inf" parse as numbers and would let everything through."""
    try:
        return math.isfinite(float(text))
    except (TypeError, ValueError):
        return False


# ---- one entry at a time -------------------------------------------------------------------------------------
def _entry_shape(out: _Complaints, tag: str, e) -> None:
    out.unless(len(e.region) > 0, f"{tag}: empty region")
    out.unless(list(e.region) == sorted(e.region), f"{tag}: region tuple must be sorted")
    out.unless(e.route in ROUTES, f"{tag}: unknown route {e.route!r}")
    out.unless(e.half in HALVES, f"{tag}: unknown half {e.half!r}")
    proof = e.discharge
    if proof is not None:
        out.unless(proof.kind in DISCHARGE_KINDS, f"{tag}: unknown discharge kind {proof.kind!r}")
        out.unless(proof.ref.strip() != "", f"{tag}: {proof.kind} discharge with an empty ref")
    if e.coverage is not None:
        out.unless(e.coverage.kind in COVERAGE_KINDS, f"{tag}: unknown coverage kind {e.coverage.kind!r}")


def _entry_obligations(out: _Complaints, tag: str, e) -> None:
    """What a route or a half obliges an entry to carry."""
    if e.route == "composition_defining":
        out.unless(e.artifact is not None, f"{tag}: composition_defining requires an artifact")
    if e.route == "reference_preserving":
        out.unless(e.reference is not None, f"{tag}: reference_preserving requires a reference")
    if e.half == "deployment":
        neutral = e.discharge is not None and e.discharge.kind == "neutrality_proof"
        out.unless(neutral, f"{tag}: deployment-half entry requires a neutrality_proof discharge")


def _entry_constants(out: _Complaints, tag: str, e) -> None:
    for name, value in e.constants:
        out.unless(not isinstance(value, float), f"{tag}: constant {name!r} is a raw float")
        if isinstance(value, BitPattern):
            out.unless(_is_hex_word(value.bits), f"{tag}: constant {name!r} has invalid bit pattern {value.bits!r}")


def _entries(out: _Complaints, contract, case_ids) -> None:
    claims = set()
    for e in contract.composition:
        tag = f"entry {e.region}@{e.impl.id}"
        _entry_shape(out, tag, e)
        for case in e.cases:
            out.unless(case in case_ids, f"{tag}: unknown case {case!r}")
            out.unless((e.region, case) not in claims, f"{tag}: duplicate (region, case) claim for {case!r}")
            claims.add((e.region, case))
        _entry_obligations(out, tag, e)
        _entry_constants(out, tag, e)


# ---- across entries ------------------------------------------------------------------------------------------
def _ownership(out: _Complaints, contract, case_ids, required) -> None:
    """Inside one case an op has one owning region, and every op the case needs has an owner."""
    for case in case_ids:
        owner = {}
        for e in contract.composition:
            if case in e.cases:
                for op in e.region:
                    prior = owner.setdefault(op, e.region)
                    out.unless(prior == e.region, f"case {case!r}: op {op!r} owned by both {prior} and {e.region}")
                    owner[op] = e.region
        needed = (required or {}).get(case)
        if needed is not None:
            orphans = sorted(set(needed) - owner.keys())
            out.unless(not orphans, f"case {case!r}: uncovered required op(s) {orphans}")


def _asymmetry(out: _Complaints, contract) -> None:
    """A region that different cases run with different impls owes a discharge on every one of its entries."""
    by_region = defaultdict(list)
    for e in contract.composition:
        by_region[e.region].append(e)
    for region, group in by_region.items():
        if len({e.impl.id for e in group}) < 2:
            continue
        for e in group:
            out.unless(e.discharge is not None, f"entry {region}@{e.impl.id}: asymmetric region requires a discharge")


# ---- claims --------------------------------------------------------------------------------------------------
def _tolerances(out: _Complaints, contract, case_ids) -> None:
    for t in contract.claims.tolerances:
        tag = f"tolerance {t.case_pair}"
        for case in t.case_pair:
            out.unless(case in case_ids, f"{tag}: unknown case {case!r}")
        out.unless(len(t.bounds) > 0, f"{tag}: no bounds (an envelope without a threshold admits everything)")
        for name, bound in t.bounds:
            out.unless(_is_finite_number(bound), f"{tag}: bound {name}={bound!r} is not a finite threshold")


def _state_claims(out: _Complaints, contract) -> None:
    for s in contract.claims.state:
        tag = f"state {s.state_id!r}"
        out.unless(s.ref.strip() != "", f"{tag}: empty ref (no hook is named that implements the claim)")
        out.unless(len(s.invalidated_by) > 0, f"{tag}: empty invalidated_by (nothing ever invalidates this state?)")
        unknown = sorted(set(s.invalidated_by) - STATE_EVENTS)
        out.unless(not unknown, f"{tag}: unknown lifecycle event(s) {unknown}; the vocabulary is {sorted(STATE_EVENTS)} "
                                f"(an event no boundary observes cannot be enforced)")


def _one_topology_claim(out: _Complaints, t) -> None:
    tag = f"topology {t.axis!r}"
    if t.proof is not None:
        out.unless(t.proof.strip() != "", f"{tag}: empty proof ref (it names nothing)")
    if not out.unless(t.kind in TOPOLOGY_KINDS, f"{tag}: unknown kind {t.kind!r}"):
        return
    if t.kind == "pinned":
        if out.unless(t.degree is not None and t.collective_plan is not None,
                      f"{tag}: pinned requires degree and collective_plan"):
            out.unless(t.degree >= 1, f"{tag}: pinned degree {t.degree} is not a deployable degree (>= 1)")
        return
    if out.unless(bool(t.domain) and bool(t.proof), f"{tag}: invariant requires a non-empty domain and a proof"):
        degrees = sorted(set(t.domain))
        out.unless(len(degrees) >= 2, f"{tag}: invariant over the single degree {degrees} is a tautology, not an "
                                      f"invariance claim; pin the axis instead")


def _topology(out: _Complaints, contract) -> None:
    axes = [t.axis for t in contract.claims.topology]
    out.unless(len(set(axes)) == len(axes), "duplicate topology axes")
    for t in contract.claims.topology:
        _one_topology_claim(out, t)


def _identities(out: _Complaints, contract) -> None:
    try:
        recomputed = compute_identities(contract)
    except SerializationError as exc:
        out.append(f"identity recomputation failed: {exc}")
        return
    out.unless(contract.identities == recomputed, "stored identities do not match recomputed identities")


def validate(contract: ExecutionContract, required_ops: Mapping | None = None) -> list:
    """Every complaint about ``contract``, as text. ``required_ops`` maps a case id to the ops that case must
    have an owner for."""
    out = _Complaints()
    case_ids = {c.id for c in contract.cases}
    out.unless(contract.schema_version in SUPPORTED_SCHEMA_VERSIONS, f"unsupported schema_version {contract.schema_version!r}")
    out.unless(len(case_ids) == len(contract.cases), "duplicate case ids")
    out.unless(len(contract.composition) > 0,
               "empty composition: a contract with no entry claims nothing, and two processes that both failed to "
               "derive a composition would then agree perfectly")
    _entries(out, contract, case_ids)
    _ownership(out, contract, case_ids, required_ops)
    _asymmetry(out, contract)
    _tolerances(out, contract, case_ids)
    _state_claims(out, contract)
    _topology(out, contract)
    _identities(out, contract)
    return list(out)


def validate_or_raise(contract: ExecutionContract, required_ops: Mapping | None = None) -> None:
    complaints = validate(contract, required_ops)
    if complaints:
        raise ValidationError("; ".join(complaints))
