"""The three identities of a contract: sha256 over canonical bytes of three projections.

Reference: isoexec/contract/identity.py:30-106. The projections are taken from the plain (wire) form
of each record, so there is exactly one description of a record's fields:

* ``numerical_policy`` hashes everything that can move bits: the function-half entries, the topology
  claims and the cases themselves;
* ``deployment`` hashes what is compared but proven not to move bits: deployment-half entries, state
  claims and tolerance envelopes;
* ``semantic`` hashes what the model means: its identity, the logical-op vocabulary and the cases.

Order never matters: every list inside a projection is sorted (by canonical bytes for records).
"""

from __future__ import annotations

import hashlib

from .types import ExecutionContract, Identities
from .serialize import canonical_bytes, to_plain


def _entry_view(entry) -> dict:
    # Bit-relevant fields only: ``half`` selects the projection and is not hashed, the case list is a
    # set, and coverage contributes its kind but not its prose.
    view = to_plain(entry)
    del view["half"]
    view["cases"] = sorted(view["cases"])
    if view["coverage"] is not None:
        view["coverage"] = view["coverage"]["kind"]
    return view


def _case_view(case) -> dict:
    view = to_plain(case)
    view["constraints"] = sorted(view["constraints"])
    return view


def _by_bytes(plains) -> list:
    return sorted(plains, key=canonical_bytes)


def function_half(contract: ExecutionContract) -> dict:
    return {
        "schema_version": contract.schema_version,
        "cases": _by_bytes(_case_view(c) for c in contract.cases),
        "entries": _by_bytes(_entry_view(e) for e in contract.composition if e.half == "function"),
        "topology": _by_bytes(to_plain(t) for t in contract.claims.topology),
    }


def deployment_half(contract: ExecutionContract) -> dict:
    return {
        "entries": _by_bytes(_entry_view(e) for e in contract.composition if e.half == "deployment"),
        "state": _by_bytes(to_plain(s) for s in contract.claims.state),
        "tolerances": _by_bytes(to_plain(t) for t in contract.claims.tolerances),
    }


def semantic_inputs(contract: ExecutionContract) -> dict:
    model = to_plain(contract.model)
    model["architectures"] = sorted(model["architectures"])
    return {
        "model": model,
        "logical_ops": sorted({op for e in contract.composition for op in e.region}),
        "cases": _by_bytes(_case_view(c) for c in contract.cases),
    }


def digest(plain) -> str:
    return hashlib.sha256(canonical_bytes(plain)).hexdigest()


def compute_identities(contract: ExecutionContract) -> Identities:
    """All three hashes recomputed from content; the stored ``identities`` field is not read."""
    return Identities(
        semantic=digest(semantic_inputs(contract)),
        numerical_policy=digest(function_half(contract)),
        deployment=digest(deployment_half(contract)),
    )
