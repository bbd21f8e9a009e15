"""ExecutionContract: record types, canonical JSON, identities, structural validation.

Mirrors the public surface of the reference's ``isoexec/contract`` package
(contract/__init__.py:1-71).
"""

from .identity import compute_identities, deployment_half, function_half, semantic_inputs
from .types import (
    COVERAGE_KINDS,
    DISCHARGE_KINDS,
    HALVES,
    ROUTES,
    STATE_EVENTS,
    TOPOLOGY_KINDS,
    BitPattern,
    Claims,
    CompositionEntry,
    Coverage,
    EquivalenceProof,
    ExecutionCase,
    ExecutionContract,
    Identities,
    ImplRef,
    ModelRef,
    StateClaim,
    ToleranceClaim,
    TopologyClaim,
)
from .validate import ValidationError, validate, validate_or_raise
from .serialize import (
    SUPPORTED_SCHEMA_VERSIONS,
    SerializationError,
    UnknownFieldError,
    canonical_bytes,
    encode_constants,
    from_canonical_json,
    to_canonical_json,
)

SCHEMA_VERSION = "2"


def freeze(contract: ExecutionContract) -> ExecutionContract:
    """The same contract with its identities recomputed from content."""
    import dataclasses

    return dataclasses.replace(contract, identities=compute_identities(contract))
