"""The ExecutionContract: its records, its canonical bytes, its three identities and its structural checks.
The names exported here are those of the reference's ``isoexec/contract`` package (contract/__init__.py:1-71)."""

import dataclasses as _dataclasses

from .identity import compute_identities, deployment_half, function_half, semantic_inputs
from .serialize import (SUPPORTED_SCHEMA_VERSIONS, SerializationError, UnknownFieldError, canonical_bytes,
                        encode_constants, from_canonical_json, to_canonical_json)
from .types import (COVERAGE_KINDS, DISCHARGE_KINDS, HALVES, ROUTES, STATE_EVENTS, TOPOLOGY_KINDS, BitPattern, Claims,
                    CompositionEntry, Coverage, EquivalenceProof, ExecutionCase, ExecutionContract, Identities, ImplRef,
                    ModelRef, StateClaim, ToleranceClaim, TopologyClaim)
from .validate import ValidationError, validate, validate_or_raise

SCHEMA_VERSION = "2"


def freeze(contract: ExecutionContract) -> ExecutionContract:
    """``contract`` with the identities its content hashes to."""
    return _dataclasses.replace(contract, identities=compute_identities(contract))
