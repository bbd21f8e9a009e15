"""Deliver a frozen contract as a file both runtimes read, cross-checked against an environment hash.

Reference: isoexec/core/contract_delivery.py:20-104.
"""

from __future__ import annotations

import logging
import os

from ..contract import ExecutionContract, compute_identities, from_canonical_json, to_canonical_json
from .fingerprint import ResolvedFingerprint
from .registry import Registry

CONTRACT_HASH_ENV = "ISOEXEC_CONTRACT_HASH"


class ContractDeliveryError(ValueError):
    pass


def write_contract_file(contract: ExecutionContract, path: str) -> str:
    """Write the canonical bytes atomically; returns the numerical_policy hash to export alongside."""
    scratch = f"{path}.tmp.{os.getpid()}"
    with open(scratch, "wb") as fh:
        fh.write(to_canonical_json(contract))
    os.replace(scratch, path)
    return contract.identities.numerical_policy


def load_contract(path: str, expected_hash_env: str = CONTRACT_HASH_ENV) -> ExecutionContract:
    """Read a delivered contract. File self-consistency is always enforced; only the environment
    cross-check can be demoted."""
    from . import enforce

    with open(path, "rb") as fh:
        contract = from_canonical_json(fh.read())
    if compute_identities(contract) != contract.identities:
        raise ContractDeliveryError(f"serialized contract identities at {path!r} do not match the recomputed identities")
    stamped = os.environ.get(expected_hash_env)
    if stamped is not None and stamped != contract.identities.numerical_policy:
        msg = (
            f"contract delivery cross-check FAILED: {expected_hash_env}={stamped!r} but the file at {path!r} "
            f"carries numerical_policy {contract.identities.numerical_policy!r}."
        )
        enforce.report(f"{enforce.BUILD_VALID}:contract", enforce.INSTALL, enforce.VIOLATION, msg)
        if not enforce.demoted():
            raise ContractDeliveryError(msg)
        logging.getLogger(__name__).error("[ISOEXEC] demoted (violation still recorded): %s", msg)
    return contract


def primary_op(registry: Registry, entry) -> str:
    """The region member whose OpSpec registers the entry's impl; subsumed ops never install."""
    owners = [op for op in entry.region if registry.has_op(op) and entry.impl.id in registry.get_op(op).impls]
    if len(owners) != 1:
        raise ContractDeliveryError(
            f"entry {entry.region} impl {entry.impl.id!r}: expected exactly one owning op, got {owners}"
        )
    return owners[0]


_primary_op = primary_op


def expected_installed_keys(contract: ExecutionContract, registry: Registry) -> frozenset:
    return frozenset((primary_op(registry, e), case) for e in contract.composition for case in e.cases)


def validate_contract_against_installed(contract: ExecutionContract, registry: Registry, fingerprint) -> None:
    """Every installed (op, site) must be named by the contract and vice versa."""
    if isinstance(fingerprint, ResolvedFingerprint):
        installed = fingerprint.keys()
    elif isinstance(fingerprint, Registry):
        installed = fingerprint.installed_keys()
    else:
        installed = frozenset(fingerprint)
    named = expected_installed_keys(contract, registry)
    if installed != named:
        raise ContractDeliveryError(
            "contract does not match the installed composition:\n"
            f"  installed but UNNAMED by the contract: {sorted(installed - named)}\n"
            f"  named by the contract but NOT installed: {sorted(named - installed)}\n"
            "Every installed (op, site) carries an explicit entry; absence means 'no such site'."
        )
