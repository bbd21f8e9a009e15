"""Handing a frozen contract from the process that built it to the processes that run under it.

The contract travels as a file of canonical bytes; the hash of its numerical policy travels separately, in the
environment, and the reader compares the two. A second check compares what a process has installed with what the
contract names, key by key in both directions. (Reference: isoexec/core/contract_delivery.py:20-104.)
"""

from __future__ import annotations

import logging
import os
from typing import Iterable

from ..contract import ExecutionContract, compute_identities, from_canonical_json, to_canonical_json
from .fingerprint import ResolvedFingerprint
from .registry import Registry

CONTRACT_HASH_ENV = "ISOEXEC_CONTRACT_HASH"
_log = logging.getLogger(__name__)


class ContractDeliveryError(ValueError):
    """The delivered contract is not the one this process was told to expect, or not the one it installed."""


def write_contract_file(contract: ExecutionContract, path: str) -> str:
    """Publish the contract at ``path`` (readers never see a partial file) and return the hash that belongs in
    ``ISOEXEC_CONTRACT_HASH``."""
    staging = "%s.tmp.%d" % (path, os.getpid())
    with open(staging, "wb") as out:
        out.write(to_canonical_json(contract))
    os.replace(staging, path)
    return contract.identities.numerical_policy


def _environment_disagrees(contract: ExecutionContract, path: str, env_name: str):
    """The complaint to raise when the environment names another contract than the file holds, else None."""
    told = os.environ.get(env_name)
    held = contract.identities.numerical_policy
    if told is None or told == held:
        return None
    return (f"contract delivery cross-check FAILED: {env_name}={told!r} but the file at {path!r} carries "
            f"numerical_policy {held!r}.")


def load_contract(path: str, expected_hash_env: str = CONTRACT_HASH_ENV) -> ExecutionContract:
    """Read a delivered contract. A file whose stored identities are not the ones its content hashes to is always
    refused; a disagreement with the environment is recorded as a violation and refused unless enforcement has
    been demoted."""
    from . import enforce

    with open(path, "rb") as src:
        contract = from_canonical_json(src.read())
    if contract.identities != compute_identities(contract):
        raise ContractDeliveryError(f"serialized contract identities at {path!r} do not match the recomputed identities")
    complaint = _environment_disagrees(contract, path, expected_hash_env)
    if complaint:
        enforce.report(f"{enforce.BUILD_VALID}:contract", enforce.INSTALL, enforce.VIOLATION, complaint)
        if enforce.demoted():
            _log.error("[ISOEXEC] demoted (violation still recorded): %s", complaint)
        else:
            raise ContractDeliveryError(complaint)
    return contract


def primary_op(registry: Registry, entry) -> str:
    """Of the ops in an entry's region, the one whose declaration registers the entry's impl. The others were
    absorbed by that impl and install nothing."""
    impl_id = entry.impl.id
    owning = []
    for name in entry.region:
        if registry.has_op(name) and impl_id in registry.get_op(name).impls:
            owning.append(name)
    if len(owning) == 1:
        return owning[0]
    raise ContractDeliveryError(f"entry {entry.region} impl {impl_id!r}: expected exactly one owning op, got {owning}")


_primary_op = primary_op


def expected_installed_keys(contract: ExecutionContract, registry: Registry) -> frozenset:
    """Every (op, site) a process running under ``contract`` must have installed."""
    keys = set()
    for entry in contract.composition:
        op = primary_op(registry, entry)
        keys.update((op, site) for site in entry.cases)
    return frozenset(keys)


def _installed_keys(what) -> frozenset:
    if isinstance(what, ResolvedFingerprint):
        return what.keys()
    if isinstance(what, Registry):
        return what.installed_keys()
    return frozenset(what if isinstance(what, Iterable) else ())


def validate_contract_against_installed(contract: ExecutionContract, registry: Registry, fingerprint) -> None:
    """The contract and the installation must name the same (op, site) keys. A key missing from the contract does
    not mean "whatever the default is": it means the site does not exist."""
    have = _installed_keys(fingerprint)
    want = expected_installed_keys(contract, registry)
    if have == want:
        return
    extra, absent = sorted(have - want), sorted(want - have)
    raise ContractDeliveryError(
        "contract does not match the installed composition:\n"
        f"  installed but UNNAMED by the contract: {extra}\n"
        f"  named by the contract but NOT installed: {absent}\n"
        "Every installed (op, site) carries an explicit entry; absence means 'no such site'."
    )
