"""This process's contract: derived once from the registry and the model declaration, kept for the life of the
process, and compared with the peer's by hash (a disagreement is a refusal to run).

Reference: isoexec/core/process_contract.py:17-226.
"""

from __future__ import annotations

import hashlib
import json
import logging
import os
import struct

logger = logging.getLogger(__name__)


# What the process holds once the contract exists, and the named digests (name -> callable) of components outside
# the op registry that both sides must also agree on.
_CONTRACT = None
_VIEW = None
_EXTENSIONS: dict = {}


def register_contract_extension(name: str, digest_fn) -> None:
    """Make ``digest_fn()`` part of the handshake hash. It is called every time the hash is read."""
    _EXTENSIONS[name] = digest_fn


def composite_hash(base):
    """``base`` folded with every registered extension's digest (``base`` itself when there are none)."""
    if base is None or not _EXTENSIONS:
        return base
    digests = {}
    for name, fn in sorted(_EXTENSIONS.items()):
        try:
            digests[name] = str(fn())
        except Exception as exc:  # noqa: BLE001 -- a failing extension must never look like agreement
            digests[name] = "EXTENSION-ERROR:" + type(exc).__name__
    blob = json.dumps({"base": base, "extensions": digests}, sort_keys=True, separators=(",", ":")).encode("utf-8")
    return hashlib.sha256(blob).hexdigest()


def _as_plain_value(constant):
    """A contract stores a float as the bit pattern of its fp64; the installed-state comparison wants the number."""
    from ..contract import BitPattern

    if isinstance(constant, BitPattern) and constant.dtype == "fp64":
        (number,) = struct.unpack("<d", struct.pack("<Q", int(constant.bits, 16)))
        return number
    return constant


def build_contract_view(contract, registry) -> dict:
    """The contract flattened to ``{(op, site): {impl_id, version, pinned_constants, half}}``, the shape the
    installed-state fingerprint is compared in."""
    from .contract_delivery import primary_op

    flat = {}
    for entry in contract.composition:
        owner = primary_op(registry, entry)
        constants = {name: _as_plain_value(value) for name, value in entry.constants}
        for site in entry.cases:
            flat[(owner, site)] = {"impl_id": entry.impl.id, "version": entry.impl.version,
                                   "pinned_constants": dict(constants), "half": entry.half}
    return flat


def _publish(contract) -> None:
    """Write the artifact where ``ISOEXEC_CONTRACT_PATH`` says, if it says anything; failure is logged, not fatal."""
    where = os.environ.get("ISOEXEC_CONTRACT_PATH")
    if not where:
        return
    try:
        from .contract_delivery import write_contract_file

        write_contract_file(contract, where)
    except Exception as exc:  # noqa: BLE001
        logger.warning("[ISOEXEC-CONTRACT] artifact write to %s skipped: %s", where, exc)


def get_process_contract(model_path=None, *, arch=None):
    """The process's contract, building it on the first call that names a model (None before that)."""
    global _CONTRACT, _VIEW
    if _CONTRACT is not None or not model_path:
        return _CONTRACT
    from .. import models
    from . import enforce
    from .registry_build import build_registry

    obligation = f"{enforce.BUILD_VALID}:contract"
    registry = build_registry(strict=False)
    try:
        contract = models.build_for(model_path, registry, arch=arch)
    except Exception as exc:
        enforce.report(obligation, enforce.INSTALL, enforce.VIOLATION, f"{type(exc).__name__}: {exc}")
        raise
    _CONTRACT, _VIEW = contract, build_contract_view(contract, registry)
    ids = contract.identities
    enforce.report(obligation, enforce.INSTALL, enforce.OK, f"numerical_policy={ids.numerical_policy}")
    logger.info("[ISOEXEC-CONTRACT] model=%s arch=%s numerical_policy=%s semantic=%s deployment=%s entries=%d",
                contract.model.family, contract.composition[0].impl.arch, ids.numerical_policy, ids.semantic,
                ids.deployment, len(contract.composition))
    _publish(contract)
    return contract


def cached_contract():
    return _CONTRACT


def cached_contract_view():
    return _VIEW


def _reset_for_tests() -> None:
    global _CONTRACT, _VIEW
    _CONTRACT = _VIEW = None
    _EXTENSIONS.clear()


def contract_hash(model_path=None):
    """What the two sides exchange: the numerical-policy identity folded with the extensions."""
    contract = get_process_contract(model_path)
    if contract is None:
        return None
    return composite_hash(contract.identities.numerical_policy)


def assert_contract_agreement(other_hash: str, *, other_side: str = "peer") -> bool:
    """Compare the peer's hash with ours. Equal: recorded as met. Different: recorded as a violation and refused
    (unless enforcement is demoted). No local contract yet: recorded as skipped."""
    from . import enforce

    obligation = f"{enforce.HANDSHAKE}:numerical_policy"
    mine = contract_hash()
    if mine is None:
        enforce.report(obligation, enforce.WEIGHT_SYNC, enforce.SKIPPED,
                       f"{enforce.SKIP_NO_LOCAL_CONTRACT}: local contract not built")
        return True
    if mine == other_hash:
        enforce.report(obligation, enforce.WEIGHT_SYNC, enforce.OK, f"MATCH hash={mine} ({other_side})")
        return True
    complaint = (f"[ISOEXEC-CONTRACT-HANDSHAKE] MISMATCH: local={mine} {other_side}={other_hash}. The two runtimes "
                 "resolved different numerical policies; carrying on would compare the outputs of two functions.")
    enforce.report(obligation, enforce.WEIGHT_SYNC, enforce.VIOLATION, complaint)
    return enforce.refuse(complaint)


def assert_init_info_contract(init_info, *, other_side: str = "trainer") -> bool:
    """The receiving side of the handshake: the peer's hash arrives as ``init_info.contract_hash``."""
    from . import enforce

    obligation = f"{enforce.HANDSHAKE}:numerical_policy"
    theirs = getattr(init_info, "contract_hash", None)
    if theirs is None:
        reason = f"{enforce.SKIP_NO_PEER_STAMP}: {other_side} stamped no contract_hash"
    elif contract_hash() is None:
        reason = f"{enforce.SKIP_NO_LOCAL_CONTRACT}: local contract not built"
    else:
        return assert_contract_agreement(theirs, other_side=other_side)
    enforce.report(obligation, enforce.WEIGHT_SYNC, enforce.SKIPPED, reason)
    return True
