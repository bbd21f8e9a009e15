"""The per-process contract: built once from the registry and the model's selections, then compared.

Reference: isoexec/core/process_contract.py:17-226. Both runtimes build the same contract at start-up;
``assert_contract_agreement`` turns a disagreement into a refusal to run.
"""

from __future__ import annotations

import hashlib
import json
import logging
import os
import struct

logger = logging.getLogger(__name__)

_CONTRACT = None
_VIEW = None
# Named components outside the model registry that must also agree across the pair. With none
# registered the handshake hash is the numerical_policy identity itself.
_EXTENSIONS: dict = {}


def register_contract_extension(name: str, digest_fn) -> None:
    """Fold ``digest_fn() -> str`` into the handshake hash; it is evaluated at every hash read."""
    _EXTENSIONS[name] = digest_fn


def composite_hash(base):
    if base is None or not _EXTENSIONS:
        return base
    folded = {}
    for name in sorted(_EXTENSIONS):
        try:
            folded[name] = str(_EXTENSIONS[name]())
        except Exception as exc:  # noqa: BLE001 -- a broken extension must not fake agreement
            folded[name] = f"EXTENSION-ERROR:{type(exc).__name__}"
    text = json.dumps({"base": base, "extensions": folded}, sort_keys=True, separators=(",", ":"))
    return hashlib.sha256(text.encode("utf-8")).hexdigest()


def _plain_constant(value):
    # Floats travel as fp64 bit patterns; the fingerprint compares plain values.
    from ..contract import BitPattern

    if isinstance(value, BitPattern) and value.dtype == "fp64":
        return struct.unpack("<d", struct.pack("<Q", int(value.bits, 16)))[0]
    return value


def build_contract_view(contract, registry) -> dict:
    """``{(op, site): {impl_id, version, pinned_constants, half}}`` for the fingerprint comparison."""
    from .contract_delivery import primary_op

    view = {}
    for entry in contract.composition:
        op = primary_op(registry, entry)
        row = {
            "impl_id": entry.impl.id,
            "version": entry.impl.version,
            "pinned_constants": {k: _plain_constant(v) for k, v in entry.constants},
            "half": entry.half,
        }
        for case in entry.cases:
            view[(op, case)] = dict(row)
    return view


def get_process_contract(model_path=None, *, arch=None):
    """Build (once) and return this process's contract; None when none exists and no model is named.
    With ``ISOEXEC_CONTRACT_PATH`` set, the first build also writes the canonical artifact there."""
    global _CONTRACT, _VIEW
    if _CONTRACT is not None:
        return _CONTRACT
    if not model_path:
        return None
    from .. import models
    from . import enforce
    from .registry_build import build_registry

    registry = build_registry(strict=False)
    try:
        contract = models.build_for(model_path, registry, arch=arch)
    except Exception as exc:
        enforce.report(f"{enforce.BUILD_VALID}:contract", enforce.INSTALL, enforce.VIOLATION, f"{type(exc).__name__}: {exc}")
        raise
    _CONTRACT, _VIEW = contract, build_contract_view(contract, registry)
    ids = contract.identities
    enforce.report(f"{enforce.BUILD_VALID}:contract", enforce.INSTALL, enforce.OK, f"numerical_policy={ids.numerical_policy}")
    logger.info(
        "[ISOEXEC-CONTRACT] model=%s arch=%s numerical_policy=%s semantic=%s deployment=%s entries=%d",
        contract.model.family, contract.composition[0].impl.arch, ids.numerical_policy, ids.semantic,
        ids.deployment, len(contract.composition),
    )
    path = os.environ.get("ISOEXEC_CONTRACT_PATH")
    if path:
        try:
            from .contract_delivery import write_contract_file

            write_contract_file(contract, path)
        except Exception as exc:  # noqa: BLE001 -- the artifact is best-effort
            logger.warning("[ISOEXEC-CONTRACT] artifact write to %s skipped: %s", path, exc)
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
    """The handshake hash: numerical_policy folded with the registered extensions."""
    contract = get_process_contract(model_path)
    return None if contract is None else composite_hash(contract.identities.numerical_policy)


def assert_contract_agreement(other_hash: str, *, other_side: str = "peer") -> bool:
    """The peer's handshake hash must equal ours. A mismatch is recorded and refuses unless demoted."""
    from . import enforce

    oid = f"{enforce.HANDSHAKE}:numerical_policy"
    ours = contract_hash()
    if ours is None:
        enforce.report(oid, enforce.WEIGHT_SYNC, enforce.SKIPPED, f"{enforce.SKIP_NO_LOCAL_CONTRACT}: local contract not built")
        return True
    if other_hash == ours:
        enforce.report(oid, enforce.WEIGHT_SYNC, enforce.OK, f"MATCH hash={ours} ({other_side})")
        return True
    msg = (
        f"[ISOEXEC-CONTRACT-HANDSHAKE] MISMATCH: local={ours} {other_side}={other_hash}. The two runtimes "
        "resolved different numerical policies; running on would compare outputs of different functions."
    )
    enforce.report(oid, enforce.WEIGHT_SYNC, enforce.VIOLATION, msg)
    return enforce.refuse(msg)


def assert_init_info_contract(init_info, *, other_side: str = "trainer") -> bool:
    """Receiver side: compare against the hash a peer stamped on ``init_info.contract_hash``."""
    from . import enforce

    oid = f"{enforce.HANDSHAKE}:numerical_policy"
    stamped = getattr(init_info, "contract_hash", None)
    if stamped is None:
        enforce.report(oid, enforce.WEIGHT_SYNC, enforce.SKIPPED, f"{enforce.SKIP_NO_PEER_STAMP}: {other_side} stamped no contract_hash")
        return True
    if contract_hash() is None:
        enforce.report(oid, enforce.WEIGHT_SYNC, enforce.SKIPPED, f"{enforce.SKIP_NO_LOCAL_CONTRACT}: local contract not built")
        return True
    return assert_contract_agreement(stamped, other_side=other_side)
