"""The obligation ledger: every agreement check reports here, and refusals funnel through ``refuse``.

A reduced form of the reference's enforcement module (isoexec/core/enforce.py:25-62, 252-410): the
phase and result vocabularies, an append-only ledger of (obligation, phase, result, evidence)
records, and the strict / demoted switch. The plan derivation and verdict artifacts of the reference
belong to its trainer/engine installers and are not part of this path.
"""

from __future__ import annotations

import logging
import os
from dataclasses import dataclass
from typing import Dict, List, Tuple

logger = logging.getLogger(__name__)

INSTALL, FIRST_FORWARD, WEIGHT_SYNC, STEP1 = "INSTALL", "FIRST_FORWARD", "WEIGHT_SYNC", "STEP1"
PHASES = (INSTALL, FIRST_FORWARD, WEIGHT_SYNC, STEP1)

BUILD_VALID = "build_valid"
INSTALL_ATTEST = "install_attest"
FINGERPRINT = "fingerprint"
HANDSHAKE = "handshake"

OK, VIOLATION, SKIPPED = "ok", "violation", "skipped"
SKIP_NO_PEER_STAMP = "no-peer-stamp"
SKIP_NO_LOCAL_CONTRACT = "no-local-contract"
RECOGNIZED_SKIPS = (SKIP_NO_PEER_STAMP, SKIP_NO_LOCAL_CONTRACT)


@dataclass(frozen=True)
class Record:
    obligation_id: str
    phase: str
    result: str
    evidence: str = ""


class ObligationLedger:
    def __init__(self) -> None:
        self.records: List[Record] = []

    def report(self, obligation_id: str, phase: str, result: str, evidence: str = "") -> None:
        if phase not in PHASES:
            raise ValueError(f"unknown phase {phase!r}")
        if result not in (OK, VIOLATION, SKIPPED):
            raise ValueError(f"unknown result {result!r}")
        self.records.append(Record(obligation_id, phase, result, evidence))

    def status(self) -> Dict[Tuple[str, str], str]:
        """Worst result per (obligation, phase): a violation is never overwritten by a later ok."""
        rank = {OK: 0, SKIPPED: 1, VIOLATION: 2}
        out: Dict[Tuple[str, str], str] = {}
        for r in self.records:
            key = (r.obligation_id, r.phase)
            if key not in out or rank[r.result] > rank[out[key]]:
                out[key] = r.result
        return out

    def violations(self) -> List[Record]:
        return [r for r in self.records if r.result == VIOLATION]


_LEDGER: ObligationLedger | None = None


def ledger() -> ObligationLedger:
    global _LEDGER
    if _LEDGER is None:
        _LEDGER = ObligationLedger()
    return _LEDGER


def _reset_for_tests() -> None:
    global _LEDGER
    _LEDGER = None
    try:
        from .fingerprint import _ATTESTED

        _ATTESTED.clear()
    except Exception:  # noqa: BLE001
        pass


def report(obligation_id: str, phase: str, result: str, evidence: str = "") -> None:
    """Record one verdict. Fail-safe: a reporting bug never breaks the check it wraps."""
    try:
        ledger().report(obligation_id, phase, result, evidence)
    except Exception as exc:  # noqa: BLE001
        logger.warning("[ISOEXEC-ENFORCE] report(%s, %s, %s) skipped: %s", obligation_id, phase, result, exc)


def _strict() -> bool:
    return os.environ.get("SKYRL_ISOEXEC_MANIFEST_STRICT", "1").lower() not in ("", "0", "false", "no")


def debug_demoted() -> bool:
    return bool(os.environ.get("SKYRL_ISOEXEC_DEBUG_TRACE"))


def demoted() -> bool:
    """True when a refusal logs and continues instead of raising."""
    return not _strict() or debug_demoted()


def refuse(msg: str) -> bool:
    """Raise ``msg`` as the refusal, or log it and return False when demoted. The ledger entry that
    preceded the call stays red either way."""
    if demoted():
        logger.error("%s (demoted: violation recorded, run continues)", msg)
        return False
    raise RuntimeError(msg)
