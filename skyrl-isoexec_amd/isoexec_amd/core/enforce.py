"""The ledger of obligations. Every agreement check in this package files its verdict here, and every refusal to
run goes through ``refuse``, so that one switch decides whether a violation stops the process or is only recorded.

This is the part of the reference's enforcement module that the contract path needs (isoexec/core/enforce.py:25-62,
252-410): the vocabularies of phases and results, an append-only list of (obligation, phase, result, evidence), and
the strict/demoted switch. Its plan derivation and verdict files serve the reference's installers and are not here.
"""

from __future__ import annotations

import logging
import os
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

logger = logging.getLogger(__name__)

# when a verdict is filed
INSTALL = "INSTALL"
FIRST_FORWARD = "FIRST_FORWARD"
WEIGHT_SYNC = "WEIGHT_SYNC"
STEP1 = "STEP1"
PHASES = (INSTALL, FIRST_FORWARD, WEIGHT_SYNC, STEP1)

# what the verdict is about (prefix of an obligation id)
BUILD_VALID, INSTALL_ATTEST, FINGERPRINT, HANDSHAKE = "build_valid", "install_attest", "fingerprint", "handshake"

# the verdict, least to most severe
OK, SKIPPED, VIOLATION = "ok", "skipped", "violation"
_SEVERITY = {OK: 0, SKIPPED: 1, VIOLATION: 2}
# the reasons a check may be skipped for
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
    """Append-only."""

    def __init__(self) -> None:
        self.records: List[Record] = []

    def report(self, obligation_id: str, phase: str, result: str, evidence: str = "") -> None:
        for what, value, allowed in (("phase", phase, PHASES), ("result", result, _SEVERITY)):
            if value not in allowed:
                raise ValueError(f"unknown {what} {value!r}")
        self.records.append(Record(obligation_id, phase, result, evidence))

    def status(self) -> Dict[Tuple[str, str], str]:
        """The most severe result filed for each (obligation, phase): a later ``ok`` never hides a violation."""
        worst: Dict[Tuple[str, str], str] = {}
        for record in self.records:
            slot = (record.obligation_id, record.phase)
            if _SEVERITY[record.result] > _SEVERITY.get(worst.get(slot), -1):
                worst[slot] = record.result
        return worst

    def violations(self) -> List[Record]:
        return [record for record in self.records if record.result == VIOLATION]


_LEDGER: Optional[ObligationLedger] = None


def ledger() -> ObligationLedger:
    global _LEDGER
    if _LEDGER is None:
        _LEDGER = ObligationLedger()
    return _LEDGER


def _reset_for_tests() -> None:
    global _LEDGER
    _LEDGER = None
    try:
        from . import fingerprint

        fingerprint._ATTESTED.clear()
    except Exception:  # noqa: BLE001
        pass


def report(obligation_id: str, phase: str, result: str, evidence: str = "") -> None:
    """File one verdict. A bug in filing must not break the check that files, so nothing escapes from here."""
    try:
        ledger().report(obligation_id, phase, result, evidence)
    except Exception as exc:  # noqa: BLE001
        logger.warning("[ISOEXEC-ENFORCE] report(%s, %s, %s) skipped: %s", obligation_id, phase, result, exc)


def _flag(name: str, default: str) -> bool:
    return os.environ.get(name, default).lower() not in ("", "0", "false", "no")


def _strict() -> bool:
    return _flag("SKYRL_ISOEXEC_MANIFEST_STRICT", "1")


def debug_demoted() -> bool:
    return bool(os.environ.get("SKYRL_ISOEXEC_DEBUG_TRACE"))


def demoted() -> bool:
    """When True a refusal is logged and the run goes on."""
    return debug_demoted() or not _strict()


def refuse(msg: str) -> bool:
    """Stop the run with ``msg`` -- or, when demoted, log it and return False. Either way the violation that was
    filed before calling this stays in the ledger."""
    if not demoted():
        raise RuntimeError(msg)
    logger.error("%s (demoted: violation recorded, run continues)", msg)
    return False
