"""What was actually installed at each (op, site), recorded as it happens and held against the contract.

The places that bind an implementation call ``record_install``; ``log_fingerprint`` lines the records up with the
contract's per-(op, site) view and files one ledger entry per key. Neither recording nor comparing may ever stop a
run by raising. (Reference: isoexec/core/fingerprint.py:18-206.)
"""

from __future__ import annotations

import logging
from dataclasses import dataclass, field
from typing import Dict, Optional, Tuple

logger = logging.getLogger(__name__)

Key = Tuple[str, str]

# site groups, for callers that install at several sites at once
TRAINER_SITES = ("trainer_fwd", "trainer_score")
ENGINE_SITES = ("engine_prefill", "engine_decode")
ALL_SITES = TRAINER_SITES + ENGINE_SITES
SCORE_ONLY, PREFILL_ONLY, DECODE_ONLY = ("trainer_score",), ("engine_prefill",), ("engine_decode",)

# An install that was asked for and did not happen is recorded under this id: visible, not silent.
NOT_INSTALLED = "NOT_INSTALLED"


def _origin(obj) -> Tuple[Optional[str], Optional[str]]:
    """(module, qualified name) of the object that was bound, for the log."""
    if obj is None:
        return None, None
    kind = type(obj)
    return (getattr(obj, "__module__", None) or kind.__module__, getattr(obj, "__qualname__", None) or kind.__qualname__)


@dataclass
class ResolvedFingerprint:
    """A snapshot of the records."""

    installed: Dict[Key, dict] = field(default_factory=dict)

    def keys(self) -> frozenset:
        return frozenset(self.installed)


class FingerprintRecorder:
    """The records of one process: the latest install per (op, site)."""

    def __init__(self) -> None:
        self.installed: Dict[Key, dict] = {}

    def record(self, op: str, site: str, impl_id: str, obj=None, pinned=None) -> None:
        module, qualname = _origin(obj)
        entry = {"impl_id": impl_id, "module": module, "qualname": qualname}
        if pinned is not None:
            entry["pinned_constants"] = dict(pinned)
        self.installed[(op, site)] = entry

    def resolved(self) -> ResolvedFingerprint:
        return ResolvedFingerprint(installed=dict(self.installed))


_RECORDER: Optional[FingerprintRecorder] = None
_ATTESTED: set = set()      # installs already reported to the ledger (an install site may run every forward)
_LOGGED_TAGS: set = set()   # tags log_fingerprint_once has served


def recorder() -> FingerprintRecorder:
    global _RECORDER
    if _RECORDER is None:
        _RECORDER = FingerprintRecorder()
    return _RECORDER


def _reset_for_tests() -> None:
    global _RECORDER
    _RECORDER = None
    _ATTESTED.clear()
    _LOGGED_TAGS.clear()


def record_install(op: str, site: str, impl_id: str, obj=None, pinned=None) -> None:
    """Note that ``impl_id`` now serves (op, site); the first such note is also attested in the ledger."""
    try:
        recorder().record(op, site, impl_id, obj, pinned)
        pins = repr(sorted(pinned.items())) if isinstance(pinned, dict) else repr(pinned)
        seen_before = (op, site, impl_id, pins) in _ATTESTED
        _ATTESTED.add((op, site, impl_id, pins))
        if not seen_before:
            from . import enforce

            enforce.report(f"{enforce.INSTALL_ATTEST}:{op}:{site}", enforce.INSTALL, enforce.OK, impl_id)
    except Exception as exc:  # noqa: BLE001
        logger.warning("[ISOEXEC-FINGERPRINT] record_install(%s,%s) skipped: %s", op, site, exc)


def record_installs(op: str, sites, impl_id: str, obj=None, pinned=None) -> None:
    if isinstance(sites, str):
        sites = (sites,)
    for site in sites:
        record_install(op, site, impl_id, obj, pinned)


def pin_disagreements(want_pins, got_pins) -> list:
    """Where the recorded pins depart from the contract's, one line per key. Only keys the contract pins count, and
    values are compared the registry's way (a list equals the same tuple, True does not equal 1)."""
    from .registry import pin_values_equal

    want, got = dict(want_pins or {}), dict(got_pins or {})
    lines = []
    for key in sorted(want, key=str):
        pinned = want[key]
        if key not in got:
            lines.append(f"{key}: contract pins {pinned!r}, install recorded nothing")
        elif not pin_values_equal(pinned, got[key]):
            lines.append(f"{key}: contract pins {pinned!r}, install used {got[key]!r}")
    return lines


def missing_from_fingerprint(view) -> list:
    """Keys of the contract that nothing was recorded for. Not a fault by itself: a trainer records nothing for
    the engine's sites and the other way round."""
    recorded = recorder().installed
    return sorted(key for key in (view or {}) if key not in recorded)


def _objection(key, got, want) -> Optional[str]:
    """What is wrong with one recorded install given the contract's row for its key (None: nothing)."""
    if want is None:
        return f"{key} installed as {got['impl_id']!r} but the contract names no such (op,site)"
    bound = f"({got['module']}.{got['qualname']})"
    if got["impl_id"] != want["impl_id"]:
        return f"{key}: contract={want['impl_id']!r} but INSTALLED={got['impl_id']!r} {bound}"
    if "pinned_constants" not in got:
        return None  # an install that reports no pins is a blind spot; it is not a disagreement
    lines = pin_disagreements(want.get("pinned_constants"), got["pinned_constants"])
    if not lines:
        return None
    return (f"{key}: contract pins={want.get('pinned_constants')!r} but INSTALLED pins={got['pinned_constants']!r} -- "
            f"{'; '.join(lines)} {bound}")


def log_fingerprint(view=None, tag: str = "default") -> list:
    """Log the records; with ``view`` (the contract as ``{(op, site): {impl_id, pinned_constants, ...}}``) also
    return every objection, an empty list meaning the installation is the contract's."""
    from . import enforce

    recorded = recorder().installed
    logger.info("[ISOEXEC-FINGERPRINT] (%s) recorded %d instrumented install(s)", tag, len(recorded))
    if view is None:
        return []
    phase = enforce.FIRST_FORWARD if "first_forward" in tag else enforce.INSTALL
    objections = []
    for key in sorted(recorded):
        got = recorded[key]
        obligation = f"{enforce.FINGERPRINT}:{key[0]}:{key[1]}"
        complaint = _objection(key, got, view.get(key))
        if complaint is None:
            enforce.report(obligation, phase, enforce.OK, f"({tag}) {got['impl_id']}")
            continue
        objections.append(complaint)
        enforce.report(obligation, phase, enforce.VIOLATION, complaint)
        logger.error("[ISOEXEC-FINGERPRINT] MISMATCH %s", complaint)
    return objections


def log_fingerprint_once(view=None, tag: str = "default") -> list:
    """``log_fingerprint`` the first time a tag is seen, nothing afterwards; never raises."""
    if tag in _LOGGED_TAGS:
        return []
    _LOGGED_TAGS.add(tag)
    try:
        return log_fingerprint(view, tag=tag)
    except Exception as exc:  # noqa: BLE001
        logger.warning("[ISOEXEC-FINGERPRINT] log_fingerprint_once(%s) skipped: %s", tag, exc)
        return []
