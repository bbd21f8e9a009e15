"""The install fingerprint: what was actually bound per (op, site), compared against the contract.

Reference: isoexec/core/fingerprint.py:18-206. Install sites call ``record_install`` as they bind;
``log_fingerprint`` compares the records with the contract's per-(op, site) view and reports each key
to the obligation ledger. Recording and comparing never raise.
"""

from __future__ import annotations

import logging
from dataclasses import dataclass, field
from typing import Dict, Tuple

logger = logging.getLogger(__name__)

Key = Tuple[str, str]

TRAINER_SITES = ("trainer_fwd", "trainer_score")
ENGINE_SITES = ("engine_prefill", "engine_decode")
ALL_SITES = TRAINER_SITES + ENGINE_SITES
SCORE_ONLY = ("trainer_score",)
PREFILL_ONLY = ("engine_prefill",)
DECODE_ONLY = ("engine_decode",)

# Recorded when a requested install did not happen, so the skip is visible rather than silent.
NOT_INSTALLED = "NOT_INSTALLED"


@dataclass
class ResolvedFingerprint:
    installed: Dict[Key, dict] = field(default_factory=dict)

    def keys(self) -> frozenset:
        return frozenset(self.installed)


class FingerprintRecorder:
    def __init__(self) -> None:
        self.installed: Dict[Key, dict] = {}

    def record(self, op: str, site: str, impl_id: str, obj=None, pinned=None) -> None:
        where = (None, None)
        if obj is not None:
            where = (
                getattr(obj, "__module__", None) or type(obj).__module__,
                getattr(obj, "__qualname__", None) or type(obj).__qualname__,
            )
        row = {"impl_id": impl_id, "module": where[0], "qualname": where[1]}
        if pinned is not None:
            row["pinned_constants"] = dict(pinned)
        self.installed[(op, site)] = row

    def resolved(self) -> ResolvedFingerprint:
        return ResolvedFingerprint(dict(self.installed))


_RECORDER: FingerprintRecorder | None = None
_LOGGED_TAGS: set = set()
_ATTESTED: set = set()


def recorder() -> FingerprintRecorder:
    global _RECORDER
    if _RECORDER is None:
        _RECORDER = FingerprintRecorder()
    return _RECORDER


def _reset_for_tests() -> None:
    global _RECORDER
    _RECORDER = None
    _LOGGED_TAGS.clear()
    _ATTESTED.clear()


def record_install(op: str, site: str, impl_id: str, obj=None, pinned=None) -> None:
    try:
        recorder().record(op, site, impl_id, obj, pinned)
        mark = (op, site, impl_id, repr(sorted(pinned.items())) if isinstance(pinned, dict) else repr(pinned))
        if mark in _ATTESTED:  # per-forward recorders would otherwise re-report forever
            return
        _ATTESTED.add(mark)
        from . import enforce

        enforce.report(f"{enforce.INSTALL_ATTEST}:{op}:{site}", enforce.INSTALL, enforce.OK, impl_id)
    except Exception as exc:  # noqa: BLE001
        logger.warning("[ISOEXEC-FINGERPRINT] record_install(%s,%s) skipped: %s", op, site, exc)


def record_installs(op: str, sites, impl_id: str, obj=None, pinned=None) -> None:
    for site in (sites,) if isinstance(sites, str) else sites:
        record_install(op, site, impl_id, obj, pinned)


def pin_disagreements(want_pins, got_pins) -> list:
    """Per-key differences between the contract's pins and the recorded ones. Only keys the contract
    pins are compared, with the registry's JSON-tolerant, bool-strict equality."""
    from .registry import pin_values_equal

    want, got = dict(want_pins or {}), dict(got_pins or {})
    out = []
    for key in sorted(want, key=str):
        if key not in got:
            out.append(f"{key}: contract pins {want[key]!r}, install recorded nothing")
        elif not pin_values_equal(want[key], got[key]):
            out.append(f"{key}: contract pins {want[key]!r}, install used {got[key]!r}")
    return out


def missing_from_fingerprint(view) -> list:
    """Contract keys nothing recorded. Informational: the other runtime's sites are unrecorded here."""
    seen = recorder().installed
    return sorted(k for k in (view or {}) if k not in seen)


def _judge(key, got, want):
    if want is None:
        return f"{key} installed as {got['impl_id']!r} but the contract names no such (op,site)"
    if want["impl_id"] != got["impl_id"]:
        return f"{key}: contract={want['impl_id']!r} but INSTALLED={got['impl_id']!r} ({got['module']}.{got['qualname']})"
    if "pinned_constants" in got:  # reporting no pins is a blind spot, not agreement
        diffs = pin_disagreements(want.get("pinned_constants"), got["pinned_constants"])
        if diffs:
            return (
                f"{key}: contract pins={want.get('pinned_constants')!r} but INSTALLED pins="
                f"{got['pinned_constants']!r} -- {'; '.join(diffs)} ({got['module']}.{got['qualname']})"
            )
    return None


def log_fingerprint(view=None, tag: str = "default") -> list:
    """Log what was recorded and return its disagreements with ``view`` (the contract's
    ``{(op, site): {impl_id, pinned_constants, ...}}`` projection); empty means they match."""
    from . import enforce

    seen = recorder().installed
    logger.info("[ISOEXEC-FINGERPRINT] (%s) recorded %d instrumented install(s)", tag, len(seen))
    if view is None:
        return []
    phase = enforce.FIRST_FORWARD if "first_forward" in tag else enforce.INSTALL
    problems = []
    for key, got in sorted(seen.items()):
        verdict = _judge(key, got, view.get(key))
        oid = f"{enforce.FINGERPRINT}:{key[0]}:{key[1]}"
        if verdict is None:
            enforce.report(oid, phase, enforce.OK, f"({tag}) {got['impl_id']}")
        else:
            problems.append(verdict)
            enforce.report(oid, phase, enforce.VIOLATION, verdict)
            logger.error("[ISOEXEC-FINGERPRINT] MISMATCH %s", verdict)
    return problems


def log_fingerprint_once(view=None, tag: str = "default") -> list:
    if tag in _LOGGED_TAGS:
        return []
    _LOGGED_TAGS.add(tag)
    try:
        return log_fingerprint(view, tag=tag)
    except Exception as exc:  # noqa: BLE001
        logger.warning("[ISOEXEC-FINGERPRINT] log_fingerprint_once(%s) skipped: %s", tag, exc)
        return []
