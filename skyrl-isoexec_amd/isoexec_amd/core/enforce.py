"""The ledger of obligations. Every agreement check in this package files its verdict here, every refusal to run goes
through ``refuse`` (so that one switch decides whether a violation stops the process or is only recorded), and at each
phase boundary the ledger is held against the PLAN of checks the contract itself implies: a required check that left no
record is a violation like a failed one.

The plan is derived, never listed by hand (reference: isoexec/core/enforce.py:215-249): per composition entry visible on
a side one install attestation and one fingerprint comparison (and a served-count check where the implementation keeps a
counter), per claim its check, plus the contract's own build, the installed-keys backstop and the handshake. One table
says when each kind is due and whether an unmet one refuses or is logged (enforce.py:67-77); an obligation of a
deployment-half entry only ever logs; a skip discharges a refusing obligation only when it names a structural reason
(enforce.py:50-56, 316-326). ``close_phase`` is the boundary (enforce.py:427-487). The verdict is a dictionary
(enforce.py:531-574); this package writes no verdict files and merges none across processes.
"""

from __future__ import annotations

import fnmatch
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
SERVED, DOMAIN_CHECK, HOOK_EXISTS, GATE = "served", "domain_check", "hook_exists", "gate"
INSTALLED_BACKSTOP = "installed_backstop"

# the verdict, least to most severe
OK, SKIPPED, VIOLATION = "ok", "skipped", "violation"
# two more that only a phase boundary can pronounce, never a reporter: no record at all, and nothing but skips that
# name no structural reason
MISSING, UNCHECKED = "missing", "unchecked"
# what an unmet obligation does at its boundary
REFUSE, LOG = "refuse", "log"
# evidence prefix of a checker that raised: filed as a violation, so a broken checker fails closed
CHECKER_ERROR = "CHECKER-ERROR"

SIDES = {"trainer": ("trainer_fwd", "trainer_score"), "engine": ("engine_prefill", "engine_decode")}

# kind -> (the phase it is due at, what an unmet one does)
_DUE = {
    BUILD_VALID: (INSTALL, REFUSE),
    INSTALL_ATTEST: (INSTALL, REFUSE),
    DOMAIN_CHECK: (INSTALL, REFUSE),
    HOOK_EXISTS: (INSTALL, REFUSE),
    FINGERPRINT: (FIRST_FORWARD, REFUSE),
    INSTALLED_BACKSTOP: (FIRST_FORWARD, REFUSE),
    HANDSHAKE: (WEIGHT_SYNC, REFUSE),
    SERVED: (STEP1, LOG),
    GATE: (STEP1, REFUSE),
}
SEVERITY = {(kind, phase): action for kind, (phase, action) in _DUE.items()}

# (op, impl) pairs that keep a live count of the calls they served; only these owe a served-count check.
SERVED_COUNTERS = {
    ("logprobs.log_softmax", "hip_rowinv_leaftree"): "ops/logprobs/rowinv.py::stats()['served']",
    ("gdn.state", "hip_private_pool"): "ops/gdn/gdn_cpr_rows.py served/declined counters of the slot->row resolver",
}
# Of those, the ones whose one-sided absence would leave two different functions behind one matching hash: the
# log-softmax path can decline and hand a call to the incumbent, on one side only. Their served check refuses.
SERVED_REFUSE_IMPLS = {
    ("logprobs.log_softmax", "hip_rowinv_leaftree"): "a decline hands the call to the incumbent on that side only",
}
assert set(SERVED_REFUSE_IMPLS) <= set(SERVED_COUNTERS)
_SEVERITY = {OK: 0, SKIPPED: 1, VIOLATION: 2}
# the reasons a check may be skipped for
SKIP_NO_PEER_STAMP = "no-peer-stamp"
SKIP_NO_LOCAL_CONTRACT = "no-local-contract"
RECOGNIZED_SKIPS = (SKIP_NO_PEER_STAMP, SKIP_NO_LOCAL_CONTRACT)


@dataclass(frozen=True)
class Exemption:
    """A deliberate softness: obligations whose id matches ``pattern`` (fnmatch) never refuse and are counted as
    excepted. Each owes the reason and what would let it be removed."""

    pattern: str
    reason: str
    removal: str


EXCEPTIONS: Tuple[Exemption, ...] = (
    # RecurrentGDN / CprGDN pools are allocated by the engine when it is constructed with its batch limits, which a
    # deployment may do after the install boundary; the fingerprint comparison at the first forward still refuses.
    Exemption("install_attest:gdn.state:*",
              "the engine allocates its state pools when it learns its batch limits, which may follow the install boundary",
              "record the pool's install from the engine's constructor before the boundary is closed"),
)


def exemption_for(obligation_id: str) -> Optional[Exemption]:
    for exemption in EXCEPTIONS:
        if fnmatch.fnmatchcase(obligation_id, exemption.pattern):
            return exemption
    return None


@dataclass(frozen=True)
class Obligation:
    obligation_id: str
    kind: str
    phase: str
    half: str = "function"
    escalated: bool = False      # a served check that refuses (SERVED_REFUSE_IMPLS); set by the plan only


@dataclass(frozen=True)
class ObligationPlan:
    side: str
    obligations: Tuple[Obligation, ...]
    no_served_counter: Tuple[Tuple[str, str, str], ...]   # (op, site, impl) that keep no count and so owe no check

    def ids(self) -> frozenset:
        return frozenset(ob.obligation_id for ob in self.obligations)


def severity(ob: Obligation) -> str:
    """Deployment-half entries only log; an escalation can strengthen the table's answer, nothing weakens it."""
    if ob.half == "deployment":
        return LOG
    return REFUSE if ob.escalated else _DUE[ob.kind][1]


def _owed(kind: str, subject: str, half: str = "function", escalated: bool = False) -> Obligation:
    return Obligation(f"{kind}:{subject}", kind, _DUE[kind][0], half, escalated)


def derive_obligation_plan(contract, registry, side: str) -> ObligationPlan:
    """Everything a process of ``side`` owes under ``contract``, in a fixed order."""
    from .contract_delivery import primary_op

    if side not in SIDES:
        raise ValueError(f"unknown side {side!r}; expected one of {sorted(SIDES)}")
    owed = [_owed(BUILD_VALID, "contract"), _owed(INSTALLED_BACKSTOP, "first_forward"),
            _owed(HANDSHAKE, "numerical_policy")]
    countless = []
    for entry in contract.composition:
        op = primary_op(registry, entry)
        for site in entry.cases:
            if site not in SIDES[side]:
                continue
            owed.append(_owed(INSTALL_ATTEST, f"{op}:{site}", entry.half))
            owed.append(_owed(FINGERPRINT, f"{op}:{site}", entry.half))
            who = (op, entry.impl.id)
            if who in SERVED_COUNTERS:
                owed.append(_owed(SERVED, f"{op}:{site}", entry.half, escalated=who in SERVED_REFUSE_IMPLS))
            else:
                countless.append((op, site, entry.impl.id))
    owed.extend(_owed(DOMAIN_CHECK, claim.axis) for claim in contract.claims.topology)
    owed.extend(_owed(HOOK_EXISTS, claim.state_id) for claim in contract.claims.state)
    owed.extend(_owed(GATE, "|".join(claim.case_pair)) for claim in contract.claims.tolerances)
    owed.sort(key=lambda ob: (PHASES.index(ob.phase), ob.kind, ob.obligation_id))
    return ObligationPlan(side, tuple(owed), tuple(sorted(countless)))


@dataclass(frozen=True)
class Record:
    obligation_id: str
    phase: str
    result: str
    evidence: str = ""


def skip_recognized(evidence: str) -> bool:
    """Does a skip's evidence ("<reason>: <detail>") name one of the structural reasons?"""
    return str(evidence).split(":", 1)[0].strip() in RECOGNIZED_SKIPS


def _summarise(records) -> str:
    results = [record.result for record in records]
    if not results:
        return MISSING
    if VIOLATION in results:
        return VIOLATION
    return SKIPPED if all(result == SKIPPED for result in results) else OK


class ObligationLedger:
    """Append-only list of verdicts, plus the plans armed in this process and the boundaries already closed."""

    def __init__(self) -> None:
        self.records: List[Record] = []
        self.plans: Dict[str, ObligationPlan] = {}
        self.closed: set = set()                # {(side, phase)}
        self.reopened: List[Record] = []        # verdicts filed for a phase after its boundary was closed
        self.internal_errors: List[str] = []    # what went wrong inside a boundary itself

    def report(self, obligation_id: str, phase: str, result: str, evidence: str = "") -> None:
        for what, value, allowed in (("phase", phase, PHASES), ("result", result, _SEVERITY)):
            if value not in allowed:
                raise ValueError(f"unknown {what} {value!r}")
        record = Record(obligation_id, phase, result, str(evidence))
        self.records.append(record)
        # late for the side that owes it (one ledger may serve both sides of a colocated process); an obligation no
        # armed plan names counts as late for any closed boundary of its phase
        owing = {side for side, plan in self.plans.items() if obligation_id in plan.ids()}
        if any(p == phase and (not owing or side in owing) for side, p in self.closed):
            self.reopened.append(record)

    def by_id(self, obligation_id: str) -> List[Record]:
        return [record for record in self.records if record.obligation_id == obligation_id]

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

    def status_of(self, ob: Obligation) -> str:
        return _summarise(self.by_id(ob.obligation_id))

    def judged_status(self, ob: Obligation) -> str:
        """``status_of``, except that nothing but skips discharges a refusing obligation only if every one of them
        names a structural reason; otherwise the obligation is ``unchecked``."""
        status = self.status_of(ob)
        if status != SKIPPED or severity(ob) != REFUSE:
            return status
        return status if all(skip_recognized(r.evidence) for r in self.by_id(ob.obligation_id)) else UNCHECKED


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


# ---- phase boundaries ------------------------------------------------------------------------------------------
def arm(side: str, contract=None, registry=None) -> Optional[ObligationPlan]:
    """The plan this process owes as ``side``, derived once from the process contract (or from the arguments)."""
    book = ledger()
    if side in book.plans:
        return book.plans[side]
    if contract is None:
        from .process_contract import cached_contract

        contract = cached_contract()
        if contract is None:
            return None
    if registry is None:
        from .registry_build import build_registry

        registry = build_registry(strict=True)
    book.plans[side] = derive_obligation_plan(contract, registry, side)
    return book.plans[side]


def close_phase(phase: str, side: str) -> bool:
    """Hold the ledger against the plan at the end of ``phase``: every obligation due now needs a record, and a
    refusing one needs a clean record. Returns True when nothing refuses; otherwise ``refuse`` decides. A bug in
    here must not stop a run: it is logged, kept in ``internal_errors``, and the boundary passes."""
    unmet: List[str] = []
    try:
        book = ledger()
        plan = arm(side)
        book.closed.add((side, phase))
        if plan is None:
            logger.error("[ISOEXEC-ENFORCE] side=%s phase=%s closed with NO contract built: no plan can be derived "
                         "and nothing was enforced", side, phase)
            return True
        for ob in plan.obligations:
            if ob.phase != phase:
                continue
            status = book.judged_status(ob)
            if status not in (VIOLATION, MISSING, UNCHECKED):
                continue
            exemption = exemption_for(ob.obligation_id)
            if exemption is not None:
                logger.warning("[ISOEXEC-ENFORCE] side=%s %s %s EXCEPTED (%s)", side, ob.obligation_id, status, exemption.reason)
            elif severity(ob) == REFUSE:
                unmet.append(f"{ob.obligation_id} ({status})")
            else:
                logger.error("[ISOEXEC-ENFORCE] side=%s %s %s (severity=log)", side, ob.obligation_id, status)
        counts = verdict_counts()
        logger.warning("[ISOEXEC-ENFORCE] side=%s phase=%s %s", side, phase, " ".join(f"{k}={v}" for k, v in counts.items()))
    except Exception as exc:  # noqa: BLE001
        note = f"close_phase({phase}, {side}) internal error: {type(exc).__name__}: {exc}"
        logger.warning("[ISOEXEC-ENFORCE] %s", note)
        try:
            ledger().internal_errors.append(note)
        except Exception:  # noqa: BLE001
            pass
        return True
    if not unmet:
        return True
    return refuse(f"[ISOEXEC-ENFORCE] side={side} phase={phase} REFUSED: {len(unmet)} required obligation(s) violated or "
                  f"never checked: {'; '.join(unmet)}. The contract derives these obligations; a required check with "
                  "no record is itself a violation. Fix the reporter or the install -- or add an EXCEPTIONS entry "
                  "with its reason.")


def verdict_counts() -> Dict[str, int]:
    """ok / refused / logged / missing / excepted over the obligations of every closed boundary."""
    counts = dict.fromkeys(("ok", "refused", "logged", "missing", "excepted"), 0)
    book = ledger()
    for side, plan in book.plans.items():
        for ob in plan.obligations:
            if (side, ob.phase) not in book.closed:
                continue
            status = book.judged_status(ob)
            if exemption_for(ob.obligation_id) is not None:
                counts["excepted"] += 1
            elif status == OK:
                counts["ok"] += 1
            elif status == MISSING:
                counts["missing"] += 1
            elif status == UNCHECKED or (status == VIOLATION and severity(ob) == REFUSE):
                counts["refused"] += 1
            else:           # a logged violation, or a skip that said why it could not check
                counts["logged"] += 1
    return counts


def verdict() -> dict:
    """Everything the ledger knows, as plain data: one row per planned obligation (``open`` until its boundary is
    closed), one per reported id that no plan derives, late records, internal errors, the exemptions in force."""
    book = ledger()

    def rows_of(records):
        return [{"phase": r.phase, "result": r.result, "evidence": r.evidence} for r in records]

    rows, planned = [], set()
    for side, plan in book.plans.items():
        for ob in plan.obligations:
            planned.add(ob.obligation_id)
            exemption = exemption_for(ob.obligation_id)
            rows.append({"id": ob.obligation_id, "side": side, "kind": ob.kind, "phase": ob.phase, "half": ob.half,
                         "severity": severity(ob),
                         "status": book.judged_status(ob) if (side, ob.phase) in book.closed else "open",
                         "excepted": exemption.pattern if exemption else None,
                         "records": rows_of(book.by_id(ob.obligation_id))})
    for stray in sorted({r.obligation_id for r in book.records} - planned):
        records = book.by_id(stray)
        exemption = exemption_for(stray)
        rows.append({"id": stray, "side": None, "kind": "unplanned", "phase": records[0].phase, "half": None,
                     "severity": "unplanned", "status": _summarise(records),
                     "excepted": exemption.pattern if exemption else None, "records": rows_of(records)})
    return {"pid": os.getpid(), "sides": sorted(book.plans),
            "phases_closed": sorted(f"{side}:{phase}" for side, phase in book.closed),
            "counts": verdict_counts(), "obligations": rows, "reopened": rows_of(book.reopened),
            "internal_errors": list(book.internal_errors),
            "no_served_counter": [list(t) for side in sorted(book.plans) for t in book.plans[side].no_served_counter],
            "exceptions": [{"pattern": e.pattern, "reason": e.reason, "removal": e.removal} for e in EXCEPTIONS]}


# ---- reporters for the claims ----------------------------------------------------------------------------------
def checked(obligation_id: str, phase: str, check) -> bool:
    """Run ``check() -> (ok, evidence)`` and file its verdict; a check that raises is a violation (fail closed)."""
    try:
        ok, evidence = check()
    except Exception as exc:  # noqa: BLE001
        report(obligation_id, phase, VIOLATION, f"{CHECKER_ERROR}: {type(exc).__name__}: {exc}")
        return False
    report(obligation_id, phase, OK if ok else VIOLATION, evidence)
    return bool(ok)


def report_topology(contract, degrees: Dict[str, int]) -> bool:
    """domain_check: the degree this deployment runs each claimed axis at is the pinned one, or inside the domain
    the axis was proved invariant over. An axis the deployment does not name runs at degree 1."""
    clean = True
    for claim in contract.claims.topology:
        degree = int(degrees.get(claim.axis, 1))

        def check(claim=claim, degree=degree):
            if claim.kind == "pinned":
                return degree == int(claim.degree), f"{claim.axis}={degree}, pinned {claim.degree}"
            allowed = sorted(int(d) for d in claim.domain)
            return degree in allowed, f"{claim.axis}={degree}, invariant over {allowed}"

        clean &= checked(f"{DOMAIN_CHECK}:{claim.axis}", INSTALL, check)
    return clean


def attest_state_hooks(contract, package_root: Optional[str] = None) -> bool:
    """hook_exists: each state claim's ``ref`` ("path.py::symbol", relative to this package) names a file that
    defines that symbol."""
    root = package_root or os.path.normpath(os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
    clean = True
    for claim in contract.claims.state:

        def check(claim=claim):
            path, _, symbol = claim.ref.partition("::")
            with open(os.path.join(root, path)) as fh:
                source = fh.read()
            found = any(f"{kind} {symbol}(" in source or f"{kind} {symbol}:" in source for kind in ("def", "class"))
            return bool(symbol) and found, f"{claim.ref} {'defines' if found else 'does NOT define'} the hook"

        clean &= checked(f"{HOOK_EXISTS}:{claim.state_id}", INSTALL, check)
    return clean


def report_installed_backstop(side: str) -> bool:
    """installed_backstop: every (op, site) the contract names for ``side`` has an install on record."""
    from . import fingerprint
    from .process_contract import cached_contract_view

    obligation = f"{INSTALLED_BACKSTOP}:first_forward"
    view = cached_contract_view()
    if view is None:
        report(obligation, FIRST_FORWARD, SKIPPED, f"{SKIP_NO_LOCAL_CONTRACT}: local contract not built")
        return True
    recorded = fingerprint.recorder().installed
    absent = sorted(key for key in view if key[1] in SIDES[side] and key not in recorded)
    if not absent:
        report(obligation, FIRST_FORWARD, OK, f"all {sum(1 for k in view if k[1] in SIDES[side])} keys of {side} installed")
        return True
    complaint = f"[ISOEXEC-ENFORCE] {len(absent)} contract key(s) NOT installed on {side}: {absent}"
    report(obligation, FIRST_FORWARD, VIOLATION, complaint)
    return refuse(complaint)


def report_gate(contract, case_pair, measured: Dict[str, float]) -> bool:
    """gate: measured differences between two cases against the contract's tolerance claim for that pair. Every
    bound the claim names must be measured, and no measurement may exceed its bound (a NaN exceeds everything)."""
    wanted = tuple(case_pair)
    claim = next((c for c in contract.claims.tolerances if tuple(c.case_pair) == wanted), None)
    obligation = f"{GATE}:{'|'.join(wanted)}"
    if claim is None:
        report(obligation, STEP1, VIOLATION, f"the contract holds no tolerance claim for {wanted}")
        return refuse(f"[ISOEXEC-ENFORCE] no tolerance claim for {wanted}")
    bounds = dict(claim.bounds)
    over = []
    for name, limit in sorted(bounds.items()):
        if name not in measured:
            over.append(f"{name}: not measured")
        elif not float(measured[name]) <= float(limit):
            over.append(f"{name}: {measured[name]!r} > {limit}")
    if not over:
        report(obligation, STEP1, OK, ", ".join(f"{k}={measured[k]!r}<={v}" for k, v in sorted(bounds.items())))
        return True
    complaint = f"[ISOEXEC-ENFORCE] forward gate {wanted} RED: " + "; ".join(over)
    report(obligation, STEP1, VIOLATION, complaint)
    return refuse(complaint)


def report_served(op: str, site: str, served: int, detail: str = "") -> None:
    """served: the implementation's own count of calls it served at ``site`` since start-up."""
    result = OK if served > 0 else VIOLATION
    report(f"{SERVED}:{op}:{site}", STEP1, result, f"served={served} {detail}".strip())


def install_boundary(side: str) -> bool:
    return close_phase(INSTALL, side)


def first_forward_boundary(side: str) -> bool:
    report_installed_backstop(side)
    return close_phase(FIRST_FORWARD, side)


def weight_sync_boundary(side: str) -> bool:
    return close_phase(WEIGHT_SYNC, side)


def step1_boundary(side: str) -> bool:
    """Close STEP1 only in a process that has a contract: a controller that built none must not pronounce."""
    try:
        if arm(side) is None:
            return True
    except Exception as exc:  # noqa: BLE001
        logger.warning("[ISOEXEC-ENFORCE] step1_boundary(%s) plan check skipped: %s", side, exc)
        return True
    return close_phase(STEP1, side)
