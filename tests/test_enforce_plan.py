"""The obligation plan and the phase boundaries: what a contract makes a process owe, and what an unmet obligation
does at the boundary it is due at. The cases are those the reference's own tests of this layer set out
(isoexec/core/tests/test_enforce.py:78-180, 226-240, 408-560): derived plan, a suppressed reporter is a missing
violation, the severity table both ways, exemptions, recognised and unrecognised skips, a checker that raises, late
records, stray ids, the backstop, the gate."""

from collections import Counter

import pytest

from isoexec_amd.core import enforce, fingerprint, process_contract
from isoexec_amd.core.registry_build import build_registry
from isoexec_amd.models import qwen3_5


@pytest.fixture(autouse=True)
def fresh(monkeypatch):
    enforce._reset_for_tests()
    fingerprint._reset_for_tests()
    process_contract._reset_for_tests()
    for name in ("SKYRL_ISOEXEC_MANIFEST_STRICT", "SKYRL_ISOEXEC_DEBUG_TRACE"):
        monkeypatch.delenv(name, raising=False)
    yield
    enforce._reset_for_tests()


@pytest.fixture
def world(monkeypatch):
    reg = build_registry(strict=True)
    contract = qwen3_5.build(reg, arch="gfx950", profile=qwen3_5.PATH_PROFILE)
    monkeypatch.setattr(process_contract, "_CONTRACT", contract)
    monkeypatch.setattr(process_contract, "_VIEW", process_contract.build_contract_view(contract, reg))
    return contract, reg


def report_phase(plan, phase, skip=()):
    for ob in plan.obligations:
        if ob.phase == phase and ob.obligation_id not in skip:
            enforce.report(ob.obligation_id, phase, enforce.OK, "test")


def test_plan_is_derived_complete_and_deterministic(world):
    contract, reg = world
    view = process_contract.cached_contract_view()
    for side in ("trainer", "engine"):
        plan = enforce.derive_obligation_plan(contract, reg, side)
        assert plan == enforce.derive_obligation_plan(contract, reg, side)
        keys = [k for k in view if k[1] in enforce.SIDES[side]]
        kinds = Counter((ob.kind, ob.phase) for ob in plan.obligations)
        # one attestation and one fingerprint per (primary op, site) of the side that a composition entry names
        assert kinds[(enforce.INSTALL_ATTEST, enforce.INSTALL)] == kinds[(enforce.FINGERPRINT, enforce.FIRST_FORWARD)] > 0
        assert {f"fingerprint:{op}:{site}" for op, site in keys} >= {ob.obligation_id for ob in plan.obligations
                                                                     if ob.kind == enforce.FINGERPRINT}
        assert kinds[(enforce.DOMAIN_CHECK, enforce.INSTALL)] == len(contract.claims.topology) == 3
        assert kinds[(enforce.HOOK_EXISTS, enforce.INSTALL)] == len(contract.claims.state) == 1
        assert kinds[(enforce.GATE, enforce.STEP1)] == len(contract.claims.tolerances) == 1
        assert kinds[(enforce.HANDSHAKE, enforce.WEIGHT_SYNC)] == kinds[(enforce.BUILD_VALID, enforce.INSTALL)] == 1
        assert kinds[(enforce.INSTALLED_BACKSTOP, enforce.FIRST_FORWARD)] == 1
        # a served check only where the implementation keeps a count; everything else is listed, not dropped
        assert kinds[(enforce.SERVED, enforce.STEP1)] + len(plan.no_served_counter) == kinds[(enforce.INSTALL_ATTEST, enforce.INSTALL)]
        assert all((op, impl) not in enforce.SERVED_COUNTERS for op, _site, impl in plan.no_served_counter)
        phases = [enforce.PHASES.index(ob.phase) for ob in plan.obligations]
        assert phases == sorted(phases)
    with pytest.raises(ValueError, match="unknown side"):
        enforce.derive_obligation_plan(contract, reg, "controller")
    engine = enforce.derive_obligation_plan(contract, reg, "engine")
    served = {ob.obligation_id: ob for ob in engine.obligations if ob.kind == enforce.SERVED}
    assert "served:gdn.state:engine_decode" in served and "served:moe.experts:engine_decode" not in served
    assert ("moe.experts", "engine_decode", "hip_grouped_mfma") in engine.no_served_counter
    # the log-softmax path may decline on one side only: its served check refuses, the others log
    assert enforce.severity(served["served:logprobs.log_softmax:engine_decode"]) == enforce.REFUSE
    assert enforce.severity(served["served:gdn.state:engine_decode"]) == enforce.LOG


def test_a_check_that_never_ran_refuses_at_the_boundary(world, monkeypatch):
    contract, reg = world
    plan = enforce.arm("trainer")
    report_phase(plan, enforce.INSTALL, skip={"install_attest:mm:trainer_fwd"})
    with pytest.raises(RuntimeError, match=r"install_attest:mm:trainer_fwd \(missing\)"):
        enforce.close_phase(enforce.INSTALL, "trainer")
    assert enforce.verdict_counts()["missing"] == 1
    monkeypatch.setenv("SKYRL_ISOEXEC_MANIFEST_STRICT", "0")
    assert enforce.close_phase(enforce.INSTALL, "trainer") is False          # demoted: recorded, the run goes on
    enforce.report("install_attest:mm:trainer_fwd", enforce.INSTALL, enforce.OK, "late but there")
    monkeypatch.delenv("SKYRL_ISOEXEC_MANIFEST_STRICT")
    assert enforce.close_phase(enforce.INSTALL, "trainer") is True


def test_severity_table_both_ways(world):
    contract, reg = world
    plan = enforce.arm("engine")
    report_phase(plan, enforce.INSTALL)
    enforce.report("install_attest:moe.experts:engine_prefill", enforce.INSTALL, enforce.VIOLATION, "test violation")
    with pytest.raises(RuntimeError, match="install_attest:moe.experts:engine_prefill"):
        enforce.close_phase(enforce.INSTALL, "engine")
    # a served count of zero on a counter that only logs does not refuse STEP1 ...
    report_phase(plan, enforce.STEP1)
    enforce.report_served("gdn.state", "engine_decode", 0, "resolver never ran")
    assert enforce.close_phase(enforce.STEP1, "engine") is True
    assert enforce.verdict_counts()["logged"] == 1
    # ... while the escalated one does
    enforce.report_served("logprobs.log_softmax", "engine_decode", 0)
    with pytest.raises(RuntimeError, match=r"served:logprobs.log_softmax:engine_decode \(violation\)"):
        enforce.close_phase(enforce.STEP1, "engine")
    # a deployment-half entry's obligations only ever log
    soft = enforce.Obligation("install_attest:x:engine_decode", enforce.INSTALL_ATTEST, enforce.INSTALL, half="deployment")
    assert enforce.severity(soft) == enforce.LOG
    assert enforce.severity(enforce.Obligation("served:x:y", enforce.SERVED, enforce.STEP1, "deployment", escalated=True)) == enforce.LOG


def test_exemptions_cover_exactly_their_target(world):
    contract, reg = world
    assert enforce.exemption_for("install_attest:gdn.state:engine_prefill") is not None
    assert enforce.exemption_for("fingerprint:gdn.state:engine_prefill") is None
    plan = enforce.arm("engine")
    attest_state = {ob.obligation_id for ob in plan.obligations if ob.obligation_id.startswith("install_attest:gdn.state:")}
    assert len(attest_state) == 2
    report_phase(plan, enforce.INSTALL, skip=attest_state)
    assert enforce.close_phase(enforce.INSTALL, "engine") is True
    assert enforce.verdict_counts()["excepted"] == 2
    enforce._reset_for_tests()
    plan = enforce.arm("engine")
    report_phase(plan, enforce.INSTALL, skip={"install_attest:gdn.core:engine_prefill"})
    with pytest.raises(RuntimeError, match="install_attest:gdn.core:engine_prefill"):
        enforce.close_phase(enforce.INSTALL, "engine")
    assert all(e.reason and e.removal for e in enforce.EXCEPTIONS)


def test_skips_discharge_only_with_a_structural_reason(world):
    contract, reg = world
    plan = enforce.arm("trainer")
    report_phase(plan, enforce.WEIGHT_SYNC, skip={"handshake:numerical_policy"})
    enforce.report("handshake:numerical_policy", enforce.WEIGHT_SYNC, enforce.SKIPPED, f"{enforce.SKIP_NO_PEER_STAMP}: engine stamped nothing")
    assert enforce.close_phase(enforce.WEIGHT_SYNC, "trainer") is True
    assert enforce.verdict_counts()["logged"] == 1
    enforce._reset_for_tests()
    enforce.arm("trainer")
    enforce.report("handshake:numerical_policy", enforce.WEIGHT_SYNC, enforce.SKIPPED, "did not feel like it")
    with pytest.raises(RuntimeError, match=r"handshake:numerical_policy \(unchecked\)"):
        enforce.close_phase(enforce.WEIGHT_SYNC, "trainer")
    assert enforce.verdict_counts()["refused"] == 1


def test_nothing_reported_cannot_close_clean(world):
    enforce.arm("trainer")
    with pytest.raises(RuntimeError, match="never checked"):
        enforce.install_boundary("trainer")


def test_a_checker_that_raises_fails_closed(world):
    def broken():
        raise KeyError("boom")

    assert enforce.checked("domain_check:TP", enforce.INSTALL, broken) is False
    last = enforce.ledger().records[-1]
    assert last.result == enforce.VIOLATION and last.evidence.startswith(enforce.CHECKER_ERROR) and "KeyError" in last.evidence


def test_claim_reporters(world, monkeypatch):
    contract, reg = world
    assert enforce.report_topology(contract, {}) is True                        # one device: every axis at degree 1
    assert enforce.report_topology(contract, {"TP": 2}) is False
    assert enforce.ledger().by_id("domain_check:TP")[-1].evidence == "TP=2, pinned 1"
    assert enforce.attest_state_hooks(contract) is True
    assert "defines the hook" in enforce.ledger().by_id("hook_exists:gdn_recurrent_state")[-1].evidence
    import dataclasses

    ghost = dataclasses.replace(contract.claims.state[0], ref="ops/gdn/gdn_recurrent_state.py::no_such_hook_anywhere")
    moved = dataclasses.replace(contract, claims=dataclasses.replace(contract.claims, state=(ghost,)))
    assert enforce.attest_state_hooks(moved) is False
    gone = dataclasses.replace(contract.claims.state[0], ref="ops/gdn/not_a_file.py::x")
    moved = dataclasses.replace(contract, claims=dataclasses.replace(contract.claims, state=(gone,)))
    assert enforce.attest_state_hooks(moved) is False
    assert enforce.ledger().records[-1].evidence.startswith(enforce.CHECKER_ERROR)


def test_gate_reporter_and_step1(world):
    contract, reg = world
    pair = ("engine_decode", "trainer_score")
    plan = enforce.arm("trainer")
    report_phase(plan, enforce.STEP1, skip={"gate:engine_decode|trainer_score"})
    assert enforce.report_gate(contract, pair, {"abs_diff_max_max": 0.0, "abs_diff_mean_max": 0.0}) is True
    assert enforce.step1_boundary("trainer") is True
    with pytest.raises(RuntimeError, match="RED"):
        enforce.report_gate(contract, pair, {"abs_diff_max_max": 1e-6, "abs_diff_mean_max": 0.0})
    with pytest.raises(RuntimeError, match="gate:engine_decode"):
        enforce.step1_boundary("trainer")                                        # the recorded violation refuses the close too
    enforce._reset_for_tests()
    with pytest.raises(RuntimeError, match="not measured"):
        enforce.report_gate(contract, pair, {"abs_diff_max_max": 0.0})
    with pytest.raises(RuntimeError, match="abs_diff_mean_max"):
        enforce.report_gate(contract, pair, {"abs_diff_max_max": 0.0, "abs_diff_mean_max": float("nan")})
    with pytest.raises(RuntimeError, match="no tolerance claim"):
        enforce.report_gate(contract, ("trainer_fwd", "trainer_score"), {})


def test_backstop_wants_every_key_of_the_side(world):
    view = process_contract.cached_contract_view()
    keys = [k for k in view if k[1].startswith("trainer")]
    for op, site in keys:
        fingerprint.record_install(op, site, "x")
    assert enforce.report_installed_backstop("trainer") is True
    assert enforce.ledger().by_id("installed_backstop:first_forward")[-1].result == enforce.OK
    enforce._reset_for_tests()
    fingerprint._reset_for_tests()
    for op, site in keys[1:]:
        fingerprint.record_install(op, site, "x")
    with pytest.raises(RuntimeError, match="NOT installed"):
        enforce.report_installed_backstop("trainer")
    assert enforce.ledger().by_id("installed_backstop:first_forward")[-1].result == enforce.VIOLATION


def test_without_a_contract_boundaries_pass_and_say_so(caplog):
    assert enforce.step1_boundary("trainer") is True and enforce.ledger().closed == set()
    assert enforce.close_phase(enforce.INSTALL, "trainer") is True
    assert "NO contract built" in caplog.text
    assert enforce.report_installed_backstop("trainer") is True
    assert enforce.SKIP_NO_LOCAL_CONTRACT in enforce.ledger().records[-1].evidence


def test_late_records_stray_ids_and_internal_errors_reach_the_verdict(world, monkeypatch):
    contract, reg = world
    plan = enforce.arm("trainer")
    report_phase(plan, enforce.INSTALL)
    assert enforce.close_phase(enforce.INSTALL, "trainer") is True
    enforce.report("install_attest:mm:trainer_fwd", enforce.INSTALL, enforce.VIOLATION, "after the boundary")
    enforce.report("install_attest:mm:engine_decode", enforce.INSTALL, enforce.OK, "another side's: not late for an engine that has not closed")
    enforce.arm("engine")
    enforce.report("install_attest:mm:engine_decode", enforce.INSTALL, enforce.OK, "owed by the engine, whose boundary is open")
    enforce.report("made_up:thing", enforce.INSTALL, enforce.OK, "nobody planned this")
    v = enforce.verdict()
    late = [r["evidence"] for r in v["reopened"]]
    assert "after the boundary" in late and "owed by the engine, whose boundary is open" not in late
    assert "nobody planned this" in late                                         # unowned: late for any closed boundary
    stray = [row for row in v["obligations"] if row["kind"] == "unplanned"]
    assert [row["id"] for row in stray] == ["made_up:thing"]
    assert v["phases_closed"] == ["trainer:INSTALL"] and v["sides"] == ["engine", "trainer"]
    row = next(r for r in v["obligations"] if r["id"] == "install_attest:mm:trainer_fwd" and r["side"] == "trainer")
    assert row["status"] == enforce.VIOLATION and row["severity"] == enforce.REFUSE and len(row["records"]) == 2
    assert next(r for r in v["obligations"] if r["id"] == "gate:engine_decode|trainer_score" and r["side"] == "trainer")["status"] == "open"
    import json

    assert json.loads(json.dumps(v)) == v                                        # plain data
    monkeypatch.setattr(enforce, "verdict_counts", lambda: 1 / 0)
    assert enforce.close_phase(enforce.FIRST_FORWARD, "trainer") is True         # a bug in the boundary does not stop the run
    assert "ZeroDivisionError" in enforce.ledger().internal_errors[-1]


def test_hybrid_runtimes_close_every_boundary_green_and_a_one_sided_choice_refuses(monkeypatch):
    """The whole life of a run on the host: contract from the configuration's own declaration, installs recorded from
    what the runtimes bind, the claims' checks, fingerprint against the contract, handshake -- every boundary closes
    with nothing missing. An engine that sums the experts' rows in bf16 under a contract that says fp32 is refused at
    its first forward."""
    import dataclasses

    from isoexec_amd.runtimes.hybrid import HybridConfig, bound_implementations, record_runtime_installs

    cfg = HybridConfig()
    reg = build_registry(strict=True)
    contract = qwen3_5.build(reg, arch="gfx950", profile=cfg.profile())
    view = process_contract.build_contract_view(contract, reg)
    monkeypatch.setattr(process_contract, "_CONTRACT", contract)
    monkeypatch.setattr(process_contract, "_VIEW", view)
    assert view[("moe.router", "engine_decode")]["pinned_constants"] == {"topk": 8, "experts": 128, "score": "softmax_then_topk"}
    assert set(bound_implementations(cfg)) == {op for op, _ in view}
    for side in ("trainer", "engine"):
        enforce.report("build_valid:contract", enforce.INSTALL, enforce.OK, "built above")
        assert record_runtime_installs(cfg, side, reg) == sum(1 for k in view if k[1] in enforce.SIDES[side])
        assert enforce.report_topology(contract, {}) and enforce.attest_state_hooks(contract)
        assert enforce.install_boundary(side) is True
        assert fingerprint.log_fingerprint(view, tag=f"{side}_first_forward") == []
        assert enforce.first_forward_boundary(side) is True
        assert process_contract.assert_contract_agreement(contract.identities.numerical_policy, other_side="peer") is True
        assert enforce.weight_sync_boundary(side) is True
    counts = enforce.verdict_counts()
    assert counts["missing"] == counts["refused"] == counts["logged"] == 0 and counts["ok"] > 60
    assert counts["excepted"] == 2          # the engine's two state-pool attestations stay in the excepted column even when met
    assert all(row["status"] in (enforce.OK, "open") for row in enforce.verdict()["obligations"])

    enforce._reset_for_tests()
    fingerprint._reset_for_tests()
    engine_cfg = dataclasses.replace(cfg, moe_combine_dtype="bf16")
    enforce.report("build_valid:contract", enforce.INSTALL, enforce.OK, "built above")
    record_runtime_installs(engine_cfg, "engine", reg)
    enforce.report_topology(contract, {})
    enforce.attest_state_hooks(contract)
    assert enforce.install_boundary("engine") is True                       # an attestation says THAT something was bound
    found = fingerprint.log_fingerprint(view, tag="engine_first_forward")   # the fingerprint says WHAT
    assert len(found) == 2 and all("leaf_dtype: contract pins 'fp32', install used 'bf16'" in line for line in found)
    with pytest.raises(RuntimeError, match=r"fingerprint:moe.combine:engine_decode \(violation\)"):
        enforce.first_forward_boundary("engine")
