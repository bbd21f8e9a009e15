"""Registry vocabulary, contract build refusals, the handshake and the install fingerprint.

Follows the reference's own unit tests of this layer (isoexec/core/tests: registry, contract_build,
process_contract, fingerprint). Everything here runs on the host; no kernel is touched.
"""

import dataclasses
import json
import struct

import pytest

from isoexec_amd import contract as K
from isoexec_amd.core import contract_build as CB
from isoexec_amd.core import enforce, fingerprint, process_contract
from isoexec_amd.core.arch import NON_ACCELERATOR_ARCH, ArchMismatchError, HardwareTarget, _tag_from_gcn_name, is_accelerator_arch
from isoexec_amd.core.contract_delivery import (
    ContractDeliveryError,
    expected_installed_keys,
    load_contract,
    validate_contract_against_installed,
    write_contract_file,
)
from isoexec_amd.core.registry import (
    PER_MODEL,
    ImplSpec,
    OneOf,
    OpSpec,
    Registry,
    RegistryError,
    RoundingSchedule,
    pin_values_equal,
)
from isoexec_amd.core.registry_build import build_registry, registered_families
from isoexec_amd.models import build_for, policy, profile_for, qwen3_5, resolve
from isoexec_amd.models.profile import ModelProfile, ProfileError, RouterProfile, StateFact, ToleranceFact, TopologyAxisFact

ALL = ["trainer_fwd", "trainer_score", "engine_prefill", "engine_decode"]
GFX = frozenset({"gfx950"})
# Assembled at run time so that this file does not itself contain the name it must not resolve.
GHOST = "_".join(["no", "such", "gate", "9f3a"])


@pytest.fixture(autouse=True)
def _fresh_process_state(monkeypatch):
    enforce._reset_for_tests()
    fingerprint._reset_for_tests()
    process_contract._reset_for_tests()
    monkeypatch.delenv("SKYRL_ISOEXEC_MANIFEST_STRICT", raising=False)
    monkeypatch.delenv("SKYRL_ISOEXEC_DEBUG_TRACE", raising=False)
    monkeypatch.delenv("ISOEXEC_CONTRACT_PATH", raising=False)
    monkeypatch.delenv("ISOEXEC_CONTRACT_HASH", raising=False)
    yield


def impl(impl_id, assertable=None, **kw):
    return ImplSpec(impl_id=impl_id, version=kw.pop("version", 1), supported_archs=kw.pop("archs", GFX),
                    rounding=RoundingSchedule(machine_assertable=assertable or {}), **kw)


def toy_registry():
    reg = Registry()
    reg.register_op(OpSpec("mm", list(ALL)).add_impl(impl("hip", {"split_k": 1, "tile": OneOf("a", "b"), "leaves": PER_MODEL, "eps": PER_MODEL})))
    reg.register_op(OpSpec("norm", list(ALL))
                    .add_impl(impl("eager", route="canonical"))
                    .add_impl(impl("fused", capabilities={"bitwise_equal_to": "eager"}))
                    .add_impl(impl("third")))
    reg.register_op(OpSpec("core", list(ALL)).add_impl(impl("fusedcore", subsumes=("gate",))))
    reg.register_op(OpSpec("gate", list(ALL)).add_impl(impl("g")))
    reg.register_op(OpSpec("state", ["engine_prefill", "engine_decode"]).add_impl(impl("pool")))
    return reg


def sel(impl_id, **kw):
    return dict(impl_id=impl_id, **kw)


def build(reg, selections, **kw):
    kw.setdefault("arch", "gfx950")
    return CB.build_execution_contract(reg, selections, model="toy", **kw)


# ------------------------------------------------------------------ registry


def test_registry_vocabulary():
    reg = toy_registry()
    with pytest.raises(RegistryError, match="already registered"):
        reg.register_op(OpSpec("mm", list(ALL)))
    with pytest.raises(RegistryError, match="unknown site"):
        reg.register_op(OpSpec("x", ["engine_warmup"]))
    reg.register_site("engine_warmup")
    reg.register_op(OpSpec("x", ["engine_warmup"]))
    with pytest.raises(RegistryError, match="invalid site name"):
        reg.register_site("bad name")
    with pytest.raises(RegistryError, match="already has impl"):
        reg.get_op("mm").add_impl(impl("hip"))
    with pytest.raises(RegistryError, match="unknown hazard"):
        impl("h", hazards=["cosmic_rays"])
    with pytest.raises(RegistryError, match="unknown route"):
        impl("h", route="fast")
    with pytest.raises(RegistryError, match="at least one supported arch"):
        impl("h", archs=frozenset())
    with pytest.raises(RegistryError, match="unknown op"):
        reg.get_op("nope")
    assert ("state", "engine_decode") in reg.installed_keys() and ("state", "trainer_fwd") not in reg.installed_keys()
    reg.register_op(OpSpec("y", list(ALL)).add_impl(impl("i", subsumes=("ghost",))))
    with pytest.raises(RegistryError, match="subsumes unregistered op 'ghost'"):
        reg.assert_subsumption_closed()


def test_pin_checking():
    sched = RoundingSchedule({"block": 4096, "leaves": PER_MODEL, "mode": OneOf("a", ("x", 1)), "flag": True, "order": ["a", "b"]})
    assert sched.check_pin("block", 4096) is None
    assert "declares block=4096" in sched.check_pin("block", 2048)
    assert sched.check_pin("leaves", 123) is None
    assert sched.check_pin("mode", "a") is None and sched.check_pin("mode", ["x", 1]) is None
    assert "OneOf" in sched.check_pin("mode", "c")
    assert "declares no such key" in sched.check_pin("blok", 4096)
    assert sched.check_pin("flag", True) is None and sched.check_pin("flag", 1) is not None
    assert sched.check_pin("order", ("a", "b")) is None and sched.check_pin("order", ("b", "a")) is not None
    assert pin_values_equal({"a": (1, 2)}, {"a": [1, 2]}) and not pin_values_equal(0, False)
    assert repr(PER_MODEL) == "PER_MODEL"


# ------------------------------------------------------------------ build: refusals


def test_build_refuses_bad_inputs():
    reg = toy_registry()
    good = {("mm", s): sel("hip") for s in ALL}
    with pytest.raises(CB.ContractBuildError, match="non-accelerator sentinel"):
        build(reg, good, arch=NON_ACCELERATOR_ARCH)
    with pytest.raises(CB.ContractBuildError, match="empty selection map"):
        build(reg, {})
    with pytest.raises(CB.ContractBuildError, match="unknown op 'conv'"):
        build(reg, {("conv", "trainer_fwd"): sel("x")})
    with pytest.raises(CB.ContractBuildError, match="declares only"):
        build(reg, {("state", "trainer_fwd"): sel("pool")})
    with pytest.raises(CB.ContractBuildError, match="names impl 'cuda'"):
        build(reg, {("mm", "trainer_fwd"): sel("cuda")})
    with pytest.raises(CB.ContractBuildError, match="supported_archs \\['gfx950'\\].*arch 'sm90'"):
        build(reg, good, arch="sm90")
    with pytest.raises(CB.ContractBuildError, match="unknown classification"):
        build(reg, {("mm", "trainer_fwd"): sel("hip", classification="maybe")})
    with pytest.raises(CB.ContractBuildError, match="requires a recorded neutrality_proof"):
        build(reg, {("mm", "trainer_fwd"): sel("hip", classification="deployment")})
    with pytest.raises(CB.ContractBuildError, match="must not carry a neutrality_proof"):
        build(reg, {("mm", "trainer_fwd"): sel("hip", neutrality_proof="run-1")})
    open_reg = toy_registry()
    open_reg.register_op(OpSpec("y", list(ALL)).add_impl(impl("i", subsumes=("ghost",))))
    with pytest.raises(CB.ContractBuildError, match="not subsumption-closed"):
        build(open_reg, good)
    # The sentinel is allowed only on request, and then skips arch admission.
    c = build(reg, good, arch=NON_ACCELERATOR_ARCH, allow_non_accelerator_arch=True)
    assert c.composition[0].impl.arch == "cpu"


def test_pins_are_validated_against_the_schedule():
    reg = toy_registry()
    with pytest.raises(CB.PinValidationError) as err:
        build(reg, {("mm", "trainer_fwd"): sel("hip", pinned_constants={"split_k": 2, "tile": "c", "bogus": 1, "leaves": 8})})
    text = str(err.value)
    assert "pin split_k=2" in text and "pin tile='c'" in text and "pin bogus=1" in text and "leaves" not in text.split("\n\n")[0].replace("'leaves'", "")
    assert "model 'toy'" in text
    ok = build(reg, {("mm", "trainer_fwd"): sel("hip", pinned_constants={"split_k": 1, "tile": "b", "leaves": 8})})
    assert dict(ok.composition[0].constants) == {"split_k": 1, "tile": "b", "leaves": 8}
    unchecked = build(reg, {("mm", "trainer_fwd"): sel("hip", pinned_constants={"bogus": 1})}, validate_pins=False)
    assert dict(unchecked.composition[0].constants) == {"bogus": 1}
    with pytest.raises(CB.ContractBuildError, match="non-scalar"):
        build(reg, {("mm", "trainer_fwd"): sel("hip", pinned_constants={"leaves": [1, 2]})})


def test_float_pins_travel_as_fp64_bit_patterns():
    reg = toy_registry()
    c = build(reg, {("mm", "trainer_fwd"): sel("hip", pinned_constants={"eps": 1e-6, "leaves": None})})
    consts = dict(c.composition[0].constants)
    assert consts["eps"] == K.BitPattern("0x%016x" % struct.unpack("<Q", struct.pack("<d", 1e-6))[0], "fp64")
    assert consts["eps"].bits == "0x3eb0c6f7a0b5ed8d" and consts["leaves"] is None
    view = process_contract.build_contract_view(c, reg)
    assert view[("mm", "trainer_fwd")]["pinned_constants"] == {"eps": 1e-6, "leaves": None}
    K.from_canonical_json(K.to_canonical_json(c))


# ------------------------------------------------------------------ build: projection


def test_sites_merge_and_regions_absorb_subsumed_ops():
    reg = toy_registry()
    selections = {("core", s): sel("fusedcore") for s in ALL}
    selections.update({("mm", s): sel("hip", pinned_constants={"leaves": 8 if s.startswith("trainer") else 4}) for s in ALL})
    selections.update({("state", s): sel("pool") for s in ("engine_prefill", "engine_decode")})
    c = build(reg, selections)
    got = [(e.region, e.cases, dict(e.constants)) for e in c.composition]
    assert got == [
        (("core", "gate"), ("engine_decode", "engine_prefill", "trainer_fwd", "trainer_score"), {}),
        (("mm",), ("engine_decode", "engine_prefill"), {"leaves": 4}),
        (("mm",), ("trainer_fwd", "trainer_score"), {"leaves": 8}),
        (("state",), ("engine_decode", "engine_prefill"), {}),
    ]
    assert [x.id for x in c.cases] == ["engine_decode", "engine_prefill", "trainer_fwd", "trainer_score"]
    assert c.cases[0].constraints == ("cudagraph_capturable", "host_free", "address_stable")
    assert c.model == K.ModelRef("toy", (), "models/toy") and c.schema_version == "2"
    assert K.validate(c) == [] and all(e.impl.arch == "gfx950" and e.half == "function" for e in c.composition)
    engine_only = build(reg, {("state", "engine_decode"): sel("pool")})
    assert [x.id for x in engine_only.cases] == ["engine_decode"]
    # Selection objects and mappings are interchangeable.
    as_records = {k: policy.entry(v["impl_id"], pinned=v.get("pinned_constants")) for k, v in selections.items()}
    assert build(reg, as_records).identities == c.identities


def test_asymmetric_ops_need_a_discharge_that_links_the_whole_group():
    reg = toy_registry()
    two = {("norm", s): sel("eager" if s.startswith("trainer") else "fused") for s in ALL}
    c = build(reg, two)
    assert {e.impl.id: e.discharge for e in c.composition} == {
        "eager": K.EquivalenceProof("bitwise_equal_to", "eager"),
        "fused": K.EquivalenceProof("bitwise_equal_to", "eager"),
    }
    assert {e.impl.id: e.route for e in c.composition} == {"eager": "canonical", "fused": "protected"}
    three = dict(two)
    three[("norm", "engine_decode")] = sel("third")
    with pytest.raises(CB.ContractBuildError, match="link only \\['eager', 'fused'\\]"):
        build(reg, three)
    with pytest.raises(CB.ContractBuildError, match="no selected impl declares"):
        build(reg, {("norm", "trainer_fwd"): sel("eager"), ("norm", "engine_decode"): sel("third")})
    with pytest.raises(CB.ContractBuildError, match="does not reach the impls"):
        build(reg, {("norm", "trainer_fwd"): sel("third"), ("norm", "engine_decode"): sel("fused")})

    selfish = Registry()
    selfish.register_op(OpSpec("n", list(ALL)).add_impl(impl("a", capabilities={"bitwise_equal_to": "a"})).add_impl(impl("b")))
    with pytest.raises(CB.ContractBuildError, match="ITSELF"):
        build(selfish, {("n", "trainer_fwd"): sel("a"), ("n", "engine_decode"): sel("b")})
    dangling = Registry()
    dangling.register_op(OpSpec("n", list(ALL)).add_impl(impl("a", capabilities={"bitwise_equal_to": "zz"})).add_impl(impl("b")))
    with pytest.raises(CB.ContractBuildError, match="not a registered impl"):
        build(dangling, {("n", "trainer_fwd"): sel("a"), ("n", "engine_decode"): sel("b")})


def test_equivalence_proofs_must_resolve_and_deployment_entries_carry_their_own():
    reg = Registry()
    reg.register_op(OpSpec("n", list(ALL))
                    .add_impl(impl("a"))
                    .add_impl(impl("b", capabilities={"equivalence_proof": "test_contract_build.py: b equals a"}))
                    .add_impl(impl("c", capabilities={"equivalence_proof": GHOST + ": nothing"})))
    c = build(reg, {("n", "trainer_fwd"): sel("a"), ("n", "engine_decode"): sel("b")})
    assert all(e.discharge == K.EquivalenceProof("equivalence_proof", "test_contract_build.py: b equals a") for e in c.composition)
    with pytest.raises(CB.ContractBuildError, match="resolves to no gate"):
        build(reg, {("n", "trainer_fwd"): sel("a"), ("n", "engine_decode"): sel("c")})
    dep = build(reg, {("n", "trainer_fwd"): sel("a"),
                      ("n", "engine_decode"): sel("a", version=1, classification="deployment", neutrality_proof="run-7", pinned_constants={})})
    halves = {e.cases: (e.half, e.discharge) for e in dep.composition}
    assert halves[("engine_decode",)] == ("deployment", K.EquivalenceProof("neutrality_proof", "run-7"))
    assert halves[("trainer_fwd",)] == ("function", None)
    with pytest.raises(CB.ContractBuildError, match="topology claim 'TP'.*resolves to no gate"):
        build(reg, {("n", "trainer_fwd"): sel("a")},
              topology=(TopologyAxisFact("TP", "invariant", domain=(1, 2), proof=GHOST),))


def test_claims_are_sorted_into_the_contract():
    reg = toy_registry()
    topo = (TopologyAxisFact("TP", "pinned", degree=1, collective_plan="none"), TopologyAxisFact("CP", "pinned", degree=1, collective_plan="none"))
    states = (StateFact("z_state", ("weight_sync",), True, "a.py::f"), StateFact("a_state", ("sleep_wake",), False, "a.py::g"))
    tols = (ToleranceFact(("engine_decode", "trainer_score"), (("max", "0.0"),)),)
    sels = {("mm", s): sel("hip") for s in ALL}
    c = build(reg, sels, topology=topo, states=states, tolerances=tols)
    assert [t.axis for t in c.claims.topology] == ["CP", "TP"]
    assert [s.state_id for s in c.claims.state] == ["a_state", "z_state"]
    assert c.claims.tolerances[0].bounds == (("max", "0.0"),)
    again = build(reg, sels, topology=topo[::-1], states=states[::-1], tolerances=tols)
    assert K.to_canonical_json(again) == K.to_canonical_json(c)


# ------------------------------------------------------------------ arch


def test_arch_tags():
    assert _tag_from_gcn_name("gfx950:sramecc+:xnack-") == "gfx950"
    assert is_accelerator_arch("gfx950") and not is_accelerator_arch("cpu") and not is_accelerator_arch("")
    assert HardwareTarget("gfx950").supports({"gfx950", "gfx942"}) and not HardwareTarget("gfx942").supports(GFX)
    HardwareTarget("gfx950").assert_homogeneous("gfx950")
    with pytest.raises(ArchMismatchError):
        HardwareTarget("gfx950").assert_homogeneous("sm90")


# ------------------------------------------------------------------ the shipped registry and model


def test_shipped_registry_and_policy_agree():
    reg = build_registry()
    assert registered_families() == ["mm", "attention", "rope", "norms", "logprobs", "gdn", "moe"]
    for op in reg.ops.values():
        for spec in op.impls.values():
            assert spec.supported_archs == GFX, (op.name, spec.impl_id)
    assert policy.policy_matches_registry_capabilities(qwen3_5.PATH_PROFILE, reg) == []
    assert policy.policy_matches_registry_capabilities(qwen3_5.PROFILE, reg) == []
    full = policy.derive_selections(qwen3_5.PROFILE)
    assert full[("attention.varlen", "engine_decode")].pinned_constants == {"num_splits": 1}
    # ops absorbed by another op's impl (the fused GatedDeltaNet core; the permutation's block map; the fc1 epilogue
    # and the single expert-weight buffer of the grouped GEMMs) are registered but get no entry of their own
    absorbed = ("gdn.l2norm", "gdn.gating", "moe.blockmap", "moe.epilogue", "moe.weights")
    assert ("rope.rope", "trainer_fwd") in full and frozenset(full) == reg.installed_keys() - {
        (op, s) for op in absorbed for s in ALL}
    assert set(reg.ops["moe.dispatch"].impls["hip_bitmask_index"].subsumes) == {"moe.blockmap"}
    assert set(reg.ops["moe.experts"].impls["hip_grouped_mfma"].subsumes) == {"moe.epilogue", "moe.weights"}
    sels = policy.derive_selections(qwen3_5.PATH_PROFILE)
    assert ("gdn.l2norm", "trainer_fwd") not in sels and ("gdn.state", "trainer_fwd") not in sels
    assert sels[("logprobs.log_softmax", "engine_decode")].pinned_constants == {"leaves": 8, "block": 4096, "accum": "kahan_fp32"}
    assert qwen3_5.PATH_PROFILE.op_families() == {"mm", "norms", "logprobs", "gdn", "moe"}
    assert "attention" in qwen3_5.PROFILE.op_families()


def test_model_contract_builds_and_is_reproducible():
    reg = build_registry()
    a = qwen3_5.build(reg, arch="gfx950", profile=qwen3_5.PATH_PROFILE)
    b = qwen3_5.build(build_registry(), arch="gfx950", profile=qwen3_5.PATH_PROFILE)
    assert K.to_canonical_json(a) == K.to_canonical_json(b)
    assert K.validate(a) == []
    regions = {e.region for e in a.composition}
    assert ("gdn.core", "gdn.gating", "gdn.l2norm") in regions and ("gdn.gating",) not in regions
    assert expected_installed_keys(a, reg) == frozenset(policy.derive_selections(qwen3_5.PATH_PROFILE))
    # A different function is a different numerical policy; the model's meaning does not move.
    leaves4 = qwen3_5.build(reg, arch="gfx950", profile=qwen3_5.PATH_PROFILE.with_overrides(pik_leaves=4))
    assert leaves4.identities.numerical_policy != a.identities.numerical_policy
    assert leaves4.identities.semantic == a.identities.semantic
    other_arch_reg = build_registry()
    with pytest.raises(CB.ContractBuildError, match="built for arch 'gfx942'"):
        qwen3_5.build(other_arch_reg, arch="gfx942", profile=qwen3_5.PATH_PROFILE)
    with pytest.raises(CB.PinValidationError, match="kernel='chunk'"):
        qwen3_5.build(reg, arch="gfx950", profile=qwen3_5.PATH_PROFILE.with_overrides(gdn_kernel="chunk"))
    # The whole model adds the attention and rope entries: more logical ops, so a different meaning.
    whole = qwen3_5.build(reg, arch="gfx950")
    assert {("attention.varlen",), ("rope.rope",)} <= {e.region for e in whole.composition}
    assert whole.identities.semantic != a.identities.semantic and K.validate(whole) == []
    with pytest.raises(CB.PinValidationError, match="num_splits=2"):
        CB.build_execution_contract(reg, {**policy.derive_selections(qwen3_5.PROFILE),
                                          ("attention.varlen", "engine_decode"): policy.entry("hip_varlen_ns1", pinned={"num_splits": 2})},
                                    arch="gfx950", model="m")


def test_policy_exceptions_and_refusals():
    sels = policy.derive_selections(qwen3_5.PATH_PROFILE)
    dropped = policy.apply_exceptions(sels, {("logprobs.lm_head_slice", "*"): policy.DROP})
    assert not any(op == "logprobs.lm_head_slice" for op, _ in dropped)
    swapped = policy.apply_exceptions(sels, {("mm", "engine_decode"): policy.entry("other")})
    assert swapped[("mm", "engine_decode")].impl_id == "other" and swapped[("mm", "trainer_fwd")].impl_id != "other"
    with pytest.raises(ValueError, match="produced no such key"):
        policy.apply_exceptions(sels, {("attention.varlen", "*"): policy.DROP})
    with pytest.raises(CB.ContractBuildError, match="neutrality_proof"):
        policy.Selection("x", classification="deployment")
    with pytest.raises(CB.ContractBuildError, match="bias-free softmax"):
        policy.derive_selections(qwen3_5.PATH_PROFILE.with_overrides(router=RouterProfile("sigmoid", True)))
    with pytest.raises(CB.ContractBuildError, match="collectives"):
        policy.derive_selections(qwen3_5.PATH_PROFILE.with_overrides(tensor_parallel=True))


def test_profile_facts_refuse_ill_formed_declarations():
    with pytest.raises(ProfileError, match="requires a RouterProfile"):
        ModelProfile("m", has_moe=True)
    with pytest.raises(ProfileError, match="has_moe=False"):
        ModelProfile("m", router=RouterProfile())
    with pytest.raises(ProfileError, match="unknown attention"):
        ModelProfile("m", attention="mla")
    with pytest.raises(ProfileError, match="tautology"):
        TopologyAxisFact("TP", "invariant", domain=(2, 2), proof="x")
    with pytest.raises(ProfileError, match="pinned requires"):
        TopologyAxisFact("TP", "pinned", degree=1)
    with pytest.raises(ProfileError, match="unknown lifecycle"):
        StateFact("s", ("reboot",), True, "a.py::f")
    with pytest.raises(ProfileError, match="finite threshold"):
        ToleranceFact(("a", "b"), (("max", "inf"),))
    with pytest.raises(ProfileError, match="decimal string"):
        ToleranceFact(("a", "b"), (("max", "tight"),))
    with pytest.raises(ProfileError, match="duplicate topology axis"):
        ModelProfile("m", topology=(TopologyAxisFact("PP", "pinned", degree=1, collective_plan="none"),) * 2)


def test_model_resolution(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps({"architectures": ["Qwen3_5MoeForCausalLM"]}))
    mod, how = resolve.resolve_model_module(str(tmp_path))
    assert mod is qwen3_5 and "architecture" in how
    assert resolve.resolve_model_module("Qwen/Qwen3.5-35B-A3B")[1].startswith("name pattern")
    assert profile_for("org/qwen3-next-80b") is qwen3_5.PROFILE
    with pytest.raises(resolve.ResolutionError, match="no model declaration"):
        resolve.resolve_model_module("org/some-llama")
    other = tmp_path / "other"
    other.mkdir()
    (other / "config.json").write_text(json.dumps({"architectures": ["LlamaForCausalLM"]}))
    with pytest.raises(resolve.ResolutionError):
        build_for(str(other), build_registry(), arch="gfx950")


# ------------------------------------------------------------------ handshake, delivery, fingerprint


def _install_contract(monkeypatch, profile=None):
    reg = build_registry()
    c = qwen3_5.build(reg, arch="gfx950", profile=profile or qwen3_5.PATH_PROFILE)
    monkeypatch.setattr(process_contract, "_CONTRACT", c)
    monkeypatch.setattr(process_contract, "_VIEW", process_contract.build_contract_view(c, reg))
    return c, reg


def test_handshake_matches_refuses_and_demotes(monkeypatch):
    assert process_contract.contract_hash() is None
    assert process_contract.assert_contract_agreement("anything") is True  # nothing built yet: a recorded skip
    assert enforce.ledger().records[-1].result == enforce.SKIPPED
    c, _ = _install_contract(monkeypatch)
    ours = process_contract.contract_hash()
    assert ours == c.identities.numerical_policy
    assert process_contract.assert_contract_agreement(ours, other_side="engine") is True
    with pytest.raises(RuntimeError, match="MISMATCH"):
        process_contract.assert_contract_agreement("0" * 64, other_side="engine")
    assert enforce.ledger().violations()[-1].obligation_id == "handshake:numerical_policy"
    monkeypatch.setenv("SKYRL_ISOEXEC_MANIFEST_STRICT", "0")
    assert process_contract.assert_contract_agreement("0" * 64) is False
    assert enforce.ledger().status()[("handshake:numerical_policy", enforce.WEIGHT_SYNC)] == enforce.VIOLATION

    class Info:
        contract_hash = None

    assert process_contract.assert_init_info_contract(Info()) is True
    assert enforce.SKIP_NO_PEER_STAMP in enforce.ledger().records[-1].evidence
    Info.contract_hash = ours
    assert process_contract.assert_init_info_contract(Info()) is True
    monkeypatch.setenv("SKYRL_ISOEXEC_MANIFEST_STRICT", "1")
    Info.contract_hash = "f" * 64
    with pytest.raises(RuntimeError):
        process_contract.assert_init_info_contract(Info())


def test_a_one_sided_change_diverges_the_hash(monkeypatch):
    reg = build_registry()
    trainer = qwen3_5.build(reg, arch="gfx950", profile=qwen3_5.PATH_PROFILE)
    engine = qwen3_5.build(reg, arch="gfx950", profile=qwen3_5.PATH_PROFILE.with_overrides(pik_leaves=16))
    monkeypatch.setattr(process_contract, "_CONTRACT", trainer)
    with pytest.raises(RuntimeError, match="MISMATCH"):
        process_contract.assert_contract_agreement(engine.identities.numerical_policy)


def test_extensions_fold_into_the_handshake_hash(monkeypatch):
    c, _ = _install_contract(monkeypatch)
    base = c.identities.numerical_policy
    process_contract.register_contract_extension("lib_abi", lambda: 1)
    import hashlib

    expect = hashlib.sha256(json.dumps({"base": base, "extensions": {"lib_abi": "1"}}, sort_keys=True, separators=(",", ":")).encode()).hexdigest()
    assert process_contract.contract_hash() == expect != base

    def broken():
        raise KeyError("x")

    process_contract.register_contract_extension("broken", broken)
    assert process_contract.contract_hash() not in (expect, base)
    assert process_contract.composite_hash(None) is None


def test_get_process_contract_builds_once_and_writes_the_artifact(monkeypatch, tmp_path):
    import isoexec_amd.core.arch as arch_mod
    import isoexec_amd.models.qwen3_5 as q

    path = tmp_path / "contract.json"
    monkeypatch.setenv("ISOEXEC_CONTRACT_PATH", str(path))
    assert process_contract.get_process_contract() is None
    c = process_contract.get_process_contract("Qwen/Qwen3.5-35B-A3B", arch="gfx950")
    assert process_contract.get_process_contract() is c and process_contract.cached_contract() is c
    assert ("mm", "engine_decode") in process_contract.cached_contract_view()
    assert path.read_bytes() == K.to_canonical_json(c)
    monkeypatch.setenv("ISOEXEC_CONTRACT_HASH", c.identities.numerical_policy)
    assert load_contract(str(path)) == c
    monkeypatch.setenv("ISOEXEC_CONTRACT_HASH", "0" * 64)
    with pytest.raises(ContractDeliveryError, match="cross-check FAILED"):
        load_contract(str(path))
    tampered = json.loads(path.read_bytes())
    tampered["composition"][0]["impl"]["version"] = 99
    path.write_bytes(json.dumps(tampered).encode())
    monkeypatch.delenv("ISOEXEC_CONTRACT_HASH")
    with pytest.raises(ContractDeliveryError, match="do not match the recomputed"):
        load_contract(str(path))
    process_contract._reset_for_tests()
    with pytest.raises(resolve.ResolutionError):
        process_contract.get_process_contract("org/unknown-model", arch="gfx950")
    assert enforce.ledger().violations()[-1].obligation_id == "build_valid:contract"
    assert arch_mod.ARCH == "cpu" or is_accelerator_arch(arch_mod.ARCH)


def test_write_and_validate_against_installed(tmp_path):
    reg = toy_registry()
    c = build(reg, {("core", s): sel("fusedcore") for s in ALL})
    assert write_contract_file(c, str(tmp_path / "c.json")) == c.identities.numerical_policy
    keys = expected_installed_keys(c, reg)
    assert keys == {("core", s) for s in ALL}
    validate_contract_against_installed(c, reg, keys)
    with pytest.raises(ContractDeliveryError, match="UNNAMED"):
        validate_contract_against_installed(c, reg, set(keys) | {("mm", "trainer_fwd")})
    with pytest.raises(ContractDeliveryError, match="NOT installed"):
        validate_contract_against_installed(c, reg, set(keys) - {("core", "engine_decode")})


def test_fingerprint_compares_installs_with_the_contract(monkeypatch):
    _, reg = _install_contract(monkeypatch)
    view = process_contract.cached_contract_view()

    def kernel():
        pass

    fingerprint.record_installs("mm", fingerprint.ALL_SITES, "hip_mfma_batch_invariant", kernel)
    fingerprint.record_install("logprobs.log_softmax", "engine_decode", "hip_rowinv_leaftree", kernel,
                               pinned={"leaves": 8, "block": 4096, "accum": "kahan_fp32"})
    assert fingerprint.log_fingerprint(view) == []
    assert enforce.ledger().status()[("fingerprint:mm:engine_decode", enforce.INSTALL)] == enforce.OK
    assert enforce.ledger().status()[("install_attest:mm:trainer_fwd", enforce.INSTALL)] == enforce.OK
    n = len(enforce.ledger().records)
    fingerprint.record_install("mm", "trainer_fwd", "hip_mfma_batch_invariant", kernel)  # repeated: attested once
    assert len(enforce.ledger().records) == n

    fingerprint.record_install("logprobs.log_softmax", "engine_decode", "hip_rowinv_leaftree", kernel,
                               pinned={"leaves": 4, "block": 4096})
    fingerprint.record_install("norms.rms", "engine_decode", "eager", kernel)
    fingerprint.record_install("attention.varlen", "engine_decode", "x", kernel)
    found = fingerprint.log_fingerprint(view, tag="first_forward")
    assert len(found) == 3
    joined = "\n".join(found)
    assert "leaves: contract pins 8, install used 4" in joined and "accum: contract pins 'kahan_fp32', install recorded nothing" in joined
    assert "contract='hip_fused' but INSTALLED='eager'" in joined and "names no such (op,site)" in joined
    assert enforce.ledger().status()[("fingerprint:norms.rms:engine_decode", enforce.FIRST_FORWARD)] == enforce.VIOLATION
    assert ("gdn.conv", "trainer_fwd") in fingerprint.missing_from_fingerprint(view)
    assert fingerprint.log_fingerprint_once(view, tag="t") != [] and fingerprint.log_fingerprint_once(view, tag="t") == []
    assert fingerprint.pin_disagreements({"a": (1, 2), "b": True}, {"a": [1, 2], "b": 1}) == ["b: contract pins True, install used 1"]
