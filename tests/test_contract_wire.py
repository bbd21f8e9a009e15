"""ExecutionContract: canonical bytes, strict decoding, the three identities, structural rules.

The fixture ``golden/contract_base.json`` restates the small contract the reference's own contract
tests are written against (isoexec/contract/tests/fixtures.py:26-117) in wire form, with blank
identities. The identity checks below hash projections that are spelled out key by key from that raw
JSON (isoexec/contract/identity.py:30-95), never through the implementation under test.
"""

import dataclasses
import hashlib
import json
import os

import pytest

from isoexec_amd import contract as K

HERE = os.path.dirname(__file__)


def raw():
    with open(os.path.join(HERE, "golden", "contract_base.json"), "rb") as fh:
        return json.loads(fh.read())


def canon(plain) -> bytes:
    return json.dumps(plain, sort_keys=True, separators=(",", ":"), ensure_ascii=False).encode("utf-8")


def sha(plain) -> str:
    return hashlib.sha256(canon(plain)).hexdigest()


def base() -> K.ExecutionContract:
    return K.freeze(K.from_canonical_json(canon(raw())))


def swap(c, **kw):
    return K.freeze(dataclasses.replace(c, **kw))


def with_entry(c, idx, **kw):
    comp = list(c.composition)
    comp[idx] = dataclasses.replace(comp[idx], **kw)
    try:
        return swap(c, composition=tuple(comp))
    except K.SerializationError:  # a raw float cannot be hashed; validation reports it instead
        return dataclasses.replace(c, composition=tuple(comp))


# ------------------------------------------------------------------ identities from first principles


def _entry_proj(e):
    return {
        "region": e["region"], "cases": sorted(e["cases"]), "impl": e["impl"], "route": e["route"],
        "constants": e["constants"], "artifact": e["artifact"], "reference": e["reference"],
        "coverage": None if e["coverage"] is None else e["coverage"]["kind"], "discharge": e["discharge"],
    }


def _case_proj(c):
    return dict(c, constraints=sorted(c["constraints"]))


def _expected_identities(d):
    cases = sorted((_case_proj(c) for c in d["cases"]), key=canon)
    fn = {
        "schema_version": d["schema_version"],
        "cases": cases,
        "entries": sorted((_entry_proj(e) for e in d["composition"] if e["half"] == "function"), key=canon),
        "topology": sorted(d["claims"]["topology"], key=canon),
    }
    dep = {
        "entries": sorted((_entry_proj(e) for e in d["composition"] if e["half"] == "deployment"), key=canon),
        "state": sorted(d["claims"]["state"], key=canon),
        "tolerances": sorted(d["claims"]["tolerances"], key=canon),
    }
    sem = {
        "model": dict(d["model"], architectures=sorted(d["model"]["architectures"])),
        "logical_ops": sorted({op for e in d["composition"] for op in e["region"]}),
        "cases": cases,
    }
    return sha(sem), sha(fn), sha(dep)


def test_identities_equal_the_closed_form():
    ids = base().identities
    assert (ids.semantic, ids.numerical_policy, ids.deployment) == _expected_identities(raw())


def test_identity_projection_details():
    # The half field is not hashed, coverage contributes its kind only, cases and constraints sort.
    d = raw()
    fn = K.function_half(base())
    assert all("half" not in e for e in fn["entries"])
    assert {e["coverage"] for e in fn["entries"]} == {None, "enumerated_shapes"}
    assert [c["id"] for c in fn["cases"]] != [c["id"] for c in d["cases"]]
    decode = next(c for c in fn["cases"] if c["id"] == "engine_decode")
    assert decode["constraints"] == ["address_stable", "cudagraph_capturable", "host_free"]
    assert K.semantic_inputs(base())["logical_ops"] == sorted(
        ["moe.combine", "gdn.core", "gdn.gating", "norms.l2", "moe.weights", "moe.gate_scale", "collectives.nccl_pin"]
    )


# ------------------------------------------------------------------ byte form


def test_canonical_bytes_are_sorted_compact_utf8():
    c = base()
    data = K.to_canonical_json(c)
    expect = raw()
    expect["identities"] = dataclasses.asdict(c.identities)
    assert data == canon(expect)
    assert b" " not in data.replace(b"ledger v10 shapes", b"")
    assert K.canonical_bytes({"b": "é", "a": [1, True, None]}) == '{"a":[1,true,null],"b":"é"}'.encode("utf-8")


def test_round_trip_is_byte_stable():
    c = base()
    once = K.to_canonical_json(c)
    again = K.from_canonical_json(once)
    assert again == c and K.to_canonical_json(again) == once


def _mutated(fn):
    d = json.loads(K.to_canonical_json(base()))
    fn(d)
    return canon(d)


def test_unknown_fields_refuse_at_every_level():
    for poke in (
        lambda d: d.__setitem__("extra", 1),
        lambda d: d["composition"][0].__setitem__("evidence", "x"),
        lambda d: d["composition"][0]["impl"].__setitem__("build", "x"),
        lambda d: d["claims"].__setitem__("other", []),
        lambda d: d["cases"][0].__setitem__("note", "x"),
        lambda d: d["composition"][4]["constants"]["scale"].__setitem__("unit", "x"),
    ):
        with pytest.raises(K.UnknownFieldError):
            K.from_canonical_json(_mutated(poke))


def test_missing_field_refuses():
    with pytest.raises(K.SerializationError):
        K.from_canonical_json(_mutated(lambda d: d["composition"][0].pop("half")))
    with pytest.raises(K.SerializationError):
        K.from_canonical_json(_mutated(lambda d: d["claims"]["tolerances"][0].__setitem__("case_pair", ["a"])))


def test_floats_refuse_both_ways():
    data = K.to_canonical_json(base()).replace(b'"leaves":4', b'"leaves":4.0')
    with pytest.raises(K.SerializationError, match="float"):
        K.from_canonical_json(data)
    with pytest.raises(K.SerializationError, match="float"):
        K.from_canonical_json(K.to_canonical_json(base()).replace(b'"leaves":4', b'"leaves":NaN'))
    c = base()
    entry0 = dataclasses.replace(c.composition[0], constants={"leaves": 4, "scale": 0.5})
    leaky = dataclasses.replace(c, composition=(entry0,) + c.composition[1:])
    with pytest.raises(K.SerializationError, match=r"\$\.composition\[0\]\.constants\.scale"):
        K.to_canonical_json(leaky)


@pytest.mark.parametrize("version", ["1", "3", ""])
def test_other_schema_versions_refuse(version):
    with pytest.raises(K.SerializationError, match="schema_version"):
        K.from_canonical_json(_mutated(lambda d: d.__setitem__("schema_version", version)))


# ------------------------------------------------------------------ what rotates which identity


def test_function_half_changes_rotate_numerical_policy_only():
    c = base()
    for changed in (
        with_entry(c, 0, constants={"leaves": 8, "leaf_dtype": "fp32"}),
        with_entry(c, 1, impl=K.ImplRef("native_fused_sigmoid", 2, "sm90")),
        with_entry(c, 1, impl=K.ImplRef("native_fused_sigmoid", 1, "gfx950")),
        with_entry(c, 1, route="canonical"),
        with_entry(c, 4, coverage=K.Coverage("symbolic_domain", "ledger v10 shapes")),
        with_entry(c, 0, artifact="sha256:00000000"),
    ):
        assert changed.identities.numerical_policy != c.identities.numerical_policy
        assert changed.identities.semantic == c.identities.semantic
        assert changed.identities.deployment == c.identities.deployment


def test_repartition_rotates_policy_but_not_semantics():
    c = base()
    comp = list(c.composition)
    fused = comp[1]
    comp[1:2] = [
        dataclasses.replace(fused, region=("gdn.core", "gdn.gating")),
        dataclasses.replace(fused, region=("norms.l2",), impl=K.ImplRef("eager_l2", 1, "sm90")),
    ]
    split = swap(c, composition=tuple(comp))
    assert split.identities.semantic == c.identities.semantic
    assert split.identities.numerical_policy != c.identities.numerical_policy


def test_deployment_changes_leave_numerical_policy_alone():
    c = base()
    moved = with_entry(c, 5, impl=K.ImplRef("nccl_pinned", 1, "sm90"))
    looser = swap(c, claims=dataclasses.replace(c.claims, tolerances=(
        K.ToleranceClaim(("engine_decode", "trainer_score"), {"mean": "1e-5", "max": "5e-6"}),)))
    for changed in (moved, looser):
        assert changed.identities.numerical_policy == c.identities.numerical_policy
        assert changed.identities.deployment != c.identities.deployment


def test_topology_claims_are_function_half():
    c = base()
    wider = swap(c, claims=dataclasses.replace(c.claims, topology=(
        K.TopologyClaim("TP", "invariant", domain=(1, 2, 4, 8), proof="gates/tp_invariance"),) + c.claims.topology[1:]))
    assert wider.identities.numerical_policy != c.identities.numerical_policy
    assert wider.identities.deployment == c.identities.deployment


def test_orderings_and_prose_rotate_nothing():
    c = base()
    same = (
        swap(c, composition=tuple(reversed(c.composition))),
        swap(c, cases=tuple(reversed(c.cases))),
        with_entry(c, 0, cases=tuple(reversed(c.composition[0].cases))),
        with_entry(c, 4, coverage=K.Coverage("enumerated_shapes", "a different sentence")),
        swap(c, claims=dataclasses.replace(c.claims, topology=tuple(reversed(c.claims.topology)))),
        swap(c, cases=tuple(dataclasses.replace(x, constraints=tuple(reversed(x.constraints))) for x in c.cases)),
    )
    for other in same:
        assert other.identities == c.identities


def test_case_conditions_rotate_semantic_and_policy():
    c = base()
    cases = tuple(dataclasses.replace(x, grad_mode="grad") if x.id == "trainer_score" else x for x in c.cases)
    changed = swap(c, cases=cases)
    assert changed.identities.semantic != c.identities.semantic
    assert changed.identities.numerical_policy != c.identities.numerical_policy
    dropped = swap(c, cases=tuple(dataclasses.replace(x, constraints=x.constraints[:1]) for x in c.cases))
    assert dropped.identities.numerical_policy != c.identities.numerical_policy


def test_stored_identities_are_ignored_by_recomputation():
    c = base()
    forged = dataclasses.replace(c, identities=K.Identities("a", "b", "c"))
    assert K.compute_identities(forged) == c.identities
    assert "stored identities do not match recomputed identities" in K.validate(forged)


# ------------------------------------------------------------------ structural rules

REQUIRED = {cid: frozenset({"moe.combine", "gdn.core", "moe.weights"}) for cid in
            ("engine_decode", "engine_prefill", "trainer_fwd", "trainer_recompute", "trainer_score")}


def problems(c, required=None):
    return "; ".join(K.validate(c, required))


def test_fixture_is_valid():
    assert K.validate(base(), REQUIRED) == []
    K.validate_or_raise(base(), REQUIRED)


def test_ownership_and_coverage():
    c = base()
    thief = K.CompositionEntry(("gdn.gating",), ("trainer_fwd",), K.ImplRef("eager", 1, "sm90"), "canonical")
    assert "owned by both" in problems(swap(c, composition=c.composition + (thief,)))
    gap = swap(c, composition=c.composition[1:])
    assert "uncovered required op(s) ['moe.combine']" in problems(gap, REQUIRED)
    twice = dataclasses.replace(c.composition[0], cases=("trainer_fwd",))
    assert "duplicate (region, case) claim" in problems(swap(c, composition=c.composition + (twice,)))


def test_entry_rules():
    c = base()
    assert "asymmetric region requires a discharge" in problems(with_entry(c, 2, discharge=None))
    assert "requires a neutrality_proof" in problems(with_entry(c, 5, discharge=None))
    assert "requires a neutrality_proof" in problems(
        with_entry(c, 5, discharge=K.EquivalenceProof("equivalence_proof", "gates/x")))
    assert "composition_defining requires an artifact" in problems(with_entry(c, 0, artifact=None))
    assert "reference_preserving requires a reference" in problems(with_entry(c, 4, reference=None))
    assert "invalid bit pattern" in problems(with_entry(c, 4, constants={"scale": K.BitPattern("3f800000", "fp32")}))
    assert "is a raw float" in problems(with_entry(c, 0, constants={"leaves": 4.0}))
    assert "unknown case 'engine_warmup'" in problems(with_entry(c, 0, cases=("engine_warmup",)))
    assert "region tuple must be sorted" in problems(with_entry(c, 1, region=("norms.l2", "gdn.core")))
    assert "empty region" in problems(with_entry(c, 1, region=()))
    assert "unknown route" in problems(with_entry(c, 1, route="fast"))
    assert "unknown half" in problems(with_entry(c, 1, half="both"))
    assert "discharge with an empty ref" in problems(with_entry(c, 2, discharge=K.EquivalenceProof("equivalence_proof", " ")))
    assert "unknown discharge kind" in problems(with_entry(c, 2, discharge=K.EquivalenceProof("vibes", "x")))
    assert "unknown coverage kind" in problems(with_entry(c, 4, coverage=K.Coverage("some", "x")))
    assert "empty composition" in problems(swap(c, composition=()))
    assert "duplicate case ids" in problems(swap(c, cases=c.cases + (c.cases[0],)))
    assert "unsupported schema_version" in problems(swap(c, schema_version="9"))


def test_claim_rules():
    c = base()

    def topo(*claims):
        return swap(c, claims=dataclasses.replace(c.claims, topology=claims))

    assert "duplicate topology axes" in problems(topo(*c.claims.topology, c.claims.topology[1]))
    assert "pinned requires degree and collective_plan" in problems(topo(K.TopologyClaim("PP", "pinned", degree=1)))
    assert "not a deployable degree" in problems(topo(K.TopologyClaim("PP", "pinned", degree=0, collective_plan="none")))
    assert "invariant requires a non-empty domain and a proof" in problems(topo(K.TopologyClaim("TP", "invariant", domain=(1, 2))))
    assert "tautology" in problems(topo(K.TopologyClaim("TP", "invariant", domain=(4, 4), proof="gates/x")))
    assert "empty proof ref" in problems(topo(K.TopologyClaim("PP", "pinned", degree=1, collective_plan="none", proof=" ")))
    assert "unknown kind" in problems(topo(K.TopologyClaim("PP", "elastic")))

    def tol(**kw):
        t = dataclasses.replace(c.claims.tolerances[0], **kw)
        return swap(c, claims=dataclasses.replace(c.claims, tolerances=(t,)))

    for text in ("nan", "inf", "-inf", "tight"):
        assert "not a finite threshold" in problems(tol(bounds={"max": text}))
    assert "no bounds" in problems(tol(bounds={}))
    assert "unknown case 'engine_x'" in problems(tol(case_pair=("engine_x", "trainer_score")))

    def state(**kw):
        s = dataclasses.replace(c.claims.state[0], **kw)
        return swap(c, claims=dataclasses.replace(c.claims, state=(s,)))

    assert "unknown lifecycle event(s) ['reboot']" in problems(state(invalidated_by=("weight_sync", "reboot")))
    assert "empty invalidated_by" in problems(state(invalidated_by=()))
    assert "empty ref" in problems(state(ref=" "))
    with pytest.raises(K.ValidationError):
        K.validate_or_raise(state(ref=""))
