"""Writes tests/golden/contract_vectors.json: canonical JSON texts of execution contracts and the three identity
hashes the REFERENCE's own contract package gives them.

Run once, in the build container (the reference tree is not present anywhere else):

    python tests/golden/make_contract_vectors.py

It loads the reference's ``isoexec/contract`` directory (types, serialize, identity, validate: standard library only)
as a stand-alone package by path, so nothing else of the reference is imported. The base contract is this repository's
wire-form fixture ``contract_base.json`` (the small contract of isoexec/contract/tests/fixtures.py:27-117), decoded by
the reference's ``from_canonical_json``; each variant is one ``dataclasses.replace`` away from it. For every variant
the fixture keeps data only: its name, which identities the variant must rotate relative to the base, the reference's
``to_canonical_json`` text, the reference's ``compute_identities`` strings and, for two of them, the canonical text of
the three hashed projections (so a mismatch can be located). These vectors pin the conventions no mathematics fixes: field sets, key
order, what is projected out, how cases / constraints / entries sort, how constants are encoded.
"""

from __future__ import annotations

import dataclasses
import importlib.util
import json
import os
import sys

REFERENCE_DIR = "/root/reference/skyrl/backends/skyrl_train/isoexec/contract"
HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "contract_vectors.json")


def load_reference_package():
    spec = importlib.util.spec_from_file_location("reference_contract", os.path.join(REFERENCE_DIR, "__init__.py"),
                                                  submodule_search_locations=[REFERENCE_DIR])
    module = importlib.util.module_from_spec(spec)
    sys.modules["reference_contract"] = module
    spec.loader.exec_module(module)
    return module


def main() -> int:
    R = load_reference_package()
    with open(os.path.join(HERE, "contract_base.json"), "rb") as fh:
        base = R.from_canonical_json(json.dumps(json.loads(fh.read()), sort_keys=True, separators=(",", ":"),
                                                 ensure_ascii=False).encode("utf-8"))
    rep = dataclasses.replace

    def entry(c, i, **kw):
        comp = list(c.composition)
        comp[i] = rep(comp[i], **kw)
        return rep(c, composition=tuple(comp))

    def case(c, i, **kw):
        cases = list(c.cases)
        cases[i] = rep(cases[i], **kw)
        return rep(c, cases=tuple(cases))

    ImplRef, BitPattern, Coverage, Claims = R.ImplRef, R.BitPattern, R.Coverage, R.Claims
    variants = [
        ("base", base, []),
        # --- must rotate numerical_policy only
        ("constant_changed", entry(base, 0, constants={"leaves": 8, "leaf_dtype": "fp32"}), ["numerical_policy"]),
        ("bit_pattern_changed", entry(base, 4, constants={"scale": BitPattern("0x3f000000", "fp32")}),
         ["numerical_policy"]),
        ("impl_version_changed", entry(base, 1, impl=ImplRef("native_fused_sigmoid", 2, "sm90")), ["numerical_policy"]),
        ("impl_arch_changed", entry(base, 1, impl=ImplRef("native_fused_sigmoid", 1, "gfx950")), ["numerical_policy"]),
        ("route_changed", entry(base, 1, route="canonical"), ["numerical_policy"]),
        ("artifact_changed", entry(base, 0, artifact="sha256:00000000"), ["numerical_policy"]),
        ("coverage_kind_changed", entry(base, 4, coverage=Coverage("symbolic_domain", "ledger v10 shapes")),
         ["numerical_policy"]),
        ("topology_degree_changed",
         rep(base, claims=rep(base.claims, topology=(rep(base.claims.topology[0], domain=(1, 2, 4, 8)),)
                              + base.claims.topology[1:])), ["numerical_policy"]),
        ("entry_cases_narrowed", entry(base, 0, cases=("trainer_fwd", "engine_decode")), ["numerical_policy"]),
        # --- semantic + numerical_policy (case conditions and the op vocabulary enter both)
        ("case_constraint_dropped", case(base, 4, constraints=("host_free", "address_stable")),
         ["semantic", "numerical_policy"]),
        ("case_shape_domain_changed", case(base, 3, shape_domain="padded"), ["semantic", "numerical_policy"]),
        ("region_repartitioned",
         rep(base, composition=(base.composition[0], rep(base.composition[1], region=("gdn.core", "gdn.gating")),
                                rep(base.composition[1], region=("norms.l2",))) + base.composition[2:]),
         ["numerical_policy"]),
        ("logical_op_renamed", entry(base, 0, region=("moe.combine_v2",)), ["semantic", "numerical_policy"]),
        ("model_architecture_added",
         rep(base, model=rep(base.model, architectures=("Qwen3_5MoeForConditionalGeneration", "Another"))),
         ["semantic"]),
        # --- deployment only
        ("deployment_entry_changed", entry(base, 5, impl=ImplRef("nccl_pinned", 1, "sm90")), ["deployment"]),
        ("tolerance_changed",
         rep(base, claims=rep(base.claims, tolerances=(rep(base.claims.tolerances[0],
                                                           bounds={"mean": "2e-6", "max": "5e-6"}),))),
         ["deployment"]),
        ("state_claim_changed",
         rep(base, claims=rep(base.claims, state=(rep(base.claims.state[0], invalidated_by=("weight_sync",)),))),
         ["deployment"]),
        ("half_moved_to_deployment", entry(base, 1, half="deployment"), ["numerical_policy", "deployment"]),
        # --- must rotate nothing
        ("entries_reordered", rep(base, composition=tuple(reversed(base.composition))), []),
        ("cases_reordered", rep(base, cases=tuple(reversed(base.cases))), []),
        ("entry_case_list_reordered", entry(base, 0, cases=tuple(reversed(base.composition[0].cases))), []),
        ("constraints_reordered", case(base, 4, constraints=("address_stable", "host_free", "cudagraph_capturable")),
         []),
        ("coverage_description_edited", entry(base, 4, coverage=Coverage("enumerated_shapes", "ledger v11 shapes")),
         []),
        ("claims_emptied", rep(base, claims=Claims()), ["numerical_policy", "deployment"]),
        ("non_ascii_text", entry(base, 4, coverage=Coverage("enumerated_shapes", "förmen ≤ 512 · 形状")), []),
    ]

    base_ids = R.compute_identities(base)
    records = []
    for name, contract, rotates in variants:
        ids = R.compute_identities(contract)
        frozen = rep(contract, identities=ids)
        text = R.to_canonical_json(frozen)
        if isinstance(text, bytes):
            text = text.decode("utf-8")
        again = R.to_canonical_json(R.from_canonical_json(text.encode("utf-8")))
        again = again.decode("utf-8") if isinstance(again, bytes) else again
        assert again == text, name                               # the reference's own round trip is byte-stable
        moved = [k for k in ("semantic", "numerical_policy", "deployment") if getattr(ids, k) != getattr(base_ids, k)]
        assert sorted(moved) == sorted(rotates), (name, moved, rotates)   # the reference rotates what we said it does
        record = {"name": name, "rotates": rotates, "canonical_json": text,
                  "identities": {"semantic": ids.semantic, "numerical_policy": ids.numerical_policy,
                                 "deployment": ids.deployment}}
        if name in ("base", "non_ascii_text"):   # the hashed projections themselves, where a mismatch is easiest to read
            record["projections"] = {
                "semantic": R.serialize.canonical_bytes(R.semantic_inputs(contract)).decode("utf-8"),
                "numerical_policy": R.serialize.canonical_bytes(R.function_half(contract)).decode("utf-8"),
                "deployment": R.serialize.canonical_bytes(R.deployment_half(contract)).decode("utf-8")}
        records.append(record)
    with open(OUT, "w", encoding="utf-8") as fh:
        json.dump({"made_by": "tests/golden/make_contract_vectors.py", "vectors": records}, fh, ensure_ascii=False,
                  indent=0)
    print(f"{len(records)} vectors -> {OUT} ({os.path.getsize(OUT)} bytes)")
    return 0


if __name__ == "__main__":
    sys.exit(main())
