"""The contract's canonical bytes and its three identities against what the reference's own ``isoexec/contract``
package produced (``golden/contract_vectors.json``, written once in the build container by
``golden/make_contract_vectors.py``: 26 contracts, each one edit away from the small contract of the reference's
contract tests). This package must decode every text, re-encode it to the same bytes, and hash it to the same three
strings (isoexec/contract/serialize.py:45-48, identity.py:30-106)."""

import json
import os

import pytest

from isoexec_amd import contract as K

HERE = os.path.dirname(__file__)
with open(os.path.join(HERE, "golden", "contract_vectors.json"), encoding="utf-8") as _fh:
    VECTORS = json.load(_fh)["vectors"]
BY_NAME = {v["name"]: v for v in VECTORS}


@pytest.mark.parametrize("vector", VECTORS, ids=[v["name"] for v in VECTORS])
def test_bytes_and_identities_equal_the_reference(vector):
    data = vector["canonical_json"].encode("utf-8")
    contract = K.from_canonical_json(data)
    assert K.to_canonical_json(contract) == data
    ids = K.compute_identities(contract)
    assert {"semantic": ids.semantic, "numerical_policy": ids.numerical_policy,
            "deployment": ids.deployment} == vector["identities"]
    assert contract.identities == ids            # the stored field is what the content hashes to


@pytest.mark.parametrize("name", ["base", "non_ascii_text"])
def test_hashed_projections_equal_the_reference_text(name):
    vector = BY_NAME[name]
    contract = K.from_canonical_json(vector["canonical_json"].encode("utf-8"))
    for key, view in (("semantic", K.semantic_inputs), ("numerical_policy", K.function_half),
                      ("deployment", K.deployment_half)):
        assert K.canonical_bytes(view(contract)).decode("utf-8") == vector["projections"][key], key


def test_the_vectors_cover_every_rotation_class():
    base = BY_NAME["base"]["identities"]
    seen = set()
    for vector in VECTORS:
        moved = tuple(k for k in ("semantic", "numerical_policy", "deployment") if vector["identities"][k] != base[k])
        assert sorted(moved) == sorted(vector["rotates"]), vector["name"]
        seen.add(moved)
    assert {(), ("numerical_policy",), ("semantic",), ("deployment",), ("semantic", "numerical_policy"),
            ("numerical_policy", "deployment")} <= seen


def test_fixture_base_is_the_wire_fixture_of_the_other_contract_tests():
    with open(os.path.join(HERE, "golden", "contract_base.json"), "rb") as fh:
        raw = json.loads(fh.read())
    ours = K.freeze(K.from_canonical_json(json.dumps(raw, sort_keys=True, separators=(",", ":")).encode("utf-8")))
    assert K.to_canonical_json(ours).decode("utf-8") == BY_NAME["base"]["canonical_json"]
