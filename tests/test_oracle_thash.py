"""Pins the CPU restatement of the order-invariant digest (oracle/thash.py) without reference to itself:
the published splitmix64 stream, a one-element-at-a-time sum in Python integers, what a ladder rung means, and the
vectors the reference's own eager implementation produced (tests/golden/thash_vectors.json)."""

import json
import os

import numpy as np
import pytest

from oracle import thash as OT

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "thash_vectors.json")) as _fh:
    VECTORS = json.load(_fh)["cases"]


def image_array(case) -> np.ndarray:
    return np.array(case["image"], dtype=getattr(np, OT.DTYPES[case["dtype"]][0])).reshape(-1)


def test_mix64_is_the_splitmix64_finaliser():
    # splitmix64 seeded with 0 returns mix64(n * GOLDEN) for n = 1, 2, 3: its published first outputs
    published = (0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F)
    assert tuple(OT.mix64(n * OT.GOLDEN) for n in (1, 2, 3)) == published


def test_weights_are_odd_and_differ_inside_a_group():
    w = OT.weights(0, 64, OT.salt_of(0))
    assert all(int(v) & 1 for v in w)
    assert len({int(v) for v in w}) == 64
    # the stream is keyed by absolute position: a window is a slice of the whole
    assert np.array_equal(OT.weights(24, 16, OT.salt_of(7)), OT.weights(0, 64, OT.salt_of(7))[24:40])


def slow_sum(values, mask, salt):
    total = 0
    for i, v in enumerate(values):
        w = ((OT.mix64((i >> 3) ^ salt) ^ ((i & 7) * OT.GOLDEN)) & OT.U64) | 1
        total = (total + ((v & OT.U64) & mask) * w) & OT.U64
    return total


@pytest.mark.parametrize("np_dtype", ["int8", "uint8", "int16", "int32", "int64"])
def test_weighted_sum_against_python_integers(np_dtype):
    rng = np.random.default_rng(5)
    info = np.iinfo(np_dtype)
    for count in (0, 1, 7, 8, 9, 1000):
        iv = rng.integers(info.min, info.max, size=count, dtype=np_dtype, endpoint=True)
        masks = [OT.U64, 0xFFFF, 0xFF80, 0xFFFFFFFFFFFF0000]
        salt = OT.salt_of(3)
        want = [slow_sum([int(v) for v in iv], m, salt) for m in masks]
        assert OT.weighted_sums(iv, masks, salt) == want
        assert OT.weighted_sums(iv, masks, salt, chunk=13) == want     # chunking cannot matter


def test_sign_extension_is_undone_by_the_width_mask():
    signed = np.array([-1, -128, 5], dtype=np.int8)
    unsigned = signed.view(np.uint8)
    salt = OT.salt_of(0)
    assert OT.weighted_sums(signed, [0xFF], salt) == OT.weighted_sums(unsigned, [0xFF], salt)
    assert OT.weighted_sums(signed, [OT.U64], salt) != OT.weighted_sums(unsigned, [OT.U64], salt)


def test_a_rung_keeps_the_top_k_mantissa_bits():
    rng = np.random.default_rng(9)
    base = (rng.integers(0x3F00, 0x3F7F, size=50)).astype(np.int16)       # bf16 values in [0.5, 1)
    la = OT.digest_ladder(base, "bfloat16", (50,))
    assert set(la) == {"full", "k6", "k4", "k2", "k0"}
    for bit in range(7):
        other = base.copy()
        other[7] ^= 1 << bit
        lb = OT.digest_ladder(other, "bfloat16", (50,))
        assert la["full"] != lb["full"]
        matched = [k for k in (6, 4, 2, 0) if la[f"k{k}"] == lb[f"k{k}"]]
        assert matched == [k for k in (6, 4, 2, 0) if bit < 7 - k], bit


def test_shape_dtype_seed_and_level_reach_the_digest():
    iv = np.arange(48, dtype=np.int32)
    d = OT.tensor_digest(iv, "float32", (6, 8))
    assert d != OT.tensor_digest(iv, "float32", (8, 6))
    assert d != OT.tensor_digest(iv, "float32", (48,))
    assert d != OT.tensor_digest(iv, "int32", (6, 8))
    assert d != OT.tensor_digest(iv, "float32", (6, 8), seed=1)
    assert d != OT.tensor_digest(iv, "float32", (6, 8), k=22)      # low bits are zero here: only the header moved
    swapped = iv.copy()
    swapped[[0, 1]] = swapped[[1, 0]]
    assert d != OT.tensor_digest(swapped, "float32", (6, 8))


def test_a_changed_row_moves_its_segment_only():
    rng = np.random.default_rng(2)
    a = rng.integers(-2**31, 2**31 - 1, size=(16, 32), dtype=np.int32)
    b = a.copy()
    b[5, 7] ^= 4
    sa = OT.segment_digests(a, "float32", (16, 32), rows_per_segment=4)
    sb = OT.segment_digests(b, "float32", (16, 32), rows_per_segment=4)
    assert len(sa) == 4 and [i for i in range(4) if sa[i] != sb[i]] == [1]
    # the first axis with more than one row is the one cut
    assert OT.segment_axis((1, 64, 4, 8)) == 1 and OT.segment_axis((64, 1, 9)) == 0 and OT.segment_axis((1, 1)) == 0
    assert len(OT.segment_digests(np.zeros(64 * 32, np.int32), "float32", (1, 64, 4, 8), rows_per_segment=16)) == 4


def test_reference_vectors():
    assert len(VECTORS) > 50
    seen = set()
    for case in VECTORS:
        iv, name, shape, seed = image_array(case), case["dtype"], tuple(case["shape"]), case["seed"]
        seen.add(name)
        assert f"{OT.tensor_digest(iv, name, shape, seed=seed):016x}" == case["digest"], (name, shape)
        assert OT.digest_ladder(iv, name, shape, seed=seed) == case["ladder"], (name, shape)
        for rps, want in case["segments"].items():
            assert OT.segment_digests(iv, name, shape, rows_per_segment=int(rps), seed=seed) == want, (name, shape, rps)
        if "segments_k2" in case:
            assert OT.segment_digests(iv, name, shape, rows_per_segment=2, k=2, seed=seed) == case["segments_k2"]
    assert {"bfloat16", "float16", "float32", "float64", "int8", "uint8", "int64", "bool", "complex64"} <= seen
