"""Writes tests/golden/thash_vectors.json: inputs and the digests the REFERENCE's eager implementation gives them.

Run once, in the build container (the reference tree is not present anywhere else):

    python tests/golden/make_thash_vectors.py

It loads the single file isoexec/debug/thash.py by path (torch only; the triton twin is never reached because the
backend is forced to "eager") and calls tensor_digest / digest_ladder / segment_digests on small tensors whose
integer images come from a fixed linear congruential sequence, so that the fixture holds data only: the dtype name,
the shape, the integer image and what the reference returned. These vectors pin the conventions no mathematics
fixes: dtype codes, header mixing, salts, the segment scheme.
"""

from __future__ import annotations

import importlib.util
import json
import os
import sys

import torch

REFERENCE_FILE = "/root/reference/skyrl/backends/skyrl_train/isoexec/debug/thash.py"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "thash_vectors.json")

VIEW = {"bfloat16": torch.int16, "float16": torch.int16, "float32": torch.int32, "float64": torch.int64,
        "int8": torch.int8, "uint8": torch.uint8, "int16": torch.int16, "int32": torch.int32, "int64": torch.int64,
        "bool": torch.uint8, "float8_e4m3fn": torch.int8, "float8_e5m2": torch.int8, "uint16": torch.int16,
        "uint32": torch.int32, "complex64": torch.int64}
BITS = {torch.int8: 8, torch.uint8: 8, torch.int16: 16, torch.int32: 32, torch.int64: 64}


def image(count: int, view: torch.dtype, start: int) -> list:
    """``count`` integers of the view's width from x <- x * 6364136223846793005 + 1442695040888963407 (mod 2^64),
    taking the top bits of each state."""
    bits, state, out = BITS[view], start, []
    for _ in range(count):
        state = (state * 6364136223846793005 + 1442695040888963407) & ((1 << 64) - 1)
        value = state >> (64 - bits)
        if view != torch.uint8 and value >= 1 << (bits - 1):
            value -= 1 << bits
        out.append(value)
    return out


def tensor_of(name: str, shape, ints):
    view = VIEW[name]
    flat = torch.tensor(ints, dtype=view)
    if name == "bool":
        return (flat & 1).to(torch.bool).reshape(shape)
    return flat.view(getattr(torch, name)).reshape(shape)


def main() -> int:
    os.environ["SKYRL_ISOEXEC_DEBUG_DIGEST"] = "eager"
    spec = importlib.util.spec_from_file_location("reference_thash", REFERENCE_FILE)
    thash = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(thash)

    cases = []
    every_shape = [(), (1,), (7,), (9,), (3, 1, 1), (1, 5, 3), (13, 11), (0, 8), (1, 19, 2, 4)]
    few_shapes = [(9,), (1, 5, 3)]
    for number, name in enumerate(VIEW):
        for shape in (every_shape if name in ("bfloat16", "float32", "int64") else few_shapes):
            count = 1
            for extent in shape:
                count *= extent
            ints = image(count, VIEW[name], start=1000 * number + len(shape) + count)
            if name == "bool":
                ints = [v & 1 for v in ints]
            t = tensor_of(name, shape, ints)
            for seed in ((0, 12345) if shape == (9,) else (number,)):
                case = {"dtype": name, "shape": list(shape), "image": ints, "seed": seed,
                        "digest": f"{thash.tensor_digest(t, seed=seed):016x}",
                        "ladder": thash.digest_ladder(t, seed=seed),
                        "segments": {str(rps): thash.segment_digests(t, rows_per_segment=rps, seed=seed)
                                     for rps in (1, 3, 64)}}
                if thash.mantissa_bits(t.dtype) is not None:
                    case["segments_k2"] = thash.segment_digests(t, rows_per_segment=2, k=2, seed=seed)
                cases.append(case)
    with open(OUT, "w") as fh:
        json.dump({"made_by": "tests/golden/make_thash_vectors.py", "cases": cases}, fh, separators=(",", ":"))
    print(f"{len(cases)} cases -> {OUT} ({os.path.getsize(OUT)} bytes)")
    return 0


if __name__ == "__main__":
    sys.exit(main())
