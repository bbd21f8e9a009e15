"""CPU restatement of the reference's order-invariant tensor digest (isoexec/debug/thash.py).

TEST INFRASTRUCTURE ONLY (see the package docstring).

    body   = SUM_i (x_i & mask) * w_i  mod 2**64          thash.py:1-6, 180-196
    w_i    = (mix64((i >> 3) ^ salt) ^ ((i & 7) * GOLDEN)) | 1     thash.py:174-177
    salt   = mix64(seed) ^ GOLDEN                          thash.py:170-171
    digest = mix64(body ^ header(shape, dtype, kept bits, seed))   thash.py:222-248
    segment s of seg_numel elements: positions from the segment's start,
             salt from seed ^ mix64(s * seg_numel + 1), header further mixed with s + 1     thash.py:319-354

``x_i`` is the element's bit pattern read as a same-size signed integer and widened to 64 bits; ``mask`` is the
element width's all-ones (which undoes the sign extension) with the low ``mantissa_bits - k`` bits cleared when a
truncation level ``k`` is asked for (thash.py:155-167).

The functions take the INTEGER IMAGE of a tensor as a numpy array plus the dtype's name and the logical shape, so
that nothing here depends on torch. Arithmetic is numpy uint64 (which wraps) for the sums and Python ints for the
scalar mixing.

How it is pinned, independently of this restatement (tests/test_oracle_thash.py):
  * ``mix64`` against the published first outputs of splitmix64 seeded with 0;
  * the weighted sum against a sum written with Python integers, one element at a time;
  * the masks through what a rung MEANS: flipping mantissa bit b changes exactly the rungs k > 7 - 1 - b of a bf16
    ladder (thash's own test states this expectation: debug/tests/test_thash_cpu.py:116-131);
  * header, dtype codes, salts and the segment scheme -- plain conventions that no mathematics fixes -- against
    vectors written once by the reference's own eager implementation (tests/golden/thash_vectors.json, made by
    tests/golden/make_thash_vectors.py).
"""

from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

U64 = (1 << 64) - 1
GOLDEN = 0x9E3779B97F4A7C15
MIX1 = 0xBF58476D1CE4E5B9
MIX2 = 0x94D049BB133111EB

# name -> (integer view, unsigned mask or None for 64 bits, explicit mantissa bits or None, code in the header)
# The codes are the 1-based positions in the reference's table (thash.py:27-59, 218).
DTYPES: Dict[str, Tuple[str, Optional[int], Optional[int], int]] = {
    "bfloat16": ("int16", 0xFFFF, 7, 1),
    "float16": ("int16", 0xFFFF, 10, 2),
    "float32": ("int32", 0xFFFFFFFF, 23, 3),
    "float64": ("int64", None, 52, 4),
    "int8": ("int8", 0xFF, None, 5),
    "uint8": ("uint8", 0xFF, None, 6),
    "int16": ("int16", 0xFFFF, None, 7),
    "int32": ("int32", 0xFFFFFFFF, None, 8),
    "int64": ("int64", None, None, 9),
    "bool": ("uint8", 0x1, None, 10),
    "float8_e4m3fn": ("int8", 0xFF, 3, 11),
    "float8_e5m2": ("int8", 0xFF, 2, 12),
    "float8_e4m3fnuz": ("int8", 0xFF, 3, 13),
    "float8_e5m2fnuz": ("int8", 0xFF, 2, 14),
    "uint16": ("int16", 0xFFFF, None, 15),
    "uint32": ("int32", 0xFFFFFFFF, None, 16),
    "uint64": ("int64", None, None, 17),
    "complex64": ("int64", None, None, 18),
    "complex128": ("int64", None, None, 19),
}

LADDERS = {2: (1, 0), 3: (2, 1, 0), 7: (6, 4, 2, 0), 10: (9, 7, 5, 3, 1, 0), 23: (22, 18, 14, 10, 6, 2, 0),
           52: (48, 40, 32, 24, 16, 8, 0)}


def mix64(z: int) -> int:
    """The splitmix64 finaliser (thash.py:100-105)."""
    z &= U64
    z = ((z ^ (z >> 30)) * MIX1) & U64
    z = ((z ^ (z >> 27)) * MIX2) & U64
    return z ^ (z >> 31)


def _mix64_np(z: np.ndarray) -> np.ndarray:
    z = z ^ (z >> np.uint64(30))
    z = z * np.uint64(MIX1)
    z = z ^ (z >> np.uint64(27))
    z = z * np.uint64(MIX2)
    return z ^ (z >> np.uint64(31))


def salt_of(seed: int) -> int:
    return mix64(seed) ^ GOLDEN


def weights(first: int, count: int, salt: int) -> np.ndarray:
    """w_i for i = first .. first+count-1."""
    idx = np.arange(first, first + count, dtype=np.uint64)
    base = _mix64_np((idx >> np.uint64(3)) ^ np.uint64(salt))
    return (base ^ ((idx & np.uint64(7)) * np.uint64(GOLDEN))) | np.uint64(1)


def and_mask(dtype: str, k: Optional[int]) -> Tuple[int, int]:
    """(64-bit mask, mantissa bits kept or -1 for a dtype without a mantissa)."""
    _view, umask, mbits, _code = DTYPES[dtype]
    mask = U64 if umask is None else umask
    kept = mbits
    if k is not None and mbits is not None and k < mbits:
        mask &= U64 ^ ((1 << (mbits - k)) - 1)
        kept = k
    return mask, (-1 if mbits is None else kept)


def weighted_sums(iv: np.ndarray, masks: Sequence[int], salt: int, chunk: int = 1 << 20) -> List[int]:
    """One sum per mask over the flat integer image ``iv`` (any signed/unsigned integer dtype)."""
    flat = np.ascontiguousarray(iv).reshape(-1)
    sums = [0] * len(masks)
    with np.errstate(over="ignore"):
        for start in range(0, flat.size, chunk):
            raw = flat[start:start + chunk].astype(np.int64).view(np.uint64)   # sign-extended, then reinterpreted
            w = weights(start, raw.size, salt)
            for j, m in enumerate(masks):
                sums[j] = (sums[j] + int(((raw & np.uint64(m)) * w).sum(dtype=np.uint64))) & U64
    return sums


def header(shape: Sequence[int], dtype: str, kept_bits: int, seed: int) -> int:
    h = mix64(seed ^ GOLDEN)
    h = mix64(h ^ (kept_bits & 0xFF))
    h = mix64(h ^ mix64(DTYPES[dtype][3]))
    for extent in shape:
        h = mix64(h ^ ((extent + 1) & U64))
    return h


def tensor_digest(iv: np.ndarray, dtype: str, shape: Sequence[int], k: Optional[int] = None, seed: int = 0) -> int:
    mask, kept = and_mask(dtype, k)
    body = weighted_sums(iv, [mask], salt_of(seed))[0]
    return mix64(body ^ header(shape, dtype, kept, seed))


def ladder_for(dtype: str) -> Tuple[int, ...]:
    mbits = DTYPES[dtype][2]
    return () if mbits is None else LADDERS.get(mbits, (6, 4, 2, 0))


def digest_ladder(iv: np.ndarray, dtype: str, shape: Sequence[int], ks: Optional[Sequence[int]] = None,
                  seed: int = 0) -> Dict[str, str]:
    mbits = DTYPES[dtype][2]
    rungs: List[Optional[int]] = [None]
    if mbits is not None:
        rungs += [k for k in (ladder_for(dtype) if ks is None else ks) if 0 <= k < mbits]
    out = {}
    for k in rungs:
        out["full" if k is None else f"k{k}"] = f"{tensor_digest(iv, dtype, shape, k=k, seed=seed):016x}"
    return out


def segment_axis(shape: Sequence[int]) -> int:
    for axis, extent in enumerate(shape):
        if extent > 1:
            return axis
    return 0


def segment_digests(iv: np.ndarray, dtype: str, shape: Sequence[int], rows_per_segment: int = 1024,
                    k: Optional[int] = None, seed: int = 0) -> List[str]:
    flat = np.ascontiguousarray(iv).reshape(-1)
    if len(shape) == 0 or flat.size == 0:
        return [f"{tensor_digest(iv, dtype, shape, k=k, seed=seed):016x}"]
    mask, kept = and_mask(dtype, k)
    rows = shape[segment_axis(shape)]
    rps = max(1, rows_per_segment)
    seg_numel = rps * (flat.size // rows)
    nseg = (rows + rps - 1) // rps
    head = header(shape, dtype, kept, seed)
    out = []
    for s in range(nseg):
        piece = flat[s * seg_numel:(s + 1) * seg_numel]
        body = weighted_sums(piece, [mask], salt_of(seed ^ mix64(s * seg_numel + 1)))[0]
        out.append(f"{mix64(body ^ mix64(head ^ ((s + 1) & U64))):016x}")
    return out
