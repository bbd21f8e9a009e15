"""Canonical JSON for the ExecutionContract, driven by the ``wire`` tags on the record types.

The byte form is the one the reference freezes (isoexec/contract/serialize.py:40-43, 138-170): JSON
with sorted keys, ``(",", ":")`` separators, UTF-8 without ASCII escaping, and no JSON float anywhere.
Decoding is strict (serialize.py:173-298): an unknown or missing field refuses, a float refuses, and
only schema "2" is read.
"""

from __future__ import annotations

import dataclasses
import json

from . import types as T

SUPPORTED_SCHEMA_VERSIONS = {"2"}


class SerializationError(Exception):
    pass


class UnknownFieldError(SerializationError):
    pass


# --------------------------------------------------------------------------------------- plain <-> bytes


def _find_float(node, where):
    if isinstance(node, float):
        return where
    if isinstance(node, dict):
        for key, val in node.items():
            hit = _find_float(val, f"{where}.{key}")
            if hit:
                return hit
    elif isinstance(node, (list, tuple)):
        for pos, val in enumerate(node):
            hit = _find_float(val, f"{where}[{pos}]")
            if hit:
                return hit
    return None


def canonical_bytes(plain) -> bytes:
    """The canonical bytes of a plain (dict / list / scalar) structure; a float anywhere refuses."""
    hit = _find_float(plain, "$")
    if hit:
        raise SerializationError(f"raw float at {hit}; use BitPattern or a decimal string")
    return json.dumps(plain, sort_keys=True, separators=(",", ":"), ensure_ascii=False).encode("utf-8")


# --------------------------------------------------------------------------------------- record -> plain


def _plain_const(value):
    return to_plain(value) if isinstance(value, T.BitPattern) else value


def encode_constants(pairs) -> dict:
    """Sorted (key, value) pairs -> a JSON object; a BitPattern becomes ``{"bits", "dtype"}``."""
    return {key: _plain_const(val) for key, val in pairs}


def _plain_field(tag, value):
    if tag == "val":
        return value
    if tag in ("strs", "pair"):
        return list(value)
    if tag == "map":
        return encode_constants(value)
    if isinstance(tag, list):
        return [to_plain(item) for item in value]
    if isinstance(tag, tuple):  # ("opt", cls)
        return None if value is None else to_plain(value)
    return to_plain(value)


def to_plain(record) -> dict:
    """Any contract record -> the plain dict the canonical form serialises."""
    return {f.name: _plain_field(f.metadata["wire"], getattr(record, f.name)) for f in dataclasses.fields(record)}


def to_canonical_json(contract: T.ExecutionContract) -> bytes:
    return canonical_bytes(to_plain(contract))


# --------------------------------------------------------------------------------------- plain -> record


def _check_keys(obj, names, where):
    if not isinstance(obj, dict):
        raise SerializationError(f"{where}: expected an object, got {type(obj).__name__}")
    extra = set(obj) - set(names)
    if extra:
        raise UnknownFieldError(f"{where}: unknown field(s) {sorted(extra)}")
    absent = set(names) - set(obj)
    if absent:
        raise SerializationError(f"{where}: missing field(s) {sorted(absent)}")


def _record_const(value, where):
    return from_plain(T.BitPattern, value, where) if isinstance(value, dict) else value


def _record_field(tag, value, where):
    if tag == "val":
        return value
    if tag == "strs":
        return tuple(value)
    if tag == "pair":
        if len(value) != 2:
            raise SerializationError(f"{where}: must have exactly 2 members")
        return (value[0], value[1])
    if tag == "map":
        return {key: _record_const(val, f"{where}.{key}") for key, val in value.items()}
    if isinstance(tag, list):
        return tuple(from_plain(tag[0], item, f"{where}[{pos}]") for pos, item in enumerate(value))
    if isinstance(tag, tuple):
        return None if value is None else from_plain(tag[1], value, where)
    return from_plain(tag, value, where)


def from_plain(cls, obj, where="contract"):
    """Strictly rebuild a record of type ``cls`` from its plain dict."""
    specs = dataclasses.fields(cls)
    _check_keys(obj, [f.name for f in specs], where)
    return cls(**{f.name: _record_field(f.metadata["wire"], obj[f.name], f"{where}.{f.name}") for f in specs})


def _no_float(text):
    raise SerializationError(f"raw JSON float {text!r}; use BitPattern or a decimal string")


def from_canonical_json(data: bytes) -> T.ExecutionContract:
    """Decode contract bytes. Refuses floats (also NaN/Infinity), unknown fields and other schemas."""
    plain = json.loads(data.decode("utf-8"), parse_float=_no_float, parse_constant=_no_float)
    if isinstance(plain, dict) and "schema_version" in plain and plain["schema_version"] not in SUPPORTED_SCHEMA_VERSIONS:
        raise SerializationError(
            f"unsupported schema_version {plain['schema_version']!r}; this code reads "
            f"{sorted(SUPPORTED_SCHEMA_VERSIONS)}. Identities frozen under another schema hash different "
            f"projections, so they would not mean here what they meant where they were frozen: rebuild "
            f"the contract from the model profile and deliver the new artifact."
        )
    return from_plain(T.ExecutionContract, plain)
