"""Assemble the process's Registry from the per-family ``ops/<family>/_register.py`` modules.

Reference: isoexec/core/registry_build.py:19-79. The family modules name only registry records and
string ids, never kernels, so building a registry needs neither the HIP library nor a device.
"""

from __future__ import annotations

import importlib

from .registry import Registry, RegistryError

# Fixed order, for deterministic construction. Listing a family makes its ops installed keys that a
# model's selections must then cover.
_FAMILIES = ("mm", "attention", "rope", "norms", "logprobs", "gdn", "moe")
_PACKAGE = __name__.rsplit(".core.", 1)[0]


def _family_module(family: str):
    try:
        return importlib.import_module(f"{_PACKAGE}.ops.{family}._register")
    except ModuleNotFoundError as exc:
        # Only "this family has no _register" is absence; a broken import inside one propagates.
        if exc.name and exc.name.startswith(f"{_PACKAGE}.ops.{family}"):
            return None
        raise


def registered_families() -> list:
    return [f for f in _FAMILIES if _family_module(f) is not None]


def build_registry(*, strict: bool = False) -> Registry:
    """Build and validate the Registry; ``strict`` raises on a family without a ``_register`` module."""
    reg = Registry()
    absent = []
    for family in _FAMILIES:
        mod = _family_module(family)
        if mod is None:
            absent.append(family)
        else:
            mod.register(reg)
    if strict and absent:
        raise RegistryError(f"strict build: op families missing a _register module: {absent}")
    reg.assert_subsumption_closed()
    return reg
