"""Model declarations. A model module states facts about an architecture (``ModelProfile``); the policy turns the
facts into one implementation per (op, site); the module may list exceptions to the policy. Nothing here computes.
(Reference: isoexec/models/__init__.py:16-35.)
"""

from __future__ import annotations

__all__ = ["build_for", "profile_for"]


def _declaring_module(model_path: str):
    from . import resolve

    module, _matched_by = resolve.resolve_model_module(model_path)
    return module


def build_for(model_path: str, registry, *, arch=None):
    """The contract for the model a path or hub id names. Trainer and engine both come through here, which is why
    they cannot derive different contracts for the same model; a model nobody declared is an error."""
    return _declaring_module(model_path).build(registry, arch=arch)


def profile_for(model_path: str):
    """Only the model's facts, no contract."""
    from . import resolve

    return resolve.resolve_profile(model_path)
