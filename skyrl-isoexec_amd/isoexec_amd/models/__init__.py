"""Per-model compositions: structural facts in, ``{(op, site): impl}`` selections out.

Reference: isoexec/models/__init__.py:16-35.
"""

from __future__ import annotations


def build_for(model_path: str, registry, *, arch=None):
    """Dispatch a model path or id to its contract builder. Both runtimes call this one function, so
    their identities agree by construction."""
    from .resolve import resolve_model_module

    mod, _how = resolve_model_module(model_path)
    return mod.build(registry, arch=arch)


def profile_for(model_path: str):
    from .resolve import resolve_profile

    return resolve_profile(model_path)


__all__ = ["build_for", "profile_for"]
