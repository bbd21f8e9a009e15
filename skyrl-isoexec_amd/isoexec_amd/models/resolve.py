"""Model path or id -> the ``models/<name>.py`` module that declares it.

Reference: isoexec/models/resolve.py:20-216. The ``architectures`` list of a local ``config.json`` is
the primary key; name patterns are the fallback when no config is readable. Nothing is downloaded.
"""

from __future__ import annotations

import importlib
import json
import os
from typing import Optional, Tuple

_MODEL_MODULES = ("qwen3_5",)
_PKG = __name__.rsplit(".", 1)[0]


class ResolutionError(ValueError):
    pass


def _modules() -> list:
    return [importlib.import_module(f"{_PKG}.{name}") for name in _MODEL_MODULES]


def raw_config_json(model_path: str) -> Optional[dict]:
    path = os.path.join(model_path, "config.json")
    if not os.path.isfile(path):
        return None
    try:
        with open(path, "r", encoding="utf-8") as fh:
            data = json.load(fh)
    except (OSError, ValueError):
        return None
    return data if isinstance(data, dict) else None


def resolve_architectures(model_path: str) -> Tuple[str, ...]:
    cfg = raw_config_json(model_path) or {}
    archs = cfg.get("architectures") or ()
    return tuple(a for a in archs if isinstance(a, str))


def assert_no_architecture_collisions() -> None:
    """Two model modules may share an architecture only if each carries a discriminator."""
    owner = {}
    for mod in _modules():
        for arch in mod.PROFILE.architectures:
            if arch in owner and not (mod.PROFILE.arch_discriminator and owner[arch].PROFILE.arch_discriminator):
                raise ResolutionError(
                    f"architecture {arch!r} is declared by both {owner[arch].PROFILE.model!r} and "
                    f"{mod.PROFILE.model!r} without discriminators; dispatch would be order-dependent"
                )
            owner[arch] = mod


def resolve_model_module(model_path: str):
    """``(module, how)``; ``how`` says which key matched. Unknown models raise rather than run unmanaged."""
    assert_no_architecture_collisions()
    mods = _modules()
    archs = resolve_architectures(model_path)
    cfg = raw_config_json(model_path)
    for arch in archs:
        claimants = [m for m in mods if arch in m.PROFILE.architectures]
        if cfg is not None:
            claimants = [m for m in claimants if not m.PROFILE.arch_discriminator or m.PROFILE.arch_discriminator(cfg)]
        if len(claimants) == 1:
            return claimants[0], f"architecture {arch!r}"
        if len(claimants) > 1:
            raise ResolutionError(f"architecture {arch!r} is claimed by {[m.PROFILE.model for m in claimants]}")
    lowered = model_path.lower()
    for mod in mods:
        for pattern in mod.PROFILE.name_patterns:
            if pattern in lowered:
                return mod, f"name pattern {pattern!r}"
    known = sorted(m.PROFILE.model for m in mods)
    raise ResolutionError(
        f"no model declaration matches {model_path!r} (architectures read: {list(archs)}); declared models: {known}"
    )


def resolve_profile(model_path: str):
    return resolve_model_module(model_path)[0].PROFILE


def registered_profiles() -> list:
    return [m.PROFILE for m in _modules()]
