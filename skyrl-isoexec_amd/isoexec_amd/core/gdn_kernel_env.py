"""The GatedDeltaNet delta-rule kernel selector: one vocabulary, one default, one parser
(reference: core/gdn_kernel_env.py:1-56). The declaration site and the read sites must parse
``SKYRL_ISOEXEC_GDN_KERNEL`` identically, so the parsing lives in one place."""
from __future__ import annotations

import os

KERNEL_ENV = "SKYRL_ISOEXEC_GDN_KERNEL"
# Trainer-only ablation override; a run that sets it is not an IsoExec configuration.
TRAINER_KERNEL_ENV = "SKYRL_ISOEXEC_GDN_TRAINER_KERNEL"

# "cpr": boundary states per chunk, recurrent inside a chunk. "chunk" (the chunk-parallel form) is in the
# vocabulary because launch scripts may name it; this library does not serve it and says so when asked.
KERNELS = ("chunk", "cpr", "recurrent")
DEFAULT_KERNEL = "recurrent"
SERVED_KERNELS = ("cpr", "recurrent")

_RENAMED = {"chunk_synced": "cpr"}


def parse_gdn_kernel(value, env: str = KERNEL_ENV) -> str:
    """Normalise one environment value to a kernel name. Unknown names refuse; empty or absent gives the
    default. A typo that fell back would be the same typo on both runtimes, and they would agree on a wrong
    composition."""
    name = (value or "").strip().lower()
    if not name:
        return DEFAULT_KERNEL
    if name not in KERNELS:
        successor = f" {name!r} was renamed to {_RENAMED[name]!r}." if name in _RENAMED else ""
        raise ValueError(f"{env}={value!r} names no delta-rule kernel; the vocabulary is {list(KERNELS)}.{successor}")
    return name


def gdn_kernel_mode() -> str:
    """The delta-rule kernel this process runs, read from the environment at call time."""
    return parse_gdn_kernel(os.environ.get(KERNEL_ENV), KERNEL_ENV)


def gdn_trainer_kernel_override():
    """The trainer-only kernel override, or None when unset (the supported configuration)."""
    raw = os.environ.get(TRAINER_KERNEL_ENV, "")
    return parse_gdn_kernel(raw, TRAINER_KERNEL_ENV) if raw.strip() else None
