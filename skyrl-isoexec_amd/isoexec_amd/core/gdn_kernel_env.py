"""Which delta-rule kernel the GatedDeltaNet sites run, as named by the environment.

Counterpart of the reference's core/gdn_kernel_env.py:1-56. The declaration side (what the contract pins) and the
read side (what ``ops/gdn`` dispatches on) both ask this module, so a spelling is interpreted once. An unknown
spelling is an error and not the default: both runtimes would make the same mistake and then agree with each other.
"""
from __future__ import annotations

import os
from typing import Mapping, Optional

KERNEL_ENV = "SKYRL_ISOEXEC_GDN_KERNEL"
TRAINER_KERNEL_ENV = "SKYRL_ISOEXEC_GDN_TRAINER_KERNEL"  # ablation switch for the trainer's door only

# name -> (served here, what it is)
_VOCABULARY: Mapping[str, tuple] = {
    "chunk": (False, "chunk-parallel form; its bits depend on the chunk length"),
    "cpr": (True, "fp32 chain at chunk boundaries, recurrent inside a chunk"),
    "recurrent": (True, "token-by-token recurrence"),
}
KERNELS = tuple(sorted(_VOCABULARY))
SERVED_KERNELS = tuple(k for k in KERNELS if _VOCABULARY[k][0])
DEFAULT_KERNEL = "recurrent"
_FORMER_NAMES = {"chunk_synced": "cpr"}


def parse_gdn_kernel(value, env: str = KERNEL_ENV) -> str:
    """One environment value -> a kernel name; nothing set -> the default; anything else raises."""
    text = "" if value is None else str(value).strip().lower()
    if text in _VOCABULARY:
        return text
    if not text:
        return DEFAULT_KERNEL
    message = f"{env}={value!r} names no delta-rule kernel; the vocabulary is {list(KERNELS)}."
    if text in _FORMER_NAMES:
        message += f" {text!r} was renamed to {_FORMER_NAMES[text]!r}."
    raise ValueError(message)


def _lookup(env: str) -> Optional[str]:
    raw = os.environ.get(env)
    return None if raw is None or not raw.strip() else parse_gdn_kernel(raw, env)


def gdn_kernel_mode() -> str:
    """The kernel of this process, looked up when asked (not at import)."""
    return _lookup(KERNEL_ENV) or DEFAULT_KERNEL


def gdn_trainer_kernel_override() -> Optional[str]:
    """The trainer-door override if one is set, else None. A run that sets it is an ablation."""
    return _lookup(TRAINER_KERNEL_ENV)
