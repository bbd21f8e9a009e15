"""The architecture tag: one dimension of every implementation's identity (``impl@version x arch``).

Reference: isoexec/core/arch.py:14-88. Kernel bit patterns are arch-specific, so the tag is written
into every contract entry, and a trainer/engine pair on different tags refuses to run. On this
library's target the tag is ``gfx950`` (the leading component of ``gcnArchName``); a host with no
visible accelerator gets the sentinel ``cpu``, which the contract builder refuses to key on.
"""

from __future__ import annotations

from dataclasses import dataclass

NON_ACCELERATOR_ARCH: str = "cpu"


def is_accelerator_arch(arch: str) -> bool:
    """True when ``arch`` names a real accelerator: non-empty and not the sentinel."""
    return bool(arch) and arch != NON_ACCELERATOR_ARCH


def _tag_from_gcn_name(name: str) -> str:
    # "gfx950:sramecc+:xnack-" -> "gfx950". Feature suffixes do not change kernel bit patterns.
    return name.split(":", 1)[0].strip()


def detect_arch() -> str:
    """The visible accelerator's tag, or the sentinel when none is visible.

    Once the runtime reports a device, failing to read its name is a detection bug and propagates:
    collapsing it to the sentinel would be baked into a contract identity.
    """
    try:
        import torch
    except Exception:
        return NON_ACCELERATOR_ARCH
    try:
        if not torch.cuda.is_available():
            return NON_ACCELERATOR_ARCH
    except Exception:
        return NON_ACCELERATOR_ARCH
    props = torch.cuda.get_device_properties(torch.cuda.current_device())
    name = getattr(props, "gcnArchName", "") or ""
    if name:
        return _tag_from_gcn_name(name)
    major, minor = torch.cuda.get_device_capability()
    return f"sm{major}{minor}"


ARCH: str = detect_arch()


class ArchMismatchError(RuntimeError):
    """The two runtimes report different arch tags; no cross-arch bitwise claim is ever made."""


@dataclass(frozen=True)
class HardwareTarget:
    arch: str

    @classmethod
    def current(cls) -> "HardwareTarget":
        return cls(arch=ARCH)

    def supports(self, supported_archs) -> bool:
        return self.arch in set(supported_archs)

    def assert_homogeneous(self, other_arch: str) -> None:
        assert_homogeneous(self.arch, other_arch)


def assert_homogeneous(arch_a: str, arch_b: str) -> None:
    if arch_a != arch_b:
        raise ArchMismatchError(
            f"arch handshake failed: this side is {arch_a!r}, other side is {arch_b!r}; trainer and "
            f"engine must run the same architecture."
        )
