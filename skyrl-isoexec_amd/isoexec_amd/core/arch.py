"""The architecture tag.

Kernels give different bits on different architectures, so the tag is part of what an implementation IS
(``impl@version`` on an arch): every contract entry carries it, and a trainer and an engine that report different
tags refuse to pair up -- no claim is ever made across architectures. On the hardware this library targets the tag is
``gfx950``, the first component of the device's ``gcnArchName``; a process that sees no accelerator gets the
sentinel ``cpu``, which the contract builder will not accept as a key. (Reference: isoexec/core/arch.py:14-88.)
"""

from __future__ import annotations

from dataclasses import dataclass

NON_ACCELERATOR_ARCH: str = "cpu"


class ArchMismatchError(RuntimeError):
    """Raised when the two sides of a handshake are on different architectures."""


def is_accelerator_arch(arch: str) -> bool:
    """Is ``arch`` the tag of a real accelerator (neither empty nor the sentinel)?"""
    return arch not in ("", None, NON_ACCELERATOR_ARCH)


def _tag_from_gcn_name(name: str) -> str:
    """``gfx950:sramecc+:xnack-`` -> ``gfx950``: the feature flags after the colon do not change what a kernel
    computes."""
    head, _colon, _flags = name.partition(":")
    return head.strip()


def _visible_device():
    """The torch module if it can see an accelerator, else None. Any failure up to and including the visibility
    question means "no accelerator"."""
    try:
        import torch

        return torch if torch.cuda.is_available() else None
    except Exception:
        return None


def detect_arch() -> str:
    """The tag of the accelerator this process sees, else the sentinel. Once a device IS visible, failing to read
    its name is a bug and is allowed to propagate: quietly answering ``cpu`` would end up inside a contract."""
    torch = _visible_device()
    if torch is None:
        return NON_ACCELERATOR_ARCH
    properties = torch.cuda.get_device_properties(torch.cuda.current_device())
    gcn_name = getattr(properties, "gcnArchName", None)
    if gcn_name:
        return _tag_from_gcn_name(gcn_name)
    return "sm%d%d" % tuple(torch.cuda.get_device_capability())


ARCH: str = detect_arch()


def assert_homogeneous(arch_a: str, arch_b: str) -> None:
    if arch_a == arch_b:
        return
    raise ArchMismatchError(f"arch handshake failed: this side is {arch_a!r}, other side is {arch_b!r}; trainer and "
                            f"engine must run the same architecture.")


@dataclass(frozen=True)
class HardwareTarget:
    """An architecture, with the two questions asked of it."""

    arch: str

    @classmethod
    def current(cls) -> "HardwareTarget":
        return cls(ARCH)

    def supports(self, supported_archs) -> bool:
        return any(self.arch == a for a in supported_archs)

    def assert_homogeneous(self, other_arch: str) -> None:
        assert_homogeneous(self.arch, other_arch)


# ---- device self-check -------------------------------------------------------------------------------------------
SELFCHECK_OBLIGATION = "domain_check:arch.selfcheck"
SELFCHECK_BITS = ("seeded product differs between tile shapes", "integer product differs from the integer truth",
                  "log-softmax launch shapes differ", "a tile id declined the check's shape")
_SELFCHECK = None   # None = not run in this process, else (ok, evidence)


def arch_selfcheck(verbose: bool = True, device=None) -> bool:
    """Check on THIS device that no tile shape or launch form moves the bits (the reference's ``pik_arch_selfcheck``,
    ops/collectives/pik_bootstrap.py:82-93: True on PASS; "the library's invariance guarantee does not hold if this
    fails"). The check itself runs in the library (``ix_arch_selfcheck``) on caller-owned scratch memory. The verdict
    is filed with the enforcement ledger at the install phase; a failure switches the library off for the rest of the
    process, so nothing can be served from a device whose premise failed. Run once per process; later calls return
    the first verdict."""
    global _SELFCHECK
    if _SELFCHECK is not None:
        return _SELFCHECK[0]
    import ctypes

    import torch

    from .. import _lib
    from . import enforce

    L = _lib.lib()
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    with torch.cuda.device(dev):
        need = int(L.ix_arch_selfcheck_workspace_bytes())
        ws = torch.empty(need, dtype=torch.uint8, device=dev)
        mask = ctypes.c_uint(0)
        rc = L.ix_arch_selfcheck(ws.data_ptr(), need, ctypes.byref(mask), _lib.current_stream(dev))
    if rc == _lib.IX_OK:
        ok, evidence = True, f"{ARCH}: tile ids 1-8 and both log-softmax shapes agree bit for bit"
    elif rc == _lib.IX_DECLINED:
        failed = [text for bit, text in enumerate(SELFCHECK_BITS) if mask.value >> bit & 1]
        ok, evidence = False, f"{ARCH}: " + "; ".join(failed)
    else:
        ok, evidence = False, f"{ARCH}: the self-check could not run (code {rc})"
    _SELFCHECK = (ok, evidence)
    enforce.report(SELFCHECK_OBLIGATION, enforce.INSTALL, enforce.OK if ok else enforce.VIOLATION, evidence)
    if verbose:
        print(f"[ISOEXEC-AMD] arch self-check on {ARCH}: {'PASS' if ok else 'FAIL'} ({evidence})", flush=True)
    if not ok:
        _lib.disable(f"arch self-check failed: {evidence}")
    return ok
