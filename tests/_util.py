"""Shared helpers of the parity tests: device primitives plugged into the oracle, bit views."""

from __future__ import annotations

import numpy as np
import torch

from oracle.prims import Prims


def bits(t: torch.Tensor) -> torch.Tensor:
    """Integer view for bitwise comparison (torch.equal(+0., -0.) is True; the reference compares
    integer views for the same reason, core/contracts.py:40-52)."""
    t = t.contiguous()
    return t.view({4: torch.int32, 2: torch.int16, 8: torch.int64, 1: torch.int8}[t.element_size()])


def same_bits(a: torch.Tensor, b: torch.Tensor) -> bool:
    return a.shape == b.shape and a.dtype == b.dtype and bool(torch.equal(bits(a), bits(b)))


def np_bits(a: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a)
    return a.view({4: np.uint32, 2: np.uint16, 8: np.uint64, 1: np.uint8}[a.dtype.itemsize])


def bf16_to_np(t: torch.Tensor) -> np.ndarray:
    """bf16 tensor -> fp32 numpy holding the same values."""
    return t.detach().float().cpu().numpy()


def np_to_bf16(a: np.ndarray, device="cpu") -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16).to(device)


class DevicePrims(Prims):
    """The oracle's transcendentals evaluated by the device's own functions through the C ABI
    (ix_prim_unary), so oracle-vs-kernel comparisons pin the order of operations bit for bit."""

    def __init__(self, device="cuda:0"):
        from isoexec_amd import _lib

        self._lib = _lib
        self._dev = device

    def _run(self, name, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        t = torch.from_numpy(x.reshape(-1).copy()).to(self._dev)
        return self._lib.prim_unary(name, t).cpu().numpy().reshape(x.shape)

    def exp(self, x):
        return self._run("exp", x)

    def log(self, x):
        return self._run("log", x)

    def exp_fast(self, x):
        return self._run("exp_fast", x)

    def exp2(self, x):
        return self._run("exp2", x)

    def sigmoid(self, x):
        return self._run("sigmoid", x)

    def silu_div(self, x):
        return self._run("silu_div", x)

    def softplus(self, x):
        return self._run("softplus", x)


def cpu_gen(seed: int) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g
