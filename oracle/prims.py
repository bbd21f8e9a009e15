"""Scalar primitives of the oracle: bf16 rounding and the pluggable transcendentals."""

from __future__ import annotations

import numpy as np

LOG2E = np.float32(1.44269504088896340736)
F32 = np.float32


def round_bf16(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 (round to nearest even, NaN -> 0x7fc0) -> fp32. Pinned against
    ``torch.Tensor.to(torch.bfloat16)`` in tests/test_oracle_dense.py."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    r = np.where(nan, 0x7FC0, r).astype(np.uint32) << 16
    return r.astype(np.uint32).view(np.float32).reshape(x.shape)


def bf16_bits(x: np.ndarray) -> np.ndarray:
    """uint16 bit patterns of bf16-representable fp32 values."""
    return (np.ascontiguousarray(x, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16)


def from_bf16_bits(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << 16).view(np.float32)


class Prims:
    """exp / log / ... as fp32 -> fp32 array functions. Defaults are numpy's (libm class)."""

    def exp(self, x):
        return np.exp(x.astype(F32)).astype(F32)

    def log(self, x):
        return np.log(x.astype(F32)).astype(F32)

    def exp_fast(self, x):  # device: one multiply then v_exp_f32
        return np.exp2((x.astype(F32) * LOG2E).astype(F32)).astype(F32)

    def exp2(self, x):  # device: bare v_exp_f32, results below the normal range flush to zero
        with np.errstate(under="ignore"):
            y = np.exp2(x.astype(F32)).astype(F32)
        return np.where(np.abs(y) < np.finfo(F32).tiny, F32(0.0), y).astype(F32)

    def log1p(self, x):
        return np.log1p(x.astype(F32)).astype(F32)

    # compositions the kernels write out of exp/log with IEEE +,*,/ (same order here)
    def sigmoid(self, x):
        x = x.astype(F32)
        return (F32(1.0) / (F32(1.0) + self.exp(-x))).astype(F32)

    def silu_div(self, x):
        x = x.astype(F32)
        return (x / (F32(1.0) + self.exp(-x))).astype(F32)

    def softplus(self, x):
        x = x.astype(F32)
        with np.errstate(over="ignore"):
            sp = self.log1p(self.exp(x))
        return np.where(x > F32(20.0), x, sp).astype(F32)

    @staticmethod
    def rsqrt_ieee(x):  # IEEE divide and sqrt: the same bits on any conforming host
        return (F32(1.0) / np.sqrt(x.astype(F32))).astype(F32)


DEFAULT = Prims()


def pairwise_tree(a: np.ndarray) -> np.ndarray:
    """Adjacent-pairwise binary tree over the LAST axis (length a power of two), fp32."""
    a = a.astype(F32)
    while a.shape[-1] > 1:
        a = (a[..., 0::2] + a[..., 1::2]).astype(F32)
    return a[..., 0]
