"""Oracle: the batch-invariant dense matmul ``C = A . W^T`` (what the reference's aten
mm/addmm override computes, ops/moe/moe_batch_invariant.py:422-473: fp32 accumulation of bf16
products, one bf16 round).

The fp32 accumulation ORDER inside a matrix instruction is hardware-defined, so this function is
a tolerance reference only: products of bf16 values are exact in fp32, and the result of any
accumulation order lies within the bound ``gemm_tolerance`` of the float64 sum. Pinned by
(tests/test_oracle_dense.py and the GPU tests): ``numpy.matmul`` in float64; the exact-arithmetic
special case (small-integer operands make every partial sum exact, so every order gives the same
bits: a bit-exact known answer); row m independent of M.
"""

from __future__ import annotations

import numpy as np

from .prims import F32, round_bf16


def gemm_nt_fp64(a: np.ndarray, w: np.ndarray, bias: np.ndarray | None = None) -> np.ndarray:
    c = a.astype(np.float64) @ w.astype(np.float64).T
    if bias is not None:
        c = c + bias.astype(np.float64)[None, :]
    return c


def gemm_nt_bf16(a: np.ndarray, w: np.ndarray, bias: np.ndarray | None = None) -> np.ndarray:
    """fp32-accumulated (numpy's order) reference, one bf16 round. Tolerance reference."""
    c = a.astype(F32) @ w.astype(F32).T
    if bias is not None:
        c = (c + bias.astype(F32)[None, :]).astype(F32)
    return round_bf16(c.astype(F32))


def gemm_tolerance(a: np.ndarray, w: np.ndarray) -> np.ndarray:
    """Per-element bound on |bf16(fp32 sum in any order) - float64 sum|: the accumulation error
    ``K * 2^-24 * sum_k |a_k w_k|`` plus half a bf16 ulp of the magnitude."""
    k = a.shape[1]
    mag = np.abs(a.astype(np.float64)) @ np.abs(w.astype(np.float64)).T
    exact = np.abs(a.astype(np.float64) @ w.astype(np.float64).T)
    return k * 2.0 ** -24 * mag + 2.0 ** -8 * np.maximum(exact, 2.0 ** -126) + 1e-30


def small_int_operands(rng, m, n, k, lo=-4, hi=4):
    """Operands whose every partial sum is an integer below 2^24: any order is exact."""
    a = rng.integers(lo, hi + 1, size=(m, k)).astype(F32)
    w = rng.integers(lo, hi + 1, size=(n, k)).astype(F32)
    return a, w
