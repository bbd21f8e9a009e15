"""Oracle: zero-centred RMSNorm, gated out-norm, add+norm (reference
ops/norms/fused_outnorm.py:113-232, ops/norms/zero_centered_norm.py:36-37,
runtimes/megatron/gdn_fla_shim.py:390-425).

Pinned by (tests/test_oracle_dense.py): ``torch.nn.functional.rms_norm`` on CPU plus the bf16
rounds of the eager expression (a library routine, <= 1 bf16 ulp apart because its fp32 sum runs
in another order); an fp64 brute force on tiny rows; invariance of a row's bits to the row count.
"""

from __future__ import annotations

import numpy as np

from .prims import DEFAULT, F32, Prims, pairwise_tree, round_bf16


def lanes_per_row(n: int) -> int:
    groups = (n + 7) // 8
    lanes = 1
    while lanes < groups and lanes < 64:
        lanes <<= 1
    return lanes


def row_sumsq(x: np.ndarray) -> np.ndarray:
    """fp32 sum of squares over the last axis in the kernels' order: columns c*LPR*8 + p are
    accumulated left to right over chunks c for each of the LPR*8 positions p (square rounded,
    then add rounded), then the adjacent-pairwise tree over p."""
    x = x.astype(F32)
    rows, n = x.shape
    width = lanes_per_row(n) * 8
    chunks = -(-n // width)
    pad = np.zeros((rows, chunks * width), dtype=F32)
    pad[:, :n] = x
    pad = pad.reshape(rows, chunks, width)
    acc = np.zeros((rows, width), dtype=F32)
    for c in range(chunks):
        acc = (acc + (pad[:, c] * pad[:, c]).astype(F32)).astype(F32)
    return pairwise_tree(acc)


def rms_norm_gamma(x: np.ndarray, w: np.ndarray, eps: float, zero_centered: bool = True) -> np.ndarray:
    """x, w hold bf16-representable fp32 values; returns bf16-representable fp32."""
    x = x.astype(F32)
    n = x.shape[-1]
    x2 = x.reshape(-1, n)
    ms = (row_sumsq(x2) / F32(n)).astype(F32)
    rstd = Prims.rsqrt_ieee((ms + F32(eps)).astype(F32))
    nb = round_bf16((x2 * rstd[:, None]).astype(F32))
    gam = round_bf16((F32(1.0) + w.astype(F32)).astype(F32)) if zero_centered else w.astype(F32)
    return round_bf16((nb * gam[None, :]).astype(F32)).reshape(x.shape)


def gated_out_norm(x, gate, w, eps, zero_centered=True, prims: Prims = DEFAULT):
    """``x, gate [T, HV, N]`` -> ``[T*HV, N]``: the norm chain, then ``* silu(gate)`` in fp32, one round."""
    t, hv, n = x.shape
    y = rms_norm_gamma(x.reshape(t * hv, n), w, eps, zero_centered)
    act = prims.silu_div(gate.reshape(t * hv, n).astype(F32))
    return round_bf16((y * act).astype(F32))


def add_rms_norm_gamma(x, residual, w, eps, zero_centered=True):
    h = round_bf16((x.astype(F32) + residual.astype(F32)).astype(F32))
    return rms_norm_gamma(h, w, eps, zero_centered), h
