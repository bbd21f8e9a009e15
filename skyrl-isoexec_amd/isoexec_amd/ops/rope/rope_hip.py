"""Rotary position embedding with the reference's rounding chain (isoexec/ops/rope/_register.py:17-77,
rope_fused.py:66-108): rotate-half over the first R lanes, cos/sin rounded to bf16, and
``bf16(bf16(x * cos) + bf16(rot * sin))`` -- three rounds, never one fp32 round.

The cos/sin table is built once on the host in float64 and rounded to fp32 then bf16, so it does not
depend on which device library evaluated the trigonometry; both runtimes index the same table by
absolute position.
"""

from __future__ import annotations

import numpy as np
import torch

from ... import _lib


def rope_tables(max_positions: int, rotary_dim: int, theta: float = 1.0e6, device="cuda"):
    """``(cos, sin)`` bf16 ``[max_positions, rotary_dim]``; angle of lane d at position p is
    ``p * theta ** (-2 * (d mod R/2) / R)``."""
    half = rotary_dim // 2
    inv_freq = 1.0 / (float(theta) ** (np.arange(half, dtype=np.float64) * 2.0 / rotary_dim))
    angles = np.arange(max_positions, dtype=np.float64)[:, None] * inv_freq[None, :]
    angles = np.concatenate([angles, angles], axis=1)
    to_bf16 = lambda a: torch.from_numpy(a.astype(np.float32)).to(torch.bfloat16).to(device)
    return to_bf16(np.cos(angles)), to_bf16(np.sin(angles))


def apply_rope_(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
    """Rotate ``x [T, heads, D]`` in place (a strided slice of a projection output is fine: only the
    heads of one token must be contiguous). ``positions`` int32 [T] index the tables; a position the tables do not
    hold turns that token's rotated lanes into NaN (the kernel never reads past the tables)."""
    if x.dtype is not torch.bfloat16 or cos.dtype is not torch.bfloat16 or sin.dtype is not torch.bfloat16:
        raise RuntimeError("[isoexec-amd] rope serves bf16 only")
    T, heads, D = x.shape
    if x.stride(-1) != 1 or x.stride(-2) != D:
        raise RuntimeError(f"[isoexec-amd] rope: heads must be contiguous inside a token, got strides {x.stride()}")
    R = cos.shape[-1]
    if cos.shape != sin.shape or not cos.is_contiguous() or not sin.is_contiguous():
        raise RuntimeError("[isoexec-amd] rope: cos/sin must be contiguous [positions, R]")
    if positions.dtype is not torch.int32 or positions.numel() != T:
        raise RuntimeError("[isoexec-amd] rope: positions must be int32 [T]")
    if cos.ndim != 2 or R % 2 != 0 or R > D:
        raise RuntimeError(f"[isoexec-amd] rope: tables must be [positions, R] with even R <= D, got {tuple(cos.shape)}")
    _lib.require_device(x, cos, sin, positions)
    rc = _lib.check(
        _lib.lib().ix_rope_inplace(x.data_ptr(), x.stride(0), cos.data_ptr(), sin.data_ptr(), cos.shape[0],
                                   positions.contiguous().data_ptr(),
                                   T, heads, D, R, _lib.current_stream(x.device)),
        "ix_rope_inplace")
    if rc != _lib.IX_OK:
        raise RuntimeError(f"[isoexec-amd] ix_rope_inplace declined T={T} heads={heads} D={D} R={R}")
    return x
