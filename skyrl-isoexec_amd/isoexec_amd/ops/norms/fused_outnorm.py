"""Zero-centred RMSNorm, gated GDN output norm and residual add + norm on the HIP kernels.

Same functions as the reference's ``ops/norms/fused_outnorm.py:159-271`` and
``ops/norms/zero_centered_norm.py:25-40``; the reduction order is a function of the row width
alone, so the row count only changes the grid.
"""

from __future__ import annotations

import torch

from ... import _lib


def _norm_args(x, weight):
    _lib.require_device(x, weight)
    if x.dtype is not torch.bfloat16 or weight.dtype is not torch.bfloat16:
        raise RuntimeError(f"[isoexec-amd] norms serve bf16 only, got {x.dtype} / {weight.dtype}")
    if not x.is_contiguous() or not weight.is_contiguous():
        # Rows are addressed as base + row*N + c (fused_outnorm.py:165-168).
        raise RuntimeError(f"x/weight must be contiguous, got {x.stride()} / {weight.stride()}")


def fused_rms_norm_gamma(x: torch.Tensor, weight: torch.Tensor, eps: float, *, zero_centered: bool = True):
    """``rms_norm(x) * (1.0 + weight)`` with the bf16 down-cast chain of the eager expression."""
    _norm_args(x, weight)
    n = x.shape[-1]
    x2 = x.reshape(-1, n)
    out = torch.empty_like(x2)
    _lib.check(
        _lib.lib().ix_rmsnorm_gamma(x2.data_ptr(), weight.data_ptr(), out.data_ptr(), x2.shape[0], n, float(eps),
                                    int(zero_centered), _lib.current_stream(x.device)), "ix_rmsnorm_gamma")
    return out.view(x.shape)


def fused_gated_out_norm(x: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, eps: float, *,
                         zero_centered: bool = True):
    """``x [T, HV, N]`` contiguous, ``gate [T, HV, N]`` with a free token stride -> ``[T*HV, N]``."""
    _norm_args(x, weight)
    t, hv, n = x.shape
    if gate.shape != x.shape:
        raise ValueError(f"gate shape {tuple(gate.shape)} != x shape {tuple(x.shape)}")
    if gate.stride(1) != n or gate.stride(2) != 1:
        raise RuntimeError(f"gate must be unit-stride within a token, got strides {gate.stride()}")
    _lib.require_device(gate)
    out = torch.empty(t * hv, n, dtype=x.dtype, device=x.device)
    _lib.check(
        _lib.lib().ix_gated_out_norm(x.data_ptr(), gate.data_ptr(), gate.stride(0), weight.data_ptr(),
                                     out.data_ptr(), t, hv, n, float(eps), int(zero_centered),
                                     _lib.current_stream(x.device)), "ix_gated_out_norm")
    return out


def fused_add_rms_norm_gamma(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float, *,
                             zero_centered: bool = True):
    """``h = x + residual`` (bf16), ``y = norm(h)``. Returns ``(y, h)``."""
    _norm_args(x, weight)
    _lib.require_device(residual)
    if residual.shape != x.shape or not residual.is_contiguous():
        raise RuntimeError("residual must be contiguous and shaped like x")
    n = x.shape[-1]
    out = torch.empty_like(x)
    h = torch.empty_like(x)
    _lib.check(
        _lib.lib().ix_add_rmsnorm_gamma(x.data_ptr(), residual.data_ptr(), weight.data_ptr(), out.data_ptr(),
                                        h.data_ptr(), x.numel() // n, n, float(eps), int(zero_centered),
                                        _lib.current_stream(x.device)), "ix_add_rmsnorm_gamma")
    return out, h


class ZeroCenteredRMSNorm(torch.nn.Module):
    """``y = rms_norm(x) * (1 + weight)`` (zero_centered_norm.py:25-40), served by the HIP kernel."""

    def __init__(self, hidden_size: int, eps: float = 1e-6, params_dtype=torch.bfloat16, device=None):
        super().__init__()
        self.hidden_size = (hidden_size,)
        self.eps = eps
        self.weight = torch.nn.Parameter(torch.zeros(hidden_size, dtype=params_dtype, device=device))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return fused_rms_norm_gamma(x, self.weight, self.eps)

    def extra_repr(self) -> str:
        return f"{self.hidden_size[0]}, eps={self.eps}, zero_centered_gamma=True"
