"""Row-count-invariant sampled-token and full-row logprobs on the HIP leaf-tree kernels.

Same entry points and protocol as the reference's ``ops/logprobs/rowinv.py:666-875``:
``None`` means "declined, the incumbent keeps the call"; a served call returns fp32 logprobs
shaped like ``target``. One GPU only, so ``group`` must be ``None`` (world size 1).
"""

from __future__ import annotations

import os
from collections.abc import Callable

import torch

from ... import _lib

LEAVES_ENV = "SKYRL_ISOEXEC_PIK_LEAVES"  # rowinv.py:18
BANNER = "[ISOEXEC-ROWINV-LOGPROB]"
PROBE_EVERY = 512
PROBE_MAX_ABS = 1e-4  # rowinv.py:21-22
BLOCK = 4096  # rowinv.py:23; compiled into the kernel

_S = {"calls": 0, "served": 0, "declined": 0, "decline_reason": "", "agreed": None, "probes": 0, "tokens": 0,
      "full_rows": 0, "latched_off": False}


def stats() -> dict:
    return dict(_S)


def _reset_for_test() -> None:
    _S.update({"calls": 0, "served": 0, "declined": 0, "decline_reason": "", "agreed": None, "probes": 0,
               "tokens": 0, "full_rows": 0, "latched_off": False})


def _decline(reason: str) -> None:
    _S["declined"] += 1
    _S["decline_reason"] = reason


def leaves() -> int:
    try:
        return int(os.environ.get(LEAVES_ENV, "8"))
    except ValueError:
        return 0


def _admit(logits, target, vocab_start_index, vocab_end_index, group, src_dtype) -> tuple[int | None, str]:
    """The reference's admission predicate (rowinv.py:310-381) for world size 1 on gfx950."""
    _S["calls"] += 1
    g = leaves()
    reason = ""
    if os.environ.get("SKYRL_ISOEXEC") != "1":
        reason = "SKYRL_ISOEXEC!=1"
    elif _S["latched_off"]:
        reason = "latched off by a failed probe"
    elif group is not None:
        reason = "a process group was passed: this build serves world size 1 only"
    elif not logits.is_cuda or logits.dtype not in (torch.float32, torch.bfloat16):
        reason = f"requires device fp32/bf16 logits, got device={logits.device} dtype={logits.dtype}"
    elif src_dtype not in (torch.float32, torch.bfloat16, torch.float16):
        reason = f"source dtype {src_dtype} is not fp32/bf16/fp16"
    elif logits.dtype is not torch.float32 and logits.dtype is not src_dtype:
        reason = f"low-precision logits dtype {logits.dtype} contradicts declared src_dtype {src_dtype}"
    elif logits.ndim not in (2, 3) or target.shape != logits.shape[:-1] or not logits.is_contiguous():
        reason = f"unsupported logits/target layout logits={tuple(logits.shape)} target={tuple(target.shape)}"
    elif target.dtype not in (torch.int32, torch.int64):
        reason = f"target dtype {target.dtype} is not int32/int64"
    elif target.numel() == 0:
        reason = "zero rows"
    elif vocab_start_index != 0 or vocab_end_index != logits.shape[-1]:
        reason = f"non-contiguous/equal vocab partition start={vocab_start_index} end={vocab_end_index}"
    elif g < 1 or (g & (g - 1)) != 0:
        reason = f"{LEAVES_ENV}={os.environ.get(LEAVES_ENV)!r} is not a positive power of two"
    elif logits.shape[-1] % g != 0:
        reason = f"V={logits.shape[-1]} is not divisible by G={g}: unequal leaves change the contract, declining"
    if reason:
        _decline(reason)
        return None, reason
    return g, ""


def _workspace(rows: int, vocab: int, g: int, device) -> torch.Tensor:
    n = _lib.lib().ix_logprob_workspace_bytes(rows, vocab, g)
    return torch.empty(max(n, 4) // 4, dtype=torch.float32, device=device)


def sampled_forward(x: torch.Tensor, t: torch.Tensor, g: int, *, force_shape: int = 0,
                    row_max: torch.Tensor | None = None):
    """Kernel call on a 2-D ``[rows, V]`` matrix. Returns ``(logprob [rows], lse [rows])``.
    ``row_max`` (fp32 ``[rows]``, each row's exact maximum) lets the kernel skip its max pass."""
    _lib.require_device(x, t, row_max)
    rows, vocab = x.shape
    t64 = t.to(torch.int64).contiguous()
    out = torch.empty(rows, dtype=torch.float32, device=x.device)
    lse = torch.empty(rows, dtype=torch.float32, device=x.device)
    ws = _workspace(rows, vocab, g, x.device)
    rc = _lib.check(
        _lib.lib().ix_logprob_rowinv_sampled(
            x.data_ptr(), _lib.dtype_code(x.dtype), rows, vocab, x.stride(0), t64.data_ptr(), g, out.data_ptr(),
            lse.data_ptr(), ws.data_ptr(), ws.numel() * 4, force_shape, _lib.ptr(row_max),
            _lib.current_stream(x.device)),
        "ix_logprob_rowinv_sampled")
    if rc != _lib.IX_OK:
        return None, None
    return out, lse


def full_forward(x: torch.Tensor, g: int, *, force_shape: int = 0):
    _lib.require_device(x)
    rows, vocab = x.shape
    out = torch.empty(rows, vocab, dtype=torch.float32, device=x.device)
    ws = _workspace(rows, vocab, g, x.device)
    rc = _lib.check(
        _lib.lib().ix_logprob_rowinv_full(
            x.data_ptr(), _lib.dtype_code(x.dtype), rows, vocab, x.stride(0), g, out.data_ptr(), out.stride(0),
            None, ws.data_ptr(), ws.numel() * 4, force_shape, None, _lib.current_stream(x.device)),
        "ix_logprob_rowinv_full")
    return out if rc == _lib.IX_OK else None


class _RowInvSampledLogprob(torch.autograd.Function):
    """Kernel forward; rank-local backward from per-row scalars (rowinv.py:573-612)."""

    @staticmethod
    def forward(ctx, logits, target, g):
        x = logits.reshape(-1, logits.shape[-1])
        out, lse = sampled_forward(x, target.reshape(-1), g)
        if out is None:
            raise RuntimeError(f"{BANNER} kernel declined an admitted signature")
        ctx.save_for_backward(logits, target, lse)
        return out.reshape(target.shape)

    @staticmethod
    def backward(ctx, grad_out):
        logits, target, lse = ctx.saved_tensors
        vocab = logits.shape[-1]
        x = logits.reshape(-1, vocab)
        t = target.reshape(-1).to(torch.int64)
        upstream = grad_out.reshape(-1).to(torch.float32)
        valid = (t >= 0) & (t < vocab)
        upstream = torch.where(valid, upstream, torch.zeros_like(upstream))
        grad = torch.exp(x - lse.unsqueeze(1)).mul_(-upstream.unsqueeze(1))
        grad.scatter_add_(1, t.masked_fill(~valid, 0).unsqueeze(1), upstream.unsqueeze(1))
        return grad.to(logits.dtype).reshape(logits.shape), None, None


def rowinv_sampled_logprobs(
    logits: torch.Tensor,
    target: torch.Tensor,
    *,
    vocab_start_index: int,
    vocab_end_index: int,
    group,
    src_dtype: torch.dtype,
    reference: Callable[[], torch.Tensor] | None,
) -> torch.Tensor | None:
    """Return row-invariant sampled logprobs, or ``None`` to retain the incumbent owner."""
    g, _reason = _admit(logits, target, vocab_start_index, vocab_end_index, group, src_dtype)
    if g is None:
        return None
    result = _RowInvSampledLogprob.apply(logits, target, g)
    should_probe = reference is not None and (
        _S["agreed"] is None or (_S["served"] > 0 and _S["served"] % PROBE_EVERY == 0))
    if should_probe:
        incumbent = reference()
        _S["probes"] += 1
        cand = result.detach().float()
        finite = bool(torch.isfinite(cand).all()) and bool(torch.isfinite(incumbent).all())
        max_abs = float((cand - incumbent.float()).abs().max()) if finite else float("inf")
        if not finite or max_abs > PROBE_MAX_ABS:
            _S["agreed"] = False
            _S["latched_off"] = True
            _decline(f"end-to-end probe failed: max abs {max_abs:.3e} vs {PROBE_MAX_ABS:.1e}")
            return incumbent
        _S["agreed"] = True
    _S["served"] += 1
    _S["tokens"] += target.numel()
    return result


def rowinv_full_logprobs(
    logits: torch.Tensor,
    *,
    src_dtype: torch.dtype,
    reference: Callable[[], torch.Tensor] | None,
) -> torch.Tensor | None:
    """Full-row ``[N, V]`` fp32 logprobs under the same leaf-tree denominator (rowinv.py:796-875)."""
    if logits.ndim != 2 or logits.numel() == 0:
        _S["calls"] += 1
        _decline(f"full-row entry requires a non-empty [N, V] matrix, got shape={tuple(logits.shape)}")
        return None
    rows, vocab = logits.shape
    fake_target = torch.zeros(rows, dtype=torch.int64, device=logits.device)
    g, _reason = _admit(logits, fake_target, 0, vocab, None, src_dtype)
    if g is None:
        return None
    with torch.no_grad():
        out = full_forward(logits, g)
        if out is None:
            _decline("kernel declined")
            return None
        if reference is not None and (_S["agreed"] is None):
            incumbent = reference()
            _S["probes"] += 1
            max_abs = float((out - incumbent.float()).abs().max())
            if not (max_abs <= PROBE_MAX_ABS):
                _S["agreed"] = False
                _S["latched_off"] = True
                _decline(f"full-row probe failed: max abs {max_abs:.3e}")
                return incumbent
            _S["agreed"] = True
    _S["served"] += 1
    _S["tokens"] += rows
    _S["full_rows"] += rows
    return out


def dense_head_logprobs(hidden: torch.Tensor, norm_weight: torch.Tensor, lm_head: torch.Tensor,
                        target: torch.Tensor, *, eps: float = 1e-6, zero_centered: bool = True, g: int | None = None,
                        tile: int = 0):
    """Final norm -> LM head -> sampled logprobs for ``hidden [M, H]`` (the tail of both the trainer
    scoring forward and the engine's ``compute_logits`` + logprob hook). The GEMM epilogue hands the
    row maxima to the log-softmax kernel, so the bf16 logits are written once and read once. Same
    bits as calling the three ops separately. Returns ``(logprob [M], logits [M, V])``."""
    from ..mm.mm_hip import linear_nt
    from ..norms.fused_outnorm import fused_rms_norm_gamma

    x = fused_rms_norm_gamma(hidden, norm_weight, eps, zero_centered=zero_centered)
    got = linear_nt(x, lm_head, tile=tile, want_row_max=True)
    if got is None:
        raise RuntimeError("[isoexec-amd] LM-head GEMM declined")
    logits, row_max = got
    lp, _ = sampled_forward(logits, target, g or leaves(), row_max=row_max)
    return lp, logits
