"""The callers of the row-invariant logprob: one dispatch point on the trainer, two hooks on the engine.

Reference: the trainer's ``_ix_logprobs_apply`` / ``_ix_try_rowinv_logprobs``
(skyrl_train/distributed/megatron/model_utils.py:925-1044), the engine's logprob hook
(isoexec/runtimes/vllm/vllm_patches.py:236-299) and its sampled-rows LM head
(isoexec/runtimes/vllm/gptmodel_vllm.py:676-688). What this module owes its callers:

* ONE place decides between the row-invariant kernel and the incumbent, and it sits outside any
  autograd.Function, so the same call serves scoring and training;
* a call is served by one function from its first row to its last: the sequence is walked in chunks,
  and a decline on any chunk hands the WHOLE call to the incumbent -- never a mix inside one tensor;
* the chunk walk changes no bit: chunked equals unchunked;
* ``None`` means "declined, nothing was written". A missing kernel library is not a decline: it
  raises, because silently scoring on the incumbent would break trainer/engine agreement.

This build serves one device, so ``group`` must be ``None`` (the kernel declines otherwise) and the
incumbent is the single-rank form of the reference's distributed log-softmax.
"""

from __future__ import annotations

from typing import Callable, Optional

import torch


def _ix_rowinv_available() -> bool:
    """True when the kernel library loads. Raises when it is missing; it never returns False for
    that reason. ``False`` is reserved for a caller that switched the path off."""
    from .. import _lib

    _lib.lib()
    return True


def _ix_rowinv_sampled_logprobs(*args, **kw):
    from ..ops.logprobs.rowinv import rowinv_sampled_logprobs

    return rowinv_sampled_logprobs(*args, **kw)


def _ix_rowinv_full_logprobs(*args, **kw):
    from ..ops.logprobs.rowinv import rowinv_full_logprobs

    return rowinv_full_logprobs(*args, **kw)


def _ix_rowinv_stats() -> dict:
    from ..ops.logprobs.rowinv import stats

    return stats()


# ---------------------------------------------------------------------------------------- the incumbent


def incumbent_log_softmax(logits_fp32: torch.Tensor) -> torch.Tensor:
    """The manual fp32 log-softmax ``(x - amax) - log(sum(exp(x - amax)))`` at world size 1
    (model_utils.py ``_compute_distributed_log_softmax``). Its vocabulary sum is whatever order the
    framework's reduction picks for the shape: the property the row-invariant kernel replaces."""
    shifted = logits_fp32 - logits_fp32.amax(dim=-1, keepdim=True)
    return shifted - shifted.exp().sum(dim=-1, keepdim=True).log()


def incumbent_logprobs(logits, target, vocab_start_index: int, vocab_end_index: int) -> torch.Tensor:
    """Sampled-token logprobs by the incumbent: widen, log-softmax, gather, zero the out-of-shard
    targets. Differentiable through plain autograd."""
    outside = (target < vocab_start_index) | (target >= vocab_end_index)
    local = (target - vocab_start_index).masked_fill(outside, 0)
    rows = incumbent_log_softmax(logits.to(torch.float32))
    return rows.gather(-1, local.unsqueeze(-1)).squeeze(-1).masked_fill(outside, 0.0)


def _incumbent_apply(logits, target, vocab_start_index, vocab_end_index, inference_only, chunk_size):
    grad_on = torch.is_grad_enabled() and not inference_only
    with torch.set_grad_enabled(grad_on):
        if chunk_size is None:
            return incumbent_logprobs(logits, target, vocab_start_index, vocab_end_index)
        parts = [
            incumbent_logprobs(c, t, vocab_start_index, vocab_end_index)
            for c, t in zip(torch.split(logits, chunk_size, dim=1), torch.split(target, chunk_size, dim=1))
        ]
        return torch.cat(parts, dim=1)


# ---------------------------------------------------------------------------------------- trainer side


def _ix_try_rowinv_logprobs(
    vocab_parallel_logits: torch.Tensor,  # [B, S, V]
    target: torch.Tensor,  # [B, S]
    vocab_start_index: int,
    vocab_end_index: int,
    group,
    inference_only: bool,
    chunk_size: Optional[int],
) -> Optional[torch.Tensor]:
    """Serve the whole call on the row-invariant kernel, or return None so the incumbent keeps it
    whole. Chunks travel in their native dtype; the kernel widens inside its own forward."""
    src_dtype = vocab_parallel_logits.dtype
    seq_len = int(vocab_parallel_logits.shape[1])
    step = seq_len if chunk_size is None else int(chunk_size)
    # Under inference_only the incumbent offers no backward, so the kernel must not grow one.
    grad_on = torch.is_grad_enabled() and not inference_only
    served = []
    with torch.set_grad_enabled(grad_on):
        # torch.split gives the same views as slicing (so the same forward bits) with one backward
        # node for the walk instead of one zero-filled gradient per chunk.
        for chunk, target_chunk in zip(torch.split(vocab_parallel_logits, step, dim=1), torch.split(target, step, dim=1)):
            if not chunk.is_contiguous():
                chunk = chunk.contiguous()

            def reference(chunk=chunk, target_chunk=target_chunk) -> torch.Tensor:
                with torch.no_grad():
                    return incumbent_logprobs(chunk, target_chunk, vocab_start_index, vocab_end_index)

            got = _ix_rowinv_sampled_logprobs(
                chunk,
                target_chunk,
                vocab_start_index=vocab_start_index,
                vocab_end_index=vocab_end_index,
                group=group,
                src_dtype=src_dtype,
                reference=reference,
            )
            if got is None:
                return None
            if grad_on and vocab_parallel_logits.requires_grad and not got.requires_grad:
                # A failed probe handed back the reference's tensor, which carries no graph. Refuse
                # rather than emit a chunk whose gradient is silently zero.
                return None
            served.append(got)
    if _ix_rowinv_stats().get("agreed") is False:
        # A probe failure switched the kernel off mid-walk: the chunks mix two functions.
        return None
    return served[0] if len(served) == 1 else torch.cat(served, dim=1)


def _ix_logprobs_apply(
    vocab_parallel_logits: torch.Tensor,
    target: torch.Tensor,
    vocab_start_index: int,
    vocab_end_index: int,
    group,
    inference_only: bool,
    chunk_size: Optional[int],
) -> torch.Tensor:
    """The ONE dispatch point between the row-invariant logprob and the incumbent."""
    seq_len = int(vocab_parallel_logits.shape[1])
    # Chunk only when chunking actually splits the sequence.
    walk = chunk_size if (chunk_size is not None and chunk_size < seq_len) else None
    if _ix_rowinv_available():
        got = _ix_try_rowinv_logprobs(
            vocab_parallel_logits, target, vocab_start_index, vocab_end_index, group, inference_only, walk
        )
        if got is not None:
            return got.contiguous()
    return _incumbent_apply(
        vocab_parallel_logits, target, vocab_start_index, vocab_end_index, inference_only, walk
    ).contiguous()


def from_parallel_logits_to_logprobs(
    vocab_parallel_logits: torch.Tensor,
    target: torch.Tensor,
    vocab_start_index: int = 0,
    vocab_end_index: Optional[int] = None,
    group=None,
    inference_only: bool = False,
    chunk_size: Optional[int] = None,
) -> torch.Tensor:
    """Next-token logprobs ``[B, S-1]`` of ``target [B, S]`` under ``logits [B, S, V]``: position s
    scores token s+1 (model_utils.py ``from_parallel_logits_to_logprobs``)."""
    end = vocab_parallel_logits.shape[-1] if vocab_end_index is None else vocab_end_index
    shifted = target.roll(shifts=-1, dims=-1)
    out = _ix_logprobs_apply(vocab_parallel_logits, shifted, vocab_start_index, end, group, inference_only, chunk_size)
    return out[:, :-1]


# ---------------------------------------------------------------------------------------- engine side

_CL_STATE = {"calls": 0, "rowinv_owned": 0, "incumbent": 0}


def engine_logprob_census() -> dict:
    return dict(_CL_STATE)


def _incumbent_full_rows(logits: torch.Tensor) -> torch.Tensor:
    return incumbent_log_softmax(logits.to(torch.float32))


def make_engine_compute_logprobs(orig: Callable[[torch.Tensor], torch.Tensor] | None = None):
    """Wrap the engine's logprob producer ``orig(logits [N, V]) -> fp32 [N, V]``. The wrapper returns
    the full fp32 row under the leaf-tree denominator, and hands a declined call to ``orig`` whole.
    Wrapping twice returns the existing wrapper."""
    orig = orig or _incumbent_full_rows
    if getattr(orig, "_isoexec_rowinv_full_row_hook", False):
        return orig

    def _isoexec_compute_logprobs(logits: torch.Tensor) -> torch.Tensor:
        _CL_STATE["calls"] += 1
        got = _ix_rowinv_full_logprobs(logits, src_dtype=logits.dtype, reference=lambda: orig(logits))
        if got is not None:
            _CL_STATE["rowinv_owned"] += 1
            return got
        _CL_STATE["incumbent"] += 1
        return orig(logits)

    _isoexec_compute_logprobs._isoexec_rowinv_full_row_hook = True
    _isoexec_compute_logprobs._isoexec_orig = orig
    return _isoexec_compute_logprobs


class SampledRowsHead:
    """The engine's LM head applied to the sampled rows only (``logprobs.lm_head_slice``).

    The forward pass returns hidden states; ``compute_logits`` runs ``hidden @ W^T`` on the rows
    the sampler asks for (the hidden states are already normalised). This equals slicing the all-rows logits because the GEMM's
    value for a row does not depend on which other rows share the launch.
    """

    def __init__(self, weight: torch.Tensor, *, logit_scale: float | None = None):
        self.weight = weight
        self.logit_scale = logit_scale

    def compute_logits(self, hidden_states: torch.Tensor, sample_rows: torch.Tensor | None = None) -> torch.Tensor:
        from ..ops.mm.mm_hip import linear_nt

        rows = hidden_states if sample_rows is None else hidden_states.index_select(0, sample_rows)
        if rows.dtype != self.weight.dtype:
            rows = rows.to(self.weight.dtype)  # bf16 -> fp32 -> bf16 upstream is lossless
        logits = linear_nt(rows.contiguous(), self.weight)
        if logits is None:
            raise RuntimeError("[isoexec-amd] LM-head GEMM declined")
        if self.logit_scale is not None and self.logit_scale != 1.0:
            logits = logits * self.logit_scale
        return logits
