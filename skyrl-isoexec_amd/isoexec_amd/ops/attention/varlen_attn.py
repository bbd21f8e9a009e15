"""Causal grouped-query attention whose result for a query does not depend on the launch it ran in.

The reference reaches that property by pinning FlashAttention to one split of the key walk
(``num_splits=1``; isoexec/ops/attention/_register.py:15-77, varlen_backend.py,
megatron_varlen_attn.py): the trainer's packed full-sequence call and the engine's one-token decode
step then give the same bits. Here one kernel serves both: every query walks its keys in blocks of
32 from position 0, and the only things that differ between call shapes are where the keys live
(``kv_start``) and how many tokens of context precede the first query (``q_pos0``).
"""

from __future__ import annotations

import torch

from ... import _lib

HEAD_DIM = 128


def varlen_attention(
    q: torch.Tensor,  # [Tq, HQ, D] (heads contiguous inside a token; the token pitch is free)
    k: torch.Tensor,  # [Tk, HKV, D]
    v: torch.Tensor,  # [Tk, HKV, D], same pitch as k
    cu_seqlens_q: torch.Tensor,  # int32 [N+1]
    max_q_len: int,
    *,
    kv_start: torch.Tensor | None = None,  # int64 [N]: first key token of each sequence; None = packed like q
    q_pos0: torch.Tensor | None = None,  # int32 [N]: context tokens before the first query; negative = null lane
    scale: float | None = None,
) -> torch.Tensor:
    """Returns ``o [Tq, HQ, D]`` bf16. Sequence n attends to key tokens
    ``kv_start[n] + (0 .. q_pos0[n] + len_q[n] - 1)``, causally."""
    if q.ndim != 3 or k.ndim != 3 or v.shape != k.shape:
        raise RuntimeError(f"[isoexec-amd] attention expects q [T,HQ,D], k/v [T,HKV,D]; got {tuple(q.shape)} {tuple(k.shape)} {tuple(v.shape)}")
    if q.dtype is not torch.bfloat16 or k.dtype is not torch.bfloat16 or v.dtype is not torch.bfloat16:
        raise RuntimeError("[isoexec-amd] attention serves bf16 only")
    Tq, HQ, D = q.shape
    HKV = k.shape[1]
    for name, t in (("q", q), ("k", k), ("v", v)):
        if t.stride(-1) != 1 or t.stride(-2) != D:
            raise RuntimeError(f"[isoexec-amd] {name}: heads must be contiguous inside a token, got strides {t.stride()}")
    if k.stride(0) != v.stride(0):
        raise RuntimeError("[isoexec-amd] k and v must share a token pitch")
    if cu_seqlens_q.dtype is not torch.int32:
        raise RuntimeError("[isoexec-amd] cu_seqlens_q must be int32")
    n_seq = cu_seqlens_q.numel() - 1
    if kv_start is None:
        # keys packed beside the queries: sequence n's keys are tokens cu[n] .. cu[n+1]-1 of k, so k must hold a key
        # for every query token (the kernel addresses keys from the queries' offsets)
        if k.shape[0] < Tq:
            raise RuntimeError(f"[isoexec-amd] attention: packed keys hold {k.shape[0]} tokens for {Tq} queries")
        if q_pos0 is not None:
            raise RuntimeError("[isoexec-amd] attention: q_pos0 (context before the first query) needs kv_start")
    _lib.require_device(q, k, v, cu_seqlens_q, kv_start, q_pos0)
    if kv_start is None:
        kv_start = cu_seqlens_q[:-1].to(torch.int64)
    if kv_start.dtype is not torch.int64 or kv_start.numel() != n_seq:
        raise RuntimeError("[isoexec-amd] kv_start must be int64 [N]")
    if q_pos0 is not None and (q_pos0.dtype is not torch.int32 or q_pos0.numel() != n_seq):
        raise RuntimeError("[isoexec-amd] q_pos0 must be int32 [N]")
    o = torch.empty(Tq, HQ, D, dtype=torch.bfloat16, device=q.device)
    if Tq == 0 or n_seq == 0:
        return o
    rc = _lib.check(
        _lib.lib().ix_attn_varlen(
            q.data_ptr(), q.stride(0), k.data_ptr(), v.data_ptr(), k.stride(0), o.data_ptr(), cu_seqlens_q.data_ptr(),
            kv_start.contiguous().data_ptr(), _lib.ptr(None if q_pos0 is None else q_pos0.contiguous()), n_seq,
            int(max_q_len), HQ, HKV, D, float(D) ** -0.5 if scale is None else float(scale),
            _lib.current_stream(q.device)),
        "ix_attn_varlen")
    if rc != _lib.IX_OK:
        raise RuntimeError(f"[isoexec-amd] ix_attn_varlen declined HQ={HQ} HKV={HKV} D={D} pitches={q.stride(0)},{k.stride(0)}")
    return o


class KVCache:
    """Per-sequence contiguous key/value rows for the engine: ``[rows, max_len, HKV, D]`` each, row 0
    the null row. A sequence's keys stay where prefill put them and decode appends in place, so
    ``kv_start = row * max_len`` names them for every later step."""

    def __init__(self, rows: int, max_len: int, num_kv_heads: int, head_dim: int = HEAD_DIM, device="cuda"):
        self.max_len = max_len
        self.k = torch.zeros(rows + 1, max_len, num_kv_heads, head_dim, dtype=torch.bfloat16, device=device)
        self.v = torch.zeros_like(self.k)

    def flat(self):
        return self.k.view(-1, *self.k.shape[2:]), self.v.view(-1, *self.v.shape[2:])

    def write(self, token_index: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor) -> None:
        """Store new tokens at flat indices ``row * max_len + position`` (int64 [T])."""
        kf, vf = self.flat()
        kf.index_copy_(0, token_index, k_new)
        vf.index_copy_(0, token_index, v_new)
