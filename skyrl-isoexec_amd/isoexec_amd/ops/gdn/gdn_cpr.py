"""Chunk-boundary form of the GatedDeltaNet forward (reference: ops/gdn/gdn_cpr.py:1-319).

The reference computes the state entering every chunk with a chunk-parallel state pass, keeps that boundary state
as a snapshot in the wire dtype (bf16), and then runs ONE segmented recurrent scan in which every chunk is a
sequence that starts from its snapshot; the fp32 state chain between chunks is never rounded. Both the snapshot
dtype and the fp32 chain are part of its contract (gdn_cpr.py:1-5).

Here the boundary states come from the same recurrent scan kernel that serves everything else: one pass over the
whole sequences with the per-token state-index map storing the fp32 state after the last token of every chunk
(an exact copy of the chain), then the snapshot cast, then the segmented scan. The structure, the metadata and
the snapshot/chain dtypes are the reference's; the boundary arithmetic is this library's recurrence, not the
third-party chunk kernels the reference calls (absent here), so the two agree to rounding, not bit for bit.
A chunk size that covers every sequence makes this the plain recurrent forward, bit for bit.
"""
from __future__ import annotations

import os
from collections import OrderedDict

import numpy as np
import torch

from .gdn_ops import gate_and_beta_fp32, gdn_l2norm, gdn_native_core_kernel, gdn_recurrent_kernel

# Host-built chunk metadata (gdn_cpr.py:15-51): pure integers, so identical tensors however they are built.
_META_CACHE: OrderedDict = OrderedDict()
_META_CACHE_MAX = 512


def host_meta_enabled() -> bool:
    """``SKYRL_ISOEXEC_GDN_CPR_HOST_META`` (default on); moves no bits (gdn_cpr.py:20-22)."""
    return os.environ.get("SKYRL_ISOEXEC_GDN_CPR_HOST_META", "1").lower() not in ("0", "false", "no", "")


def host_chunk_meta(lens, chunk_size: int, device, dtype=torch.int32):
    """``(chunk_indices [M, 2] = (sequence, chunk within it), chunk_offsets [N+1] int64)`` for host-known
    lengths (gdn_cpr.py:25-51). Offsets are int64 whatever ``dtype`` is."""
    key = (tuple(int(n) for n in lens), int(chunk_size), str(device), dtype)
    if key in _META_CACHE:
        _META_CACHE.move_to_end(key)
        return _META_CACHE[key]
    pairs, starts = [], [0]
    for s, n in enumerate(key[0]):
        count = -(-n // chunk_size)
        pairs.extend((s, c) for c in range(count))
        starts.append(starts[-1] + count)
    idx = torch.tensor(pairs, dtype=dtype, device=device).reshape(-1, 2)
    off = torch.tensor(starts, dtype=torch.int64, device=device)
    _META_CACHE[key] = (idx, off)
    while len(_META_CACHE) > _META_CACHE_MAX:
        _META_CACHE.popitem(last=False)
    return idx, off


def packed_lens(cu_seqlens: torch.Tensor) -> list:
    """Host sequence lengths of a packed batch: one device read (gdn_cpr.py:182-184)."""
    return (cu_seqlens[1:] - cu_seqlens[:-1]).tolist()


def chunked_cu_seqlens_and_indices(cu_seqlens: torch.Tensor, chunk_size: int, device, lens=None):
    """Split a packed batch at every chunk boundary: ``(cu_chunked [M+1] int32, state_indices [M, chunk_size]
    int32, n_chunks)`` (gdn_cpr.py:187-213). Only column 0 of the map is set (the chunk's pool row, counted from
    1: row 0 is the null row); the map is full width because the scan indexes it by token."""
    lens = packed_lens(cu_seqlens) if lens is None else lens
    cuts = [0]
    for n in lens:
        n = int(n)
        whole, rest = divmod(n, chunk_size)
        for seg in [chunk_size] * whole + ([rest] if rest else []):
            cuts.append(cuts[-1] + seg)
    m = len(cuts) - 1
    state_indices = torch.zeros(m, chunk_size, dtype=torch.int32, device=device)
    if m:
        state_indices[:, 0] = torch.arange(1, m + 1, dtype=torch.int32, device=device)
    return torch.tensor(cuts, dtype=torch.int32, device=device), state_indices, m


# Per-forward memo of the above, keyed on the identity and version of cu_seqlens (gdn_cpr.py:54-107).
_SEQ_CACHE: OrderedDict = OrderedDict()
_SEQ_CACHE_MAX = 8
_SEQ_STATS = {"served": 0, "built": 0, "declined": 0}


def seq_meta_cache_enabled() -> bool:
    return os.environ.get("SKYRL_ISOEXEC_GDN_SEQ_META_CACHE", "1").lower() not in ("0", "false", "no", "")


def seq_meta_census() -> dict:
    return dict(_SEQ_STATS)


def sequence_metadata(cu_seqlens: torch.Tensor, chunk_size: int, device):
    """``(lens, cu_fla, cu_chunked, state_indices, n_chunks)``, memoized while ``cu_seqlens`` is unchanged
    (same object, same version counter); the memo holds the tensor, so its id cannot be reissued meanwhile."""
    memo_key = None
    if seq_meta_cache_enabled() and torch.is_tensor(cu_seqlens) and cu_seqlens.numel() <= 8192:
        memo_key = (id(cu_seqlens), cu_seqlens._version, int(chunk_size), str(cu_seqlens.device))
        held = _SEQ_CACHE.get(memo_key)
        if held is not None:
            _SEQ_CACHE.move_to_end(memo_key)
            _SEQ_STATS["served"] += 1
            return held[1]
    lens = packed_lens(cu_seqlens)
    built = (lens, cu_seqlens.clone()) + chunked_cu_seqlens_and_indices(cu_seqlens, chunk_size, device, lens=lens)
    if memo_key is None:
        _SEQ_STATS["declined"] += 1
    else:
        _SEQ_STATS["built"] += 1
        _SEQ_CACHE[memo_key] = (cu_seqlens, built)
        while len(_SEQ_CACHE) > _SEQ_CACHE_MAX:
            _SEQ_CACHE.popitem(last=False)
    return built


def chunk_boundary_states(q, k, v, g, beta, cu_seqlens, chunk_size: int, initial_state=None,
                          output_final_state: bool = False, lens=None, cu_fla=None, keep_fp32: bool = False):
    """``(h, final_state, chunk_indices)`` (gdn_cpr.py:104-179): ``h [1, M, HV, V, K]`` in the wire dtype is the
    snapshot of the state ENTERING each chunk, chunks in packed order; ``final_state [N, HV, V, K]`` fp32 is the
    unrounded chain at each sequence's end (or None). ``initial_state`` ``[N, HV, V, K]`` fp32 or None.
    ``q`` may be None (the boundary states do not depend on it). ``keep_fp32`` returns ``h`` as the unrounded fp32
    chain instead of the snapshot (for a caller that keeps the chain and snapshots it itself)."""
    if chunk_size < 2:
        raise ValueError("chunk_size must be at least 2")
    if k.ndim != 4 or k.shape[0] != 1:
        raise RuntimeError("[isoexec-amd] chunk_boundary_states expects a packed batch [1, T, H, K]")
    dev = k.device
    if lens is None:
        lens = packed_lens(cu_seqlens)
    lens = [int(n) for n in lens]
    N = len(lens)
    HV, V, K = v.shape[-2], v.shape[-1], k.shape[-1]
    chunk_indices, _ = host_chunk_meta(lens, chunk_size, dev, cu_seqlens.dtype)
    nchunks = [-(-n // chunk_size) for n in lens]
    M = sum(nchunks)
    # Pool rows: 0 null | 1..N the rows the scan loads (they end up holding the state after token 0) |
    # then one row per chunk boundary (the state entering chunks 1.. of every sequence) | then N final rows.
    load0, bound0 = 1, 1 + N
    final0 = bound0 + (M - sum(1 for n in nchunks if n > 0))
    pool = torch.zeros(final0 + N, HV, V, K, dtype=torch.float32, device=dev)
    if initial_state is not None:
        pool[load0:load0 + N].copy_(initial_state)
    tmax = max(lens) if lens else 0
    idx = np.zeros((N, max(tmax, 1)), dtype=np.int32)
    b = bound0
    bound_rows = []  # per packed chunk: the pool row of its entering state, or -n-1 for "initial state of n"
    final_rows = []
    for n, (length, nc) in enumerate(zip(lens, nchunks)):
        if length == 0:
            final_rows.append(load0 + n)
            continue
        idx[n, 0] = load0 + n
        bound_rows.append(-n - 1)
        for c in range(1, nc):
            idx[n, c * chunk_size - 1] = b
            bound_rows.append(b)
            b += 1
        if length == 1:
            final_rows.append(load0 + n)  # the load row is rewritten after token 0
        else:
            idx[n, length - 1] = final0 + n
            final_rows.append(final0 + n)
    if M > 0:  # a state-only pass: q plays no part, nothing but the pool is written
        gdn_recurrent_kernel(k, k, v, g, beta, ssm_state=pool, state_indices=torch.from_numpy(idx).to(dev),
                             cu_seqlens=cu_seqlens if cu_fla is None else cu_fla, want_output=False)
    # the snapshot: entering states in packed chunk order, cast to the wire dtype
    h32 = torch.empty(M, HV, V, K, dtype=torch.float32, device=dev)
    rows_t = torch.tensor([r if r > 0 else 0 for r in bound_rows], dtype=torch.long, device=dev)
    if M > 0:
        h32.copy_(pool[rows_t])
        first = [i for i, r in enumerate(bound_rows) if r < 0]
        first_t = torch.tensor(first, dtype=torch.long, device=dev)
        if initial_state is None:
            h32[first_t] = 0.0
        else:
            seqs = torch.tensor([-bound_rows[i] - 1 for i in first], dtype=torch.long, device=dev)
            h32[first_t] = initial_state.to(torch.float32)[seqs]
    h = (h32 if keep_fp32 else h32.to(k.dtype)).unsqueeze(0)
    final_state = None
    if output_final_state:
        final_state = pool[torch.tensor(final_rows, dtype=torch.long, device=dev)].clone() if N else pool[:0].clone()
        if initial_state is not None:  # a sequence without tokens keeps its entry state
            for n, length in enumerate(lens):
                if length == 0:
                    final_state[n] = initial_state[n]
    return h, final_state, chunk_indices


def _state_pool(h: torch.Tensor, n_chunks: int, device) -> torch.Tensor:
    """The fp32 pool of the segmented scan: row 0 null, rows 1.. the snapshots widened back to fp32
    (gdn_cpr.py:216-222)."""
    h_flat = h.reshape(-1, *h.shape[-3:])
    pool = torch.empty(n_chunks + 1, *h_flat.shape[-3:], dtype=torch.float32, device=device)
    pool[0].zero_()
    pool[1:n_chunks + 1].copy_(h_flat[:n_chunks])
    return pool


def native_matched_prep(k_raw, a, b, A_log, dt_bias):
    """``(kn, g, beta)`` from raw inputs for the boundary pass (gdn_cpr.py:225-254), by the same kernels as the
    scan's own preparation, so the boundary pass and the segmented scan see identical operands."""
    HV = a.shape[-1]
    g, beta = gate_and_beta_fp32(a.reshape(-1, HV), b.reshape(-1, HV), A_log, dt_bias)
    return gdn_l2norm(k_raw), g, beta.to(k_raw.dtype)


def gdn_cpr_fwd(q, k, v, g, beta, *, cu_seqlens, chunk_size: int):
    """Boundary states + one segmented recurrent scan (gdn_cpr.py:296-319). q, k ``[1, T, H, K]`` L2-normalised,
    v ``[1, T, HV, V]``, g, beta ``[1, T, HV]``, packed with ``cu_seqlens [N+1]``. Returns ``o [1, T, HV, V]``."""
    dev = q.device
    lens, cu_fla, cu_chunked, state_indices, n_chunks = sequence_metadata(cu_seqlens, chunk_size, dev)
    h, _final, _ci = chunk_boundary_states(q, k, v, g, beta, cu_seqlens, chunk_size, lens=lens, cu_fla=cu_fla)
    pool = _state_pool(h, n_chunks, dev)
    return gdn_recurrent_kernel(q, k, v, g, beta, ssm_state=pool, state_indices=state_indices, cu_seqlens=cu_chunked)


def gdn_native_cpr_fwd(q, k, v, a, b, A_log, dt_bias, *, cu_seqlens, chunk_size: int):
    """The same from raw q/k and raw gating inputs ``a, b [T, HV]`` (gdn_cpr.py:257-293)."""
    dev = q.device
    T = q.shape[1]
    lens, cu_fla, cu_chunked, state_indices, n_chunks = sequence_metadata(cu_seqlens, chunk_size, dev)
    kn, g, beta = native_matched_prep(k, a, b, A_log, dt_bias)
    h, _final, _ci = chunk_boundary_states(None, kn, v, g.reshape(1, T, -1), beta.reshape(1, T, -1), cu_seqlens,
                                           chunk_size, lens=lens, cu_fla=cu_fla)
    pool = _state_pool(h, n_chunks, dev)
    return gdn_native_core_kernel(q, k, v, a, b, A_log, dt_bias, ssm_state=pool, state_indices=state_indices,
                                  cu_seqlens=cu_chunked)
