"""Oracle: GatedDeltaNet conv, l2norm, gating and the delta-rule scan (reference
ops/gdn/gdn_ops.py:74-170, :173-213, :261-315, :400-441, :1197-1210).

Pinned by (tests/test_oracle_gdn_moe.py): the textbook fp64 recurrence ``scan_fp64`` (written from the
math, independent of the lane structure); the chunked WY form ``chunk_fp64`` (the same algorithm
as the reference's fp32 ``_torch_chunk_gdr_one``, gdn_ops.py:261-315, in float64); closed forms
(beta = 0: pure decay ``S_T = exp(sum g) S_0``; g = 0, beta = 1, orthonormal keys: associative
recall ``o_t = v_t`` for q = k * sqrt(K)); prefix / split / cross-sequence invariance of the bits
(the reference's gates T1-T4 of gdn_native_kernel_parity_test_gpu.py and
gdn_batch_invariant.py:141-215); conv against a brute-force loop.

``cpr_forward`` restates the boundary form (reference ops/gdn/gdn_cpr.py:104-186 ``chunk_boundary_states``:
"the bf16 snapshot entering chunk c", "final_state is the fp32 accumulator ... the chaining dtype";
:222-319 ``_state_pool`` + one segmented recurrent scan in which every chunk starts from its snapshot).
Pinned by (tests/test_oracle_gdn_moe.py): every snapshot against the float64 state entering that chunk
computed by the chunk-parallel WY pass ``chunk_states_fp64`` (a different algorithm: a triangular solve per
chunk, no token loop) to within one wire-dtype rounding, over enough chunks that a chain restarted from the
rounded snapshots fails; the final states against the same pass; every chunk's outputs against the float64
recurrence started from that chunk's snapshot, far closer than to the one started from the unrounded state;
and bit for bit against ``scan`` where the structure fixes the answer (one chunk per sequence; fp32 wire).
What stays unpinned: bit parity with the third-party chunk kernels the reference calls for the boundary states
(vLLM's FLA ops, not in the reference tree; the reference's tests hold no vectors for them).
"""

from __future__ import annotations

import numpy as np

from ._clib import clib
from .prims import DEFAULT, F32, Prims, pairwise_tree, round_bf16

L2NORM_EPS = 1e-6  # gdn_ops.py:173


def causal_conv(x, weight, bias=None, initial_state=None, activation="silu", prims: Prims = DEFAULT):
    """``x [T, D]``, ``weight [D, W]`` (last tap = current token), ``initial_state [D, W-1]`` oldest
    first. fp32: taps in ascending order (product rounded, add rounded), bias after the taps,
    ``acc * sigmoid(acc)``, one bf16 round. Returns ``(y [T, D], final_state [D, W-1])``."""
    x = x.astype(F32)
    T, D = x.shape
    W = weight.shape[1]
    pad = np.zeros((W - 1, D), dtype=F32) if initial_state is None else initial_state.astype(F32).T
    xp = np.concatenate([pad, x], axis=0)
    acc = np.zeros((T, D), dtype=F32)
    wf = weight.astype(F32)
    for i in range(W):
        acc = (acc + (wf[:, i][None, :] * xp[i : i + T]).astype(F32)).astype(F32)
    if bias is not None:
        acc = (acc + bias.astype(F32)[None, :]).astype(F32)
    if activation in ("silu", "swish"):
        acc = (acc * prims.sigmoid(acc)).astype(F32)
    elif activation is not None:
        raise ValueError(activation)
    return round_bf16(acc), np.ascontiguousarray(xp[T:].T)


def l2norm(x, io_bf16=True):
    """``x [..., K]``: ``x * (1/sqrt(sum x^2 + eps))``; sum = adjacent-pairwise tree over k."""
    x = x.astype(F32)
    sq = (x * x).astype(F32)
    s = pairwise_tree(sq)
    rn = Prims.rsqrt_ieee((s + F32(L2NORM_EPS)).astype(F32))
    y = (x * rn[..., None]).astype(F32)
    return round_bf16(y) if io_bf16 else y


def gate_and_beta(a, b, A_log, dt_bias, io_bf16=True, prims: Prims = DEFAULT, exp_bf16=False):
    """``g = -exp(A_log) * softplus(a + dt_bias)`` fp32; ``beta = sigmoid(b)`` (io dtype). ``exp_bf16``: the eager
    form on a bf16 parameter (gdn_ops.py:1197-1210), whose ``A_log.exp()`` is a bf16 value; otherwise the parameter
    is widened first (the fused core's form, and ``native_matched_prep``, gdn_cpr.py:241-244)."""
    sp = prims.softplus((a.astype(F32) + dt_bias.astype(F32)[None, :]).astype(F32))
    ea = prims.exp(A_log.astype(F32))
    if exp_bf16:
        ea = round_bf16(ea)
    g = ((-ea)[None, :] * sp).astype(F32)
    beta = prims.sigmoid(b.astype(F32))
    return g, (round_bf16(beta) if io_bf16 else beta)


def scan(q, k, v, g, beta, state, scale=None, io_bf16=False, prims: Prims = DEFAULT, snapshots=False):
    """One sequence. ``q, k [T, H, K]``, ``v [T, HV, V]``, ``g, beta [T, HV]``, ``state [HV, V, K]``
    fp32 (updated in place). Returns ``o [T, HV, V]`` (bf16-rounded when ``io_bf16``), and the
    per-token state snapshots when asked."""
    T, H, K = q.shape
    HV, V = v.shape[1], v.shape[2]
    scale = F32(K ** -0.5) if scale is None else F32(scale)
    c = lambda a: np.ascontiguousarray(a, dtype=F32)
    qc, kc, vc, bc = c(q), c(k), c(v), c(beta)
    eg = c(prims.exp(g.astype(F32)))
    o = np.empty((T, HV, V), dtype=F32)
    assert state.dtype == np.float32 and state.flags.c_contiguous and state.shape == (HV, V, K)
    snap = np.empty((T, HV, V, K), dtype=F32) if snapshots else None
    clib().ixo_gdn_scan(qc.ctypes.data, kc.ctypes.data, vc.ctypes.data, eg.ctypes.data, bc.ctypes.data,
                        o.ctypes.data, state.ctypes.data, None if snap is None else snap.ctypes.data, T, H, HV,
                        K, V, float(scale))
    if io_bf16:
        o = round_bf16(o)
    return (o, snap) if snapshots else o


def scan_fp64(q, k, v, g, beta, state0=None, scale=None):
    """Textbook recurrence in float64, written from the math (no lane structure): the
    independent reference for ``scan``. Returns ``(o, final_state)``; state ``[HV, V, K]``."""
    T, H, K = q.shape
    HV, V = v.shape[1], v.shape[2]
    scale = K ** -0.5 if scale is None else scale
    rep = HV // H
    S = np.zeros((HV, V, K)) if state0 is None else state0.astype(np.float64).copy()
    o = np.zeros((T, HV, V))
    q64, k64, v64 = q.astype(np.float64), k.astype(np.float64), v.astype(np.float64)
    for t in range(T):
        kt = np.repeat(k64[t], rep, axis=0)  # [HV, K]
        qt = np.repeat(q64[t], rep, axis=0) * scale
        S = S * np.exp(g[t].astype(np.float64))[:, None, None]
        kv = np.einsum("hvk,hk->hv", S, kt)
        d = (v64[t] - kv) * beta[t].astype(np.float64)[:, None]
        S = S + d[:, :, None] * kt[:, None, :]
        o[t] = np.einsum("hvk,hk->hv", S, qt)
    return o, S


def chunk_fp64(q, k, v, g, beta, chunk=64, scale=None, state0=None, return_states=False):
    """Chunk-parallel WY form in float64 for one sequence: the algorithm of the reference's fp32
    ``_torch_chunk_gdr_one`` (gdn_ops.py:261-315). ``H == HV`` expected. ``state0 [H, V, K]`` is the entry
    state (zero when absent). With ``return_states``: ``(o, entering [NT, H, V, K], final [H, V, K])`` where
    ``entering[c]`` is the state before the first token of chunk ``c`` (the chunk pass never walks tokens:
    one triangular solve and three products per chunk). A ragged last chunk is padded with g = 0, beta = 0,
    k = 0 tokens, which leave the state untouched."""
    T, H, K = q.shape
    V = v.shape[2]
    scale = K ** -0.5 if scale is None else scale
    pad = (-T) % chunk
    f = lambda a: np.pad(a.astype(np.float64), [(0, pad)] + [(0, 0)] * (a.ndim - 1))
    q, k, v, g, beta = f(q) * scale, f(k), f(v), f(g), f(beta)
    Tp = T + pad
    o = np.zeros((Tp, H, V))
    entering = np.zeros((Tp // chunk, H, V, K))
    final = np.zeros((H, V, K))
    for h in range(H):
        S = np.zeros((K, V)) if state0 is None else state0[h].astype(np.float64).T.copy()
        for c0 in range(0, Tp, chunk):
            entering[c0 // chunk, h] = S.T
            sl = slice(c0, c0 + chunk)
            qc, kc, vc, bc = q[sl, h], k[sl, h], v[sl, h], beta[sl, h]
            gc = np.cumsum(g[sl, h])
            decay = np.tril(np.exp(np.tril(gc[:, None] - gc[None, :])))
            kb, vb = kc * bc[:, None], vc * bc[:, None]
            A = -np.tril((kb @ kc.T) * decay, -1)
            sol = np.linalg.solve(np.eye(chunk) - A, np.concatenate([vb, kb * np.exp(gc)[:, None]], axis=1))
            u, kcd = sol[:, :V], sol[:, V:]
            attn = np.tril((qc @ kc.T) * decay)
            v_new = u - kcd @ S
            o[sl, h] = (qc * np.exp(gc)[:, None]) @ S + attn @ v_new
            S = S * np.exp(gc[-1]) + (kc * np.exp(gc[-1] - gc)[:, None]).T @ v_new
        final[h] = S.T
    return (o[:T], entering, final) if return_states else o[:T]


def chunk_states_fp64(k, v, g, beta, chunk, state0=None):
    """Float64 state entering every chunk of ONE sequence, and the final state, by the chunk-parallel pass
    above (GQA-expanded here). ``k [T, H, K]``, ``v [T, HV, V]``, ``g, beta [T, HV]``.
    Returns ``(entering [ceil(T/chunk), HV, V, K], final [HV, V, K])``."""
    rep = v.shape[1] // k.shape[1]
    kx = np.repeat(k, rep, axis=1)
    _, entering, final = chunk_fp64(kx, kx, v, g, beta, chunk, state0=state0, return_states=True)
    return entering, final


def cpr_forward(q, k, v, g, beta, lens, chunk, init=None, wire="bf16", prims: Prims = DEFAULT):
    """Boundary form of the forward over a packed batch (reference ops/gdn/gdn_cpr.py:104-186, :288-319).

    Per sequence an UNROUNDED fp32 state chain runs over the tokens (the reference's ``final_state`` "is the fp32
    accumulator ... the chaining dtype"); the state ENTERING chunk ``c`` is snapshotted in the wire dtype
    (``h [N, NT, HV, V, K]`` "the bf16 snapshot entering chunk c"), widened back to fp32 (``_state_pool``:
    ``copy_`` does the widening cast) and chunk ``c`` is then scanned as its own sequence from that snapshot
    (``chunked_cu_seqlens_and_indices``: one pool row per chunk). The chain's arithmetic is this library's token
    recurrence (``scan``); the reference's comes from third-party chunk kernels.

    ``q, k [T, H, K]``, ``v [T, HV, V]``, ``g, beta [T, HV]`` packed over ``sum(lens)`` tokens (values already
    in the wire dtype's grid), ``init [N, HV, V, K]`` fp32 entry states or None, ``wire`` "bf16" | "fp32".
    Returns ``(o [T, HV, V]`` in the wire dtype's grid, ``snapshots`` list of ``[HV, V, K]`` in (sequence, chunk)
    order, ``finals`` list of fp32 ``[HV, V, K]`` per sequence``)``."""
    assert wire in ("bf16", "fp32")
    HV, V, K = v.shape[1], v.shape[2], k.shape[2]
    to_wire = round_bf16 if wire == "bf16" else (lambda a: a.astype(F32))
    outs, snaps, finals = [], [], []
    pos = 0
    for n, length in enumerate(lens):
        chain = np.zeros((HV, V, K), F32) if init is None else np.ascontiguousarray(init[n], dtype=F32).copy()
        for c0 in range(0, length, chunk):
            sl = slice(pos + c0, pos + min(c0 + chunk, length))
            snap = to_wire(chain)                      # the state entering the chunk, in the wire dtype
            snaps.append(snap.copy())
            start = np.ascontiguousarray(snap, dtype=F32).copy()
            outs.append(scan(q[sl], k[sl], v[sl], g[sl], beta[sl], start, io_bf16=wire == "bf16", prims=prims))
            scan(q[sl], k[sl], v[sl], g[sl], beta[sl], chain, prims=prims)   # the chain advances unrounded
        finals.append(chain)
        pos += length
    o = np.concatenate(outs, 0) if outs else np.zeros((0, HV, V), F32)
    return o, snaps, finals
