"""GatedDeltaNet op functions on the HIP kernels.

Same names, argument meaning and error behaviour as the reference's ``ops/gdn/gdn_ops.py``:
``gdn_recurrent_kernel`` (:400-441), ``gdn_native_core_kernel`` (:513-558), ``gdn_causal_conv``
(:74-129), ``gdn_causal_conv_batched`` (:132-170), ``gdn_l2norm`` (:202-213),
``gdn_gate_and_beta`` (:1197-1210), ``gdn_recurrent`` (:997-1027), ``gdn_native_core``
(:702-716), ``gdn_core`` (:1118-1194). Forward only: the trainer's VJP is out of scope.
"""

from __future__ import annotations

import torch

from ... import _lib

L2NORM_EPS = 1e-6  # gdn_ops.py:173


def _token_pitch(t: torch.Tensor) -> int:
    """Element pitch between tokens of a ``[..., heads, dim]`` tensor whose heads are contiguous."""
    if t.stride(-1) != 1 or t.stride(-2) != t.shape[-1]:
        raise RuntimeError(f"[isoexec-amd] heads must be contiguous inside a token, got strides {t.stride()}")
    return t.stride(-3)


def _flatten_tokens(t: torch.Tensor, tail: int) -> torch.Tensor:
    """``[B, T, *tail]`` -> a view ``[B*T, *tail]`` (copying only if B and T cannot be merged)."""
    lead = t.shape[: t.ndim - tail]
    if len(lead) == 1:
        return t
    if len(lead) != 2:
        raise RuntimeError(f"[isoexec-amd] expected [B, T, ...], got {tuple(t.shape)}")
    b, n = lead
    if b == 1:
        return t[0]
    if t.stride(0) == n * t.stride(1):
        return t.as_strided((b * n, *t.shape[2:]), (t.stride(1), *t.stride()[2:]), t.storage_offset())
    return t.reshape(b * n, *t.shape[2:])


_CU_CACHE: dict = {}


def _uniform_cu(batch: int, length: int, device) -> torch.Tensor:
    """Token offsets of ``batch`` sequences of equal ``length``; cached, so a decode loop creates none."""
    key = (batch, length, str(device))
    cu = _CU_CACHE.get(key)
    if cu is None:
        if len(_CU_CACHE) > 64:
            _CU_CACHE.clear()
        cu = _CU_CACHE[key] = torch.arange(0, (batch + 1) * length, length, dtype=torch.int32, device=device)
    return cu


def gdn_recurrent_kernel(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor,
    beta: torch.Tensor,
    *,
    ssm_state: torch.Tensor,
    state_indices: torch.Tensor,
    cu_seqlens: torch.Tensor | None = None,
    time_tile: int = 0,
    want_output: bool = True,
    gated_norm: tuple | None = None,
) -> torch.Tensor:
    """The delta-rule scan. Advances ``ssm_state`` IN PLACE. Returns ``o`` shaped like ``v`` (``None`` for a
    state-only pass, ``want_output=False``: nothing but the state pool is written).

    ``gated_norm = (gate [T, HV, V], weight [V], eps, zero_centered)``: the output leaves through the layer's gated
    output norm -- in the scan's own launch where the library serves that form (it declines before the state is
    touched), else by ``fused_gated_out_norm`` on the scan's output: the same bits either way, in ``o``'s shape.

    ``q, k``: ``[B, T, H, K]`` already L2-normalised (H may be GQA-compressed: ``HV % H == 0``);
    ``v``: ``[B, T, HV, V]``; ``g`` (fp32), ``beta``: ``[B, T, HV]``; ``ssm_state`` fp32 pool
    ``[S, HV, V, K]``; ``state_indices`` ``[N]`` (one row per sequence, stored after its last token) or ``[N, Tmax]``
    (column 0 loads, a positive entry at column t stores after token t); ``cu_seqlens``
    ``[N+1]`` int32 for a packed batch (then ``B == 1``), ``None`` for ``[B, T, ...]``.
    """
    _lib.require_device(q, k, v, g, beta, ssm_state, state_indices, cu_seqlens)
    if q.ndim != 4 or v.ndim != 4:
        raise RuntimeError(f"[isoexec-amd] gdn_recurrent_kernel expects [B,T,H,K]/[B,T,HV,V], got {tuple(q.shape)}")
    B, T, H, K = q.shape
    HV, V = v.shape[-2], v.shape[-1]
    if ssm_state.dtype is not torch.float32 or not ssm_state.is_contiguous():
        raise RuntimeError("[isoexec-amd] ssm_state must be a contiguous fp32 pool [S, HV, V, K]")
    if tuple(ssm_state.shape[1:]) != (HV, V, K):
        raise RuntimeError(f"[isoexec-amd] ssm_state {tuple(ssm_state.shape)} != [S,{HV},{V},{K}]")
    io = v.dtype
    if q.dtype is not io or k.dtype is not io:
        raise RuntimeError("[isoexec-amd] q/k/v must share a dtype")
    dev = q.device
    if cu_seqlens is None:
        cu = _uniform_cu(B, T, dev)
        n_seq = B
    else:
        if B != 1:
            raise RuntimeError("[isoexec-amd] a packed batch (cu_seqlens) needs B == 1")
        cu = cu_seqlens.to(torch.int32).contiguous()
        n_seq = cu.numel() - 1
    qf, kf, vf = _flatten_tokens(q, 2), _flatten_tokens(k, 2), _flatten_tokens(v, 2)
    gf = _flatten_tokens(g, 1).to(torch.float32).contiguous()
    bf = _flatten_tokens(beta, 1).to(io).contiguous()
    idx = state_indices.to(torch.int32)
    if idx.ndim == 1:
        # One row per sequence: loaded before its first token, stored once after its last.
        idx = idx.contiguous()
        idx_stride = 0
    else:
        if idx.stride(1) != 1:
            idx = idx.contiguous()
        idx_stride = idx.stride(0)
    if idx.shape[0] != n_seq:
        raise RuntimeError(f"[isoexec-amd] state_indices has {idx.shape[0]} rows for {n_seq} sequences")
    o = torch.empty(qf.shape[0], HV, V, dtype=io, device=dev) if want_output else None
    if time_tile == 0 and cu_seqlens is None and T == 1:
        time_tile = 1
    if gated_norm is not None:
        gate, weight, eps, zero_centered = gated_norm
        _lib.require_device(gate, weight)
        if not want_output or tuple(gate.shape) != (qf.shape[0], HV, V):
            raise RuntimeError("[isoexec-amd] gated_norm needs an output and a gate [tokens, HV, V]")
        fusable = (io is torch.bfloat16 and idx_stride == 0 and gate.dtype is io and weight.dtype is io
                   and gate.stride(2) == 1 and gate.stride(1) == V and weight.is_contiguous() and weight.numel() == V)
        rc = _lib.IX_DECLINED
        if fusable:
            rc = _lib.check(
                _lib.lib().ix_gdn_scan_gated_norm(
                    qf.data_ptr(), kf.data_ptr(), vf.data_ptr(), gf.data_ptr(), bf.data_ptr(), o.data_ptr(),
                    _token_pitch(qf), _token_pitch(kf), _token_pitch(vf), ssm_state.data_ptr(), cu.data_ptr(),
                    idx.data_ptr(), n_seq, H, HV, K, V, float(K) ** -0.5, time_tile, gate.data_ptr(), gate.stride(0),
                    weight.data_ptr(), float(eps), int(zero_centered), _lib.current_stream(dev)), "ix_gdn_scan_gated_norm")
        if rc == _lib.IX_OK:
            return o.view(B, T, HV, V) if cu_seqlens is None else o.unsqueeze(0)
    rc = _lib.check(
        _lib.lib().ix_gdn_scan(
            qf.data_ptr(), kf.data_ptr(), vf.data_ptr(), gf.data_ptr(), bf.data_ptr(), _lib.ptr(o),
            _lib.dtype_code(io), _token_pitch(qf), _token_pitch(kf), _token_pitch(vf), ssm_state.data_ptr(),
            cu.data_ptr(), idx.data_ptr(), idx_stride, n_seq, H, HV, K, V, float(K) ** -0.5, time_tile,
            _lib.current_stream(dev)), "ix_gdn_scan")
    if rc != _lib.IX_OK:
        raise RuntimeError(f"[isoexec-amd] ix_gdn_scan declined K={K} V={V} dtype={io}")
    if o is None:
        return None
    if gated_norm is not None:  # the fused form was declined (nothing launched): the two calls
        from ..norms.fused_outnorm import fused_gated_out_norm

        gate, weight, eps, zero_centered = gated_norm
        o = fused_gated_out_norm(o, gate, weight, eps, zero_centered=zero_centered).view(-1, HV, V)
    return o.view(B, T, HV, V) if cu_seqlens is None else o.unsqueeze(0)


def gdn_l2norm(x: torch.Tensor) -> torch.Tensor:
    """Row-local L2 normalisation ``x * rsqrt(sum x^2 + 1e-6)`` over the last dim; ``[..., H, K]``."""
    _lib.require_device(x)
    if x.ndim < 2:
        raise RuntimeError("[isoexec-amd] gdn_l2norm expects [..., H, K]")
    xf = x if x.ndim == 3 else x.reshape(-1, x.shape[-2], x.shape[-1])
    tokens, H, K = xf.shape
    y = torch.empty(tokens, H, K, dtype=x.dtype, device=x.device)
    rc = _lib.check(
        _lib.lib().ix_gdn_l2norm(xf.data_ptr(), _token_pitch(xf), y.data_ptr(), _lib.dtype_code(x.dtype), tokens, H,
                                 K, L2NORM_EPS, _lib.current_stream(x.device)), "ix_gdn_l2norm")
    if rc != _lib.IX_OK:
        raise RuntimeError(f"[isoexec-amd] ix_gdn_l2norm declined K={K}")
    return y.view(x.shape)


def gdn_gate_and_beta(a: torch.Tensor, b: torch.Tensor, A_log: torch.Tensor, dt_bias: torch.Tensor):
    """``g = -exp(A_log) * softplus(a + dt_bias)`` in fp32; ``beta = sigmoid(b)``. Elementwise.

    The eager form of gdn_ops.py:1197-1210: ``A_log.exp()`` is taken in the parameter's own dtype, so a bf16
    parameter's exponential is rounded to bf16 before the fp32 product ("exp(bf16(x)).float() is not exp(float(x))").
    The fused core's form, which widens the parameter first, is ``gate_and_beta_fp32``."""
    if A_log.dtype is torch.bfloat16:
        return _gate_and_beta(a, b, A_log, dt_bias, _lib.DT_BF16)
    if A_log.dtype is not torch.float32:
        raise RuntimeError(f"[isoexec-amd] gdn_gate_and_beta serves fp32 and bf16 A_log, got {A_log.dtype}")
    return _gate_and_beta(a, b, A_log, dt_bias, _lib.DT_F32)


def gate_and_beta_fp32(a: torch.Tensor, b: torch.Tensor, A_log: torch.Tensor, dt_bias: torch.Tensor):
    """The gating of the fused core (``fused_sigmoid_gating_delta_rule_update``, gdn/_register.py:33-55) and of
    ``native_matched_prep`` (gdn_cpr.py:241-244: ``-torch.exp(A_log.float())``): every parameter widened to fp32
    before any arithmetic, whatever its storage dtype."""
    return _gate_and_beta(a, b, A_log, dt_bias, _lib.DT_F32)


def _gate_and_beta(a, b, A_log, dt_bias, exp_dtype):
    _lib.require_device(a, b, A_log, dt_bias)
    HV = a.shape[-1]

    def rows_of(t):
        # [tokens, HV] with unit-stride rows is read in place at its token pitch (a column slice of a projection)
        if t.ndim == 2 and t.stride(1) == 1 and t.stride(0) >= HV:
            return t, t.stride(0)
        return t.contiguous(), HV

    (ac, ap), (bc, bp) = rows_of(a), rows_of(b)
    g = torch.empty(a.shape, dtype=torch.float32, device=a.device)
    beta = torch.empty(b.shape, dtype=b.dtype, device=b.device)
    A32 = A_log if A_log.dtype is torch.float32 and A_log.is_contiguous() else A_log.float().contiguous()
    dt32 = dt_bias if dt_bias.dtype is torch.float32 and dt_bias.is_contiguous() else dt_bias.float().contiguous()
    _lib.check(
        _lib.lib().ix_gdn_gate(ac.data_ptr(), ap, bc.data_ptr(), bp, A32.data_ptr(), dt32.data_ptr(), g.data_ptr(),
                               beta.data_ptr(), _lib.dtype_code(a.dtype), a.numel() // HV, HV, exp_dtype,
                               _lib.current_stream(a.device)),
        "ix_gdn_gate")
    return g, beta


def decode_prep(x, a, b, conv_weight, conv_bias, A_log, dt_bias, conv_state, rows, *, H, K, HV, V, activation="silu"):
    """One launch in front of a decode step's scan: conv on the stored window (slid in place), l2norm of the q and k
    heads, gate and beta. ``x [N, D]`` pre-conv (rows may be a column slice of a wider buffer), ``a, b [N, HV]``,
    ``rows`` int32 ``[N]`` pool rows (<= 0: a padded lane). Returns ``(y [N, D], g [N, HV] fp32, beta [N, HV])`` with
    the bits of ``conv_packed`` + ``gdn_l2norm`` + ``gate_and_beta_fp32``, or ``None`` when the kernel does not serve
    the shape (the caller then takes those three)."""
    if x.dtype is not torch.bfloat16 or a.dtype is not torch.bfloat16 or b.dtype is not torch.bfloat16:
        return None
    if activation not in (None, "silu", "swish") or conv_weight.shape[-1] != 4 or K != 128:
        return None
    _lib.require_device(x, a, b, conv_weight, conv_bias, A_log, dt_bias, conv_state, rows)
    N, D = x.shape
    if D != 2 * H * K + HV * V or x.stride(1) != 1 or a.stride(-1) != 1 or b.stride(-1) != 1 or a.ndim != 2 or b.ndim != 2:
        return None
    if A_log.dtype is not torch.float32 or dt_bias.dtype is not torch.float32 or rows.dtype is not torch.int32:
        return None
    y = torch.empty(N, D, dtype=x.dtype, device=x.device)
    g = torch.empty(N, HV, dtype=torch.float32, device=x.device)
    beta = torch.empty(N, HV, dtype=x.dtype, device=x.device)
    wc = conv_weight if conv_weight.is_contiguous() else conv_weight.contiguous()
    bc = None if conv_bias is None else (conv_bias if conv_bias.is_contiguous() else conv_bias.contiguous())
    rc = _lib.check(
        _lib.lib().ix_gdn_decode_prep(x.data_ptr(), x.stride(0), a.data_ptr(), a.stride(0), b.data_ptr(), b.stride(0),
                                      wc.data_ptr(), _lib.ptr(bc), A_log.contiguous().data_ptr(),
                                      dt_bias.contiguous().data_ptr(), conv_state.data_ptr(), rows.data_ptr(),
                                      y.data_ptr(), g.data_ptr(), beta.data_ptr(), N, H, K, HV, V, 4,
                                      int(activation is not None), L2NORM_EPS, _lib.current_stream(x.device)),
        "ix_gdn_decode_prep")
    return (y, g, beta) if rc == _lib.IX_OK else None


def conv_packed(x, weight, bias, *, cu_seqlens, conv_state=None, rows_in=None, rows_out=None, activation="silu",
                l2norm_qk: int = 0, head_k_dim: int = 0):
    """Packed varlen conv: ``x [T, D]`` -> ``y [T, D]``; optional pool rows for history in/out.

    ``l2norm_qk`` > 0: channels ``[0, l2norm_qk)`` of ``y`` are q and k heads of ``head_k_dim`` channels and leave
    L2-normalised -- in the same launch where the library serves that form, else by ``gdn_l2norm`` on those columns of
    the plain result: the same bits either way."""
    _lib.require_device(x, weight, bias, cu_seqlens, conv_state, rows_in, rows_out)
    if activation not in (None, "silu", "swish"):
        raise ValueError(f"unsupported activation {activation!r}")
    if x.dtype is not torch.bfloat16:
        raise RuntimeError("[isoexec-amd] conv serves bf16 only")
    T, D = x.shape
    W = weight.shape[-1]
    if weight.shape[0] != D:
        raise ValueError(f"weight {tuple(weight.shape)} incompatible with x dim {D}")
    # x may be a column slice of a wider buffer (row pitch > D); only its rows must be unit-stride
    xc = x if x.stride(1) == 1 and x.stride(0) >= D else x.contiguous()
    wc = weight.contiguous()
    y = torch.empty(T, D, dtype=x.dtype, device=x.device)
    n_seq = cu_seqlens.numel() - 1
    bc = None if bias is None else bias.contiguous()
    if l2norm_qk:
        rc = _lib.check(
            _lib.lib().ix_gdn_conv_l2norm(xc.data_ptr(), xc.stride(0), wc.data_ptr(), _lib.ptr(bc), y.data_ptr(),
                                          _lib.ptr(conv_state), cu_seqlens.data_ptr(), _lib.ptr(rows_in), _lib.ptr(rows_out),
                                          n_seq, T, D, W, int(activation is not None), int(l2norm_qk), int(head_k_dim),
                                          L2NORM_EPS, _lib.current_stream(x.device)), "ix_gdn_conv_l2norm")
        if rc == _lib.IX_OK:
            return y
    rc = _lib.check(
        _lib.lib().ix_gdn_conv(xc.data_ptr(), xc.stride(0), wc.data_ptr(), _lib.ptr(bc), y.data_ptr(), _lib.ptr(conv_state),
                               cu_seqlens.data_ptr(), _lib.ptr(rows_in), _lib.ptr(rows_out), n_seq, T, D, W,
                               int(activation is not None), _lib.current_stream(x.device)), "ix_gdn_conv")
    if rc != _lib.IX_OK:
        raise RuntimeError(f"[isoexec-amd] ix_gdn_conv declined W={W}")
    if l2norm_qk:  # the fused form was declined (nothing launched): the two calls
        heads = int(l2norm_qk) // int(head_k_dim)
        y[:, :l2norm_qk] = gdn_l2norm(y[:, :l2norm_qk].unflatten(1, (heads, int(head_k_dim)))).flatten(1)
    return y


def gdn_causal_conv(x, weight, bias=None, *, initial_state=None, activation="silu", return_final_state=False):
    """Width-W causal depthwise conv over one sequence ``x [T, D]`` (gdn_ops.py:74-129)."""
    if x.ndim != 2:
        raise ValueError(f"gdn_causal_conv expects x=[T, D], got {tuple(x.shape)}")
    T, D = x.shape
    W = weight.shape[-1]
    if initial_state is not None and tuple(initial_state.shape) != (D, W - 1):
        raise ValueError(f"initial_state must be [D, W-1]={(D, W - 1)}, got {tuple(initial_state.shape)}")
    dev = x.device
    pool = torch.zeros(2, D, W - 1, dtype=x.dtype, device=dev)
    if initial_state is not None:
        pool[1] = initial_state.to(x.dtype)
    one = torch.ones(1, dtype=torch.int32, device=dev)
    cu = torch.tensor([0, T], dtype=torch.int32, device=dev)
    y = conv_packed(x, weight, bias, cu_seqlens=cu, conv_state=pool,
                    rows_in=one if initial_state is not None else None,
                    rows_out=one if return_final_state else None, activation=activation)
    if not return_final_state:
        return y
    return y, pool[1].clone()


def gdn_causal_conv_batched(x, weight, bias=None, *, initial_state=None, activation="silu"):
    """Batched conv ``x [N, T, D]``, ``initial_state [N, D, W-1]`` -> ``y [N, T, D]`` (gdn_ops.py:132-170)."""
    if x.ndim != 3:
        raise ValueError(f"gdn_causal_conv_batched expects x=[N, T, D], got {tuple(x.shape)}")
    N, T, D = x.shape
    W = weight.shape[-1]
    dev = x.device
    cu = torch.arange(0, (N + 1) * T, T, dtype=torch.int32, device=dev)
    pool = rows = None
    if initial_state is not None:
        if tuple(initial_state.shape) != (N, D, W - 1):
            raise ValueError(f"initial_state must be [N, D, W-1]={(N, D, W - 1)}, got {tuple(initial_state.shape)}")
        pool = torch.cat([torch.zeros(1, D, W - 1, dtype=x.dtype, device=dev), initial_state.to(x.dtype)], dim=0)
        rows = torch.arange(1, N + 1, dtype=torch.int32, device=dev)
    y = conv_packed(x.reshape(N * T, D), weight, bias, cu_seqlens=cu, conv_state=pool, rows_in=rows,
                    activation=activation)
    return y.view(N, T, D)


def _recurrent_scratch_state(q, v, cu_seqlens):
    """A throwaway zero pool + row indices for a stateless forward (gdn_ops.py:444-464): row 0 unused,
    sequence n at row n+1. One row per sequence (the compact form): the final state lands in the throwaway
    pool instead of nowhere, which costs one 2 MB store per sequence and lets the scan run its branch-free
    token loop; the outputs do not depend on where, or whether, the state is stored."""
    N = cu_seqlens.numel() - 1 if cu_seqlens is not None else q.shape[0]
    HV, V, K = v.shape[-2], v.shape[-1], q.shape[-1]
    ssm_state = torch.zeros(N + 1, HV, V, K, dtype=torch.float32, device=q.device)
    idx = torch.arange(1, N + 1, dtype=torch.int32, device=q.device)
    return ssm_state, idx


def gdn_recurrent(q, k, v, g, beta, *, initial_state=None, output_final_state=False, cu_seqlens=None):
    """Stateless (training / prefill-from-zero) entry: ``(o, None)`` (gdn_ops.py:997-1027)."""
    if initial_state is not None or output_final_state:
        raise NotImplementedError(
            "isoexec GDN: gdn_recurrent is the stateless (training/prefill-from-zero) entry point. "
            "The engine carries state through gdn_recurrent_kernel + a real state pool.")
    with torch.no_grad():
        ssm_state, idx = _recurrent_scratch_state(q, v, cu_seqlens)
        o = gdn_recurrent_kernel(q, k, v, g, beta, ssm_state=ssm_state, state_indices=idx, cu_seqlens=cu_seqlens)
    return o, None


def gdn_kernel_mode() -> str:
    """The delta-rule kernel this process runs (gdn_ops.py:19-36); parsed in ``core/gdn_kernel_env``."""
    from ...core.gdn_kernel_env import gdn_kernel_mode as _mode

    return _mode()


def recurrent_mode() -> bool:
    return gdn_kernel_mode() == "recurrent"


def cpr_mode() -> bool:
    return gdn_kernel_mode() == "cpr"


def fla_chunk_size() -> int:
    """The chunk length of the boundary form (the reference reads vLLM's FLA_CHUNK_SIZE, 64; gdn_ops.py:216-219)."""
    return 64


def gdn_cpr(q, k, v, g, beta, *, initial_state=None, output_final_state=False, cu_seqlens=None):
    """Stateless boundary-form forward: ``(o, None)`` (gdn_ops.py:1063-1116). A padded ``[B, T, ...]`` batch is
    flattened to B packed sequences."""
    if initial_state is not None or output_final_state:
        raise NotImplementedError(
            "isoexec GDN: gdn_cpr is the stateless (training/prefill-from-zero) entry point.")
    from .gdn_cpr import gdn_cpr_fwd

    B, T = q.shape[0], q.shape[1]
    with torch.no_grad():
        if cu_seqlens is None:
            flat = lambda t: t.reshape(1, B * T, *t.shape[2:])
            cu = torch.arange(0, (B + 1) * T, T, dtype=torch.int32, device=q.device)
            o = gdn_cpr_fwd(flat(q), flat(k), flat(v), flat(g), flat(beta), cu_seqlens=cu, chunk_size=fla_chunk_size())
            return o.reshape(B, T, *o.shape[2:]), None
        return gdn_cpr_fwd(q, k, v, g, beta, cu_seqlens=cu_seqlens, chunk_size=fla_chunk_size()), None


def gdn_core(q, k, v, g, beta, *, initial_state=None, output_final_state=False, cu_seqlens=None):
    """The trainer's door (gdn_ops.py:1118-1194): :func:`gdn_recurrent` or :func:`gdn_cpr` per
    :func:`gdn_kernel_mode` (``SKYRL_ISOEXEC_GDN_TRAINER_KERNEL`` overrides it for this door only). The
    chunk-parallel kernel of the vocabulary is not served here: its bits depend on the chunk length, which the
    recurrent and boundary forms do not have to pay for."""
    from ...core.gdn_kernel_env import gdn_trainer_kernel_override

    mode = gdn_trainer_kernel_override() or gdn_kernel_mode()
    kw = dict(initial_state=initial_state, output_final_state=output_final_state, cu_seqlens=cu_seqlens)
    if mode == "cpr":
        return gdn_cpr(q, k, v, g, beta, **kw)
    if mode == "recurrent":
        return gdn_recurrent(q, k, v, g, beta, **kw)
    raise NotImplementedError(
        f"[isoexec-amd] delta-rule kernel {mode!r} is not served on gfx950; use 'recurrent' (default) or 'cpr'")


def gdn_native_core_kernel(q, k, v, a, b, A_log, dt_bias, *, ssm_state, state_indices, cu_seqlens):
    """Raw ``q, k [B, T, H, K]`` (GQA-compressed or expanded), raw gating inputs ``a, b [T, HV]``:
    l2norm, GQA map and fp32 gating folded in front of the scan (gdn_ops.py:513-558). The
    composition is the same three kernels in every call shape, so one varlen call equals T decode
    calls bitwise."""
    qn, kn = gdn_l2norm(q), gdn_l2norm(k)
    HV = v.shape[-2]
    g, beta = gate_and_beta_fp32(a.reshape(-1, HV), b.reshape(-1, HV), A_log, dt_bias)
    lead = v.shape[:2]
    return gdn_recurrent_kernel(qn, kn, v, g.view(*lead, HV), beta.view(*lead, HV), ssm_state=ssm_state,
                                state_indices=state_indices, cu_seqlens=cu_seqlens)


def gdn_native_core_normed(qn, kn, v, a, b, A_log, dt_bias, *, cu_seqlens=None, gated_norm: tuple | None = None):
    """``gdn_native_core`` for q and k that are normalised already (``conv_packed(..., l2norm_qk=...)``): the gating and
    the scan of the same composition, without its two l2norm launches. Same bits as ``gdn_native_core`` on the raw heads.
    ``gated_norm`` as in ``gdn_recurrent_kernel``: the output then comes back through the layer's gated output norm."""
    with torch.no_grad():
        ssm_state, idx = _recurrent_scratch_state(qn, v, cu_seqlens)
        HV = v.shape[-2]
        g, beta = gate_and_beta_fp32(a.reshape(-1, HV), b.reshape(-1, HV), A_log, dt_bias)
        lead = v.shape[:2]
        return gdn_recurrent_kernel(qn, kn, v, g.view(*lead, HV), beta.view(*lead, HV), ssm_state=ssm_state,
                                    state_indices=idx, cu_seqlens=cu_seqlens, gated_norm=gated_norm)


def gdn_native_core(q, k, v, a, b, A_log, dt_bias, *, cu_seqlens=None):
    """Stateless entry for the native composition (gdn_ops.py:702-716)."""
    with torch.no_grad():
        ssm_state, idx = _recurrent_scratch_state(q, v, cu_seqlens)
        return gdn_native_core_kernel(q, k, v, a, b, A_log, dt_bias, ssm_state=ssm_state, state_indices=idx,
                                      cu_seqlens=cu_seqlens)
