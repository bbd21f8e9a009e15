"""The mixture-of-experts doors with the reference's own call shapes, over the HIP kernels.

The reference patches four Megatron call sites (ops/moe/moe_batch_invariant.py:780-845): the router's ``routing``
(``_make_sorted_topk_routing``, :394-416), the dispatcher's ``dispatch_postprocess``
(``_dispatch_postprocess_fixed_shape``, moe_batched_experts.py:534-605), ``SequentialMLP.forward``
(``_batched_experts_forward``, moe_batched_experts.py:301-531) and ``moe_utils.unpermute``
(``_deterministic_unpermute`` / ``_fixed_order_combine``, moe_batch_invariant.py:276-385). The functions below keep
those names, argument lists and return shapes, so a maintainer binds them at the same sites; each is a thin
adapter onto the kernels behind ``moe_hip`` (same integers, same bits as the ``Permutation`` path).
"""

from __future__ import annotations

import torch

from ... import _lib
from . import moe_hip

_STACKED = {}   # id(module) -> (key, w1 [E, 2F, H], w2 [E, H, F])
_VALIDATE_FIRST_N_CALLS = 8     # moe_batch_invariant.py:24
_validated_calls = 0            # layouts checked by the combine
_validated_counts = 0           # per-expert counts checked by the experts' door


def _stacked_weights(module):
    """``[E, 2F, H]`` / ``[E, H, F]`` views of the experts' fc1 / fc2 weights. Experts whose weights already sit one
    after the other in one buffer (a stacked parameter) are viewed in place; otherwise they are stacked once and the
    stack is kept until a weight's storage or version changes."""
    experts = module.local_experts
    w1s = [e.linear_fc1.weight for e in experts]
    w2s = [e.linear_fc2.weight for e in experts]

    def in_place(ws):
        first = ws[0]
        if not first.is_contiguous():
            return None
        step = first.numel() * first.element_size()
        if all(w.is_contiguous() and w.shape == first.shape and w.data_ptr() == first.data_ptr() + i * step
               and w.untyped_storage().data_ptr() == first.untyped_storage().data_ptr() for i, w in enumerate(ws)):
            return first.as_strided((len(ws),) + tuple(first.shape), (first.numel(),) + tuple(first.stride()))
        return None

    a, b = in_place(w1s), in_place(w2s)
    if a is not None and b is not None:
        return a, b
    key = tuple((w.data_ptr(), w._version) for w in w1s + w2s)
    hit = _STACKED.get(id(module))
    if hit is None or hit[0] != key:
        hit = (key, torch.stack([w.detach() for w in w1s]).contiguous(), torch.stack([w.detach() for w in w2s]).contiguous())
        _STACKED[id(module)] = hit
    return hit[1], hit[2]


def _check_config(module) -> None:
    cfg = getattr(module, "config", None)
    if cfg is None:
        return
    if not getattr(cfg, "gated_linear_unit", True) or getattr(cfg, "add_bias_linear", False) or getattr(cfg, "fp8", False):
        raise RuntimeError("[isoexec-amd] the expert kernels serve bias-free bf16 SwiGLU experts only")
    if getattr(cfg, "activation_func_clamp_value", None) is not None or getattr(cfg, "glu_linear_offset", 0.0) != 0.0:
        raise RuntimeError("[isoexec-amd] the expert kernels serve plain silu(gate) * up (no clamp, no offset)")
    act = getattr(cfg, "activation_func", None)
    if act is not None and act is not torch.nn.functional.silu:
        raise RuntimeError("[isoexec-amd] the expert kernels serve the SiLU activation only")


def _batched_experts_forward(self, permuted_local_hidden_states, tokens_per_expert, permuted_probs):
    """Drop-in ``SequentialMLP.forward`` (moe_batched_experts.py:301): ``permuted_local_hidden_states [R, H]`` bf16
    rows already grouped by expert, ``tokens_per_expert [E]`` (any integer dtype, host or device), ``permuted_probs
    [R]`` -> ``(out [R, H], None)``. The prob multiplies the activation before fc2, as there (:496-503)."""
    x = permuted_local_hidden_states
    if x.shape[0] == 0:
        return x.new_zeros(0, x.shape[-1]), None
    _lib.require_device(x, permuted_probs)
    _check_config(self)
    w1, w2 = _stacked_weights(self)
    E = int(self.num_local_experts)
    R, H = x.shape
    F = w2.shape[2]
    dev = x.device
    L = _lib.lib()
    counts = tokens_per_expert.to(device=dev)
    if counts.dtype not in (torch.int32, torch.int64):
        counts = counts.to(torch.int64)
    counts = counts.contiguous()
    global _validated_counts
    if _validated_counts < _VALIDATE_FIRST_N_CALLS:
        # The kernels keep every tile inside the R rows whatever the counts say, but rows that no expert claims
        # would be left unwritten: on the first calls the counts are read back and checked, like the combine's layout.
        _validated_counts += 1
        total = int(counts.sum().item())
        if total != R or counts.numel() != E:
            raise RuntimeError(f"[isoexec-amd] SequentialMLP.forward: tokens_per_expert has {counts.numel()} entries "
                               f"adding up to {total} for {R} permuted rows and {E} local experts")
    BM = int(L.ix_moe_pick_bm(R, 1, E))
    max_tiles = int(L.ix_moe_max_tiles(R, 1, E, BM))
    meta = torch.empty(1 + 3 * max_tiles, dtype=torch.int32, device=dev)
    stream = _lib.current_stream(dev)
    rc = _lib.check(L.ix_moe_block_map(counts.data_ptr(), int(counts.dtype is torch.int64), E, BM, R, None,
                                       meta.data_ptr(), max_tiles, stream), "ix_moe_block_map")
    if rc != _lib.IX_OK:
        raise RuntimeError(f"[isoexec-amd] ix_moe_block_map declined E={E}")
    rows = torch.arange(R, dtype=torch.int32, device=dev)      # the rows are already in expert order
    probs = permuted_probs.to(torch.float32).contiguous()
    xc = x if x.stride(1) == 1 else x.contiguous()
    inter = torch.empty(R, F, dtype=torch.bfloat16, device=dev)
    out = torch.empty(R, H, dtype=torch.bfloat16, device=dev)
    rc = _lib.check(L.ix_moe_experts(xc.data_ptr(), xc.stride(0), rows.data_ptr(), probs.data_ptr(), w1.data_ptr(),
                                     w2.data_ptr(), meta.data_ptr(), max_tiles, BM, inter.data_ptr(), out.data_ptr(), R,
                                     R, H, F, stream), "ix_moe_experts")
    if rc != _lib.IX_OK:
        raise RuntimeError(f"[isoexec-amd] ix_moe_experts declined H={H} F={F}")
    return out, None


def reset_combine_validation() -> None:
    """Start the first-calls layout validations over (the reference resets its counter on install, :556)."""
    global _validated_calls, _validated_counts
    _validated_calls = 0
    _validated_counts = 0


def _combine_rows(sorted_indices, num_tokens: int, k: int):
    """``[T, k]`` int32 row numbers: a token's rows in ascending expert order. Rows are expert-major, so a stable sort
    by token groups them. On the first calls the layout is checked, as the reference does (:307-316): every token must
    own exactly k rows; token dropping or capacity padding would otherwise sum the wrong rows without a sign."""
    global _validated_calls
    rows = torch.argsort(sorted_indices, stable=True)
    if _validated_calls < _VALIDATE_FIRST_N_CALLS:
        _validated_calls += 1
        expected = torch.arange(num_tokens, device=sorted_indices.device).repeat_interleave(k)
        if not torch.equal(sorted_indices[rows].to(expected.dtype), expected):
            raise RuntimeError(
                "[isoexec-amd] MoE combine: tokens do not each route to exactly topk experts "
                f"(num_tokens={num_tokens}, permuted_rows={int(sorted_indices.numel())}). Token dropping / capacity "
                "padding must be disabled for bitwise IsoExec.")
    return rows.to(torch.int32).view(num_tokens, k).contiguous()


def _weighted_combine(permuted_tokens, permuted_probs, sorted_indices, restore_shape, out_dtype):
    """The eager chain of moe_batch_invariant.py:366-385 in one launch: ``(tokens * probs[:, None])`` in torch's
    promoted dtype, a token's k rows summed left to right in that dtype, one cast to ``out_dtype``. ``None`` when the
    layout is not "n rows = k per token" (the reference's decline)."""
    num_tokens = int(restore_shape[0])
    n = int(sorted_indices.numel())
    if num_tokens == 0 or n == 0 or n % num_tokens != 0:
        return None
    _lib.require_device(permuted_tokens, sorted_indices, permuted_probs)
    k = n // num_tokens
    arith = permuted_tokens.dtype if permuted_probs is None else torch.promote_types(permuted_tokens.dtype,
                                                                                       permuted_probs.dtype)
    for what, dt in (("token", permuted_tokens.dtype), ("arithmetic", arith), ("output", out_dtype)):
        if dt not in (torch.bfloat16, torch.float32):
            raise RuntimeError(f"[isoexec-amd] unpermute: {what} dtype {dt} is not served (bf16 and fp32 are)")
    rows = _combine_rows(sorted_indices, num_tokens, k)
    pt = permuted_tokens.contiguous()
    w = None if permuted_probs is None else permuted_probs.to(torch.float32).contiguous()
    out = torch.empty(num_tokens, pt.shape[1], dtype=out_dtype, device=pt.device)
    _lib.check(_lib.lib().ix_moe_combine_weighted(pt.data_ptr(), _lib.dtype_code(pt.dtype), _lib.ptr(w),
                                                  _lib.dtype_code(arith), rows.data_ptr(), out.data_ptr(),
                                                  _lib.dtype_code(out_dtype), num_tokens, pt.shape[1], k,
                                                  _lib.current_stream(pt.device)), "ix_moe_combine_weighted")
    return out


def _fixed_order_combine(permuted_tokens, sorted_indices, restore_shape):
    """Each token's k expert rows summed in ascending expert order in the rows' own dtype: a bf16 round per add for
    bf16 rows, plain fp32 adds for fp32 rows (moe_batch_invariant.py:276-320). ``None`` when the layout is not
    "every token routes to exactly k experts" (the reference's decline)."""
    num_tokens = int(restore_shape[0])
    n = int(sorted_indices.numel())
    if num_tokens == 0 or n == 0 or n % num_tokens != 0:
        return None
    _lib.require_device(permuted_tokens, sorted_indices)
    if permuted_tokens.dtype is not torch.bfloat16:
        return _weighted_combine(permuted_tokens, None, sorted_indices, restore_shape, permuted_tokens.dtype)
    k = n // num_tokens
    rows = _combine_rows(sorted_indices, num_tokens, k)
    pt = permuted_tokens.contiguous()
    out = torch.empty(num_tokens, pt.shape[1], dtype=torch.bfloat16, device=pt.device)
    _lib.check(_lib.lib().ix_moe_combine(pt.data_ptr(), rows.data_ptr(), out.data_ptr(), num_tokens, pt.shape[1], k, 0,
                                         _lib.current_stream(pt.device)), "ix_moe_combine")
    return out


def _deterministic_unpermute(permuted_tokens, sorted_indices, restore_shape, probs=None, routing_map=None, fused=False,
                             drop_and_pad=False, isoexec_out_dtype=None, **kwargs):
    """Drop-in ``moe_utils.unpermute`` (moe_batch_invariant.py:338-385). With ``probs`` the rows are weighted in torch's
    promoted dtype (bf16 rows x fp32 probs: an fp32 product and an fp32 fixed-order sum, then the trailing cast), as the
    eager expression there. There is no incumbent to fall back to here: the fused / drop-and-pad forms, and a layout
    the combine declines, raise."""
    if fused or drop_and_pad:
        raise RuntimeError("[isoexec-amd] unpermute: the fused and drop-and-pad forms are not batch-invariant; not served")
    out_dtype = permuted_tokens.dtype if isoexec_out_dtype is None else isoexec_out_dtype
    if probs is not None:
        assert routing_map is not None, "Mask must be provided to permute the probs."
        permuted_probs = probs.T.contiguous().masked_select(routing_map.T.contiguous())
        out = _weighted_combine(permuted_tokens, permuted_probs, sorted_indices, restore_shape, out_dtype)
    else:
        out = _fixed_order_combine(permuted_tokens, sorted_indices, restore_shape)
    if out is None:
        raise RuntimeError("[isoexec-amd] unpermute: the row count is not a multiple of the token count "
                           f"(tokens {int(restore_shape[0])}, rows {int(sorted_indices.numel())}); token dropping / "
                           "capacity padding is not served")
    return out.to(dtype=out_dtype)


_deterministic_unpermute._isoexec_accepts_out_dtype = True


def _dispatch_postprocess_fixed_shape(self, hidden_states, probs):
    """Drop-in ``MoEAllGatherTokenDispatcher.dispatch_postprocess`` (moe_batched_experts.py:534-605): from
    ``self.routing_map [T, E]`` and ``probs [T, E]`` to ``(permuted hidden [T*k, H], tokens_per_expert [E] on the
    device, permuted_probs [T*k])`` without a data-dependent shape; leaves the inverse map on ``self``."""
    self.hidden_shape_before_permute = hidden_states.shape
    lo, hi = self.local_expert_indices[0], self.local_expert_indices[-1] + 1
    self.local_map = self.routing_map[:, lo:hi].contiguous()
    self.local_probs = probs[:, lo:hi].contiguous()
    topk = int(self.config.moe_router_topk)
    sorted_indices, permuted_probs, tokens_per_expert = moe_hip.fused_permute_index(self.local_map, self.local_probs, topk)
    self.reversed_local_input_permutation_mapping = sorted_indices
    return hidden_states.index_select(0, sorted_indices), tokens_per_expert, permuted_probs


def topk_router_routing(self, logits):
    """Drop-in ``TopKRouter.routing(logits) -> (routing_probs [T, E] fp32, routing_map [T, E] bool)`` with the sorted
    (score descending, lowest index on ties) selection the reference forces (``_make_sorted_topk_routing``,
    moe_batch_invariant.py:394-416). Reads ``self.topk`` and, from ``self.config``, ``moe_router_pre_softmax`` and
    ``moe_router_topk_scaling_factor``."""
    cfg = getattr(self, "config", None)
    pre = bool(getattr(cfg, "moe_router_pre_softmax", False))
    scaling = getattr(cfg, "moe_router_topk_scaling_factor", None)
    lg = logits.reshape(-1, logits.shape[-1]).to(torch.float32)
    _, _, dprob, dmap = moe_hip.router_topk(lg, int(self.topk), pre_softmax=pre, scaling_factor=scaling, dense=True)
    return dprob, dmap


def _make_sorted_topk_routing(orig=None):
    """Same entry as the reference's wrapper factory: returns the routing function to bind (``orig`` is accepted and
    not called: the kernel IS the sorted selection)."""
    return topk_router_routing
