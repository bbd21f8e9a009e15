"""MoE FFN on the HIP kernels: router, permutation, grouped experts, fixed-order combine.

Function names follow the reference: ``fused_router_dense`` / ``fused_permute_index``
(``ops/moe/moe_router_o2_kernel.py:272-351``), the batched expert forward
(``ops/moe/moe_batched_experts.py:301-531``), the deterministic unpermute
(``ops/moe/moe_batch_invariant.py:276-385``). ``moe_ffn_forward`` chains them the way
``MoELayer.forward`` does on both runtimes.
"""

from __future__ import annotations

import torch

from ... import _lib
from ..mm.mm_hip import router_gemm


def router_topk(logits: torch.Tensor, k: int, *, pre_softmax: bool = False, scaling_factor: float | None = None,
                dense: bool = False):
    """Top-k routing. Returns ``(topk_idx [T,k] int32, topk_prob [T,k] fp32, dense_probs, dense_map)``."""
    _lib.require_device(logits)
    if logits.dtype is not torch.float32 or logits.ndim != 2:
        raise RuntimeError("[isoexec-amd] router logits must be fp32 [T, E]")
    lg = logits if logits.stride(1) == 1 else logits.contiguous()
    T, E = lg.shape
    dev = lg.device
    idx = torch.empty(T, k, dtype=torch.int32, device=dev)
    prob = torch.empty(T, k, dtype=torch.float32, device=dev)
    dprob = torch.empty(T, E, dtype=torch.float32, device=dev) if dense else None
    dmap = torch.empty(T, E, dtype=torch.uint8, device=dev) if dense else None
    rc = _lib.check(
        _lib.lib().ix_moe_router_topk(lg.data_ptr(), lg.stride(0), T, E, k, int(pre_softmax),
                                      float(scaling_factor or 0.0), idx.data_ptr(), prob.data_ptr(),
                                      _lib.ptr(dprob), _lib.ptr(dmap), _lib.current_stream(dev)),
        "ix_moe_router_topk")
    if rc != _lib.IX_OK:
        raise RuntimeError(f"[isoexec-amd] router declined E={E} k={k} (k must be a power of two <= 16, E <= 512)")
    return idx, prob, dprob, (dmap.view(torch.bool) if dmap is not None else None)


def fused_router_dense(logits: torch.Tensor, k: int, *, scaling_factor: float | None = None):
    """``(routing_probs [T,E] fp32, routing_map [T,E] bool)`` (moe_router_o2_kernel.py:272-311)."""
    _, _, dprob, dmap = router_topk(logits, k, scaling_factor=scaling_factor, dense=True)
    return dprob, dmap


class Permutation:
    """Device-side routing plan: everything the grouped GEMMs and the combine need."""

    __slots__ = ("T", "E", "k", "BM", "BN", "counts", "offsets", "sorted_token", "permuted_prob", "combine_rows",
                 "tile_meta", "max_tiles")


def permute(topk_idx: torch.Tensor, topk_prob: torch.Tensor, E: int, *, BM: int | None = None,
            BN: int | None = None, static_scratch: bool = False) -> Permutation:
    """Expert-major, token-ascending permutation + block map (integer only, no host sync).

    ``static_scratch=True`` keeps the kernels' internal tables in the library's file-scope device array instead of a
    torch allocation (``ix_moe_permute_static``; calls that overlap on one GPU race on that array)."""
    _lib.require_device(topk_idx, topk_prob)
    T, k = topk_idx.shape
    dev = topk_idx.device
    L = _lib.lib()
    p = Permutation()
    p.T, p.E, p.k = T, E, k
    p.BM = int(BM or L.ix_moe_pick_bm(T, k, E))
    p.BN = int(BN or 256)          # weight-tile width of the grouped GEMMs: 256, or 128 with BM = 128
    p.max_tiles = int(L.ix_moe_max_tiles(T, k, E, p.BM))
    i32 = dict(dtype=torch.int32, device=dev)
    p.counts = torch.empty(E, **i32)
    p.offsets = torch.empty(E + 1, **i32)
    p.sorted_token = torch.empty(T * k, **i32)
    p.permuted_prob = torch.empty(T * k, dtype=torch.float32, device=dev)
    p.combine_rows = torch.empty(T, k, **i32)
    p.tile_meta = torch.empty(1 + 3 * p.max_tiles, **i32)
    if static_scratch:
        rc = L.ix_moe_permute_static(topk_idx.contiguous().data_ptr(), topk_prob.contiguous().data_ptr(), T, E, k, p.BM,
                                     p.counts.data_ptr(), p.offsets.data_ptr(), p.sorted_token.data_ptr(),
                                     p.permuted_prob.data_ptr(), p.combine_rows.data_ptr(), p.tile_meta.data_ptr(),
                                     p.max_tiles, _lib.current_stream(dev))
        if rc == _lib.IX_ERR_SIZE:
            raise RuntimeError(
                f"[isoexec-amd] ix_moe_permute_static: T={T}, E={E} needs {int(L.ix_moe_permute_scratch_ints(T, E))} "
                f"table entries, the static array holds {int(L.ix_moe_permute_static_max_ints())}")
        _lib.check(rc, "ix_moe_permute_static")
        return p
    scratch = torch.empty(max(1, int(L.ix_moe_permute_scratch_ints(T, E))), **i32)
    _lib.check(
        L.ix_moe_permute(topk_idx.contiguous().data_ptr(), topk_prob.contiguous().data_ptr(), T, E, k, p.BM,
                         p.counts.data_ptr(), p.offsets.data_ptr(), p.sorted_token.data_ptr(),
                         p.permuted_prob.data_ptr(), p.combine_rows.data_ptr(), p.tile_meta.data_ptr(), p.max_tiles,
                         scratch.data_ptr(), _lib.current_stream(dev)), "ix_moe_permute")
    return p


def route_and_permute(logits: torch.Tensor, k: int, *, pre_softmax: bool = False, scaling_factor: float | None = None,
                      BM: int | None = None):
    """``router_topk`` then ``permute`` -> ``(topk_idx, topk_prob, Permutation)``. A batch of at most one token tile
    (T <= 256, E <= 128: a decode step) takes ONE launch for both (``ix_moe_route_one_tile``); the integers and the
    weights are the same either way."""
    _lib.require_device(logits)
    if logits.dtype is not torch.float32 or logits.ndim != 2:
        raise RuntimeError("[isoexec-amd] router logits must be fp32 [T, E]")
    T, E = logits.shape
    if T > 256 or E > 128 or T == 0:
        idx, prob, _, _ = router_topk(logits, k, pre_softmax=pre_softmax, scaling_factor=scaling_factor)
        return idx, prob, permute(idx, prob, E, BM=BM)
    lg = logits if logits.stride(1) == 1 else logits.contiguous()
    dev = lg.device
    L = _lib.lib()
    p = Permutation()
    p.T, p.E, p.k = T, E, k
    p.BM = int(BM or L.ix_moe_pick_bm(T, k, E))
    p.BN = 256
    p.max_tiles = int(L.ix_moe_max_tiles(T, k, E, p.BM))
    i32 = dict(dtype=torch.int32, device=dev)
    idx = torch.empty(T, k, **i32)
    prob = torch.empty(T, k, dtype=torch.float32, device=dev)
    p.counts = torch.empty(E, **i32)
    p.offsets = torch.empty(E + 1, **i32)
    p.sorted_token = torch.empty(T * k, **i32)
    p.permuted_prob = torch.empty(T * k, dtype=torch.float32, device=dev)
    p.combine_rows = torch.empty(T, k, **i32)
    p.tile_meta = torch.empty(1 + 3 * p.max_tiles, **i32)
    rc = _lib.check(
        L.ix_moe_route_one_tile(lg.data_ptr(), lg.stride(0), T, E, k, int(pre_softmax), float(scaling_factor or 0.0), p.BM,
                                idx.data_ptr(), prob.data_ptr(), p.counts.data_ptr(), p.offsets.data_ptr(),
                                p.sorted_token.data_ptr(), p.permuted_prob.data_ptr(), p.combine_rows.data_ptr(),
                                p.tile_meta.data_ptr(), p.max_tiles, _lib.current_stream(dev)), "ix_moe_route_one_tile")
    if rc != _lib.IX_OK:
        raise RuntimeError(f"[isoexec-amd] router declined E={E} k={k} (k must be a power of two <= 16)")
    return idx, prob, p


def fused_permute_index(routing_map: torch.Tensor, routing_probs: torch.Tensor, topk: int):
    """``(sorted_indices [T*k] int64, permuted_probs [T*k], tokens_per_expert [E] int64)`` from the
    dense routing tensors (moe_router_o2_kernel.py:313-351)."""
    T, E = routing_map.shape
    idx = routing_map.to(torch.int32).argsort(dim=1, descending=True, stable=True)[:, :topk].to(torch.int32)
    prob = torch.gather(routing_probs, 1, idx.long())
    p = permute(idx.contiguous(), prob.contiguous(), E)
    return p.sorted_token.long(), p.permuted_prob, p.counts.long()


def pack_decode(w1: torch.Tensor, w2: torch.Tensor):
    """Fragment-packed copies ``(w1f, w2f)`` of ``w1 [E, 2F, H]`` and ``w2 [E, H, F]`` for the decode-size expert kernels
    (``ix_moe_pack_decode``): the same values, laid out in the order the kernels' matrix instructions take them, so that a
    decode step streams them as contiguous memory. ``None`` when the kernels do not serve the shape. Make them once per
    weight version and hand them to ``experts_forward`` / ``moe_ffn_forward`` as ``packed``."""
    _lib.require_device(w1, w2)
    if w1.dtype is not torch.bfloat16 or w2.dtype is not torch.bfloat16 or w1.ndim != 3 or w2.ndim != 3:
        return None
    if not w1.is_contiguous() or not w2.is_contiguous():
        return None
    E, F2, H = w1.shape
    if w2.shape != (E, H, F2 // 2):
        raise RuntimeError(f"[isoexec-amd] expert matrices disagree: w1 {tuple(w1.shape)}, w2 {tuple(w2.shape)}")
    w1f, w2f = torch.empty_like(w1), torch.empty_like(w2)
    rc = _lib.check(_lib.lib().ix_moe_pack_decode(w1.data_ptr(), w2.data_ptr(), w1f.data_ptr(), w2f.data_ptr(), E, H, F2 // 2,
                                                  _lib.current_stream(w1.device)), "ix_moe_pack_decode")
    return (w1f, w2f) if rc == _lib.IX_OK else None


def experts_forward(x: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, p: Permutation, *, return_inter: bool = False,
                    packed: tuple | None = None):
    """Grouped fc1 + SwiGLU + prob epilogue + fc2 over the permuted rows. ``x [T, H]`` bf16,
    ``w1 [E, 2F, H]``, ``w2 [E, H, F]``. Returns ``expert_out [T*k, H]`` in permuted order; with ``return_inter`` also
    the activation that enters fc2, ``inter [T*k, F]`` = bf16(bf16(bf16(silu(gate)) * up) * prob). ``packed``
    (``pack_decode(w1, w2)``): read by the decode-size tile (BM = 32) instead of ``w1`` / ``w2``; same bits."""
    _lib.require_device(x, w1, w2)
    if x.dtype is not torch.bfloat16 or w1.dtype is not torch.bfloat16 or w2.dtype is not torch.bfloat16:
        raise RuntimeError("[isoexec-amd] experts serve bf16 only")
    T, H = x.shape
    E, F2, _ = w1.shape
    F = F2 // 2
    rows = T * p.k
    dev = x.device
    inter = torch.empty(rows, F, dtype=torch.bfloat16, device=dev)
    out = torch.empty(rows, H, dtype=torch.bfloat16, device=dev)
    xc = x if x.stride(1) == 1 else x.contiguous()
    if packed is not None and p.BM == 32 and p.BN == 256:
        w1f, w2f = packed
        if w1f.shape != w1.shape or w2f.shape != w2.shape or w1f.dtype is not torch.bfloat16 or w2f.dtype is not torch.bfloat16:
            raise RuntimeError("[isoexec-amd] packed must come from pack_decode(w1, w2)")
        rc = _lib.check(
            _lib.lib().ix_moe_experts_decode(xc.data_ptr(), xc.stride(0), p.sorted_token.data_ptr(),
                                             p.permuted_prob.data_ptr(), w1f.data_ptr(), w2f.data_ptr(),
                                             p.tile_meta.data_ptr(), p.max_tiles, inter.data_ptr(), out.data_ptr(), T, rows,
                                             H, F, _lib.current_stream(dev)), "ix_moe_experts_decode")
        if rc == _lib.IX_OK:
            return (out, inter) if return_inter else out
    rc = _lib.check(
        _lib.lib().ix_moe_experts_tile(xc.data_ptr(), xc.stride(0), p.sorted_token.data_ptr(),
                                       p.permuted_prob.data_ptr(), w1.contiguous().data_ptr(),
                                       w2.contiguous().data_ptr(), p.tile_meta.data_ptr(), p.max_tiles, p.BM,
                                       p.BN, inter.data_ptr(), out.data_ptr(), T, rows, H, F,
                                       _lib.current_stream(dev)),
        "ix_moe_experts")
    if rc != _lib.IX_OK:
        raise RuntimeError(f"[isoexec-amd] ix_moe_experts declined H={H} F={F}")
    return (out, inter) if return_inter else out


def combine(expert_out: torch.Tensor, p: Permutation, *, fp32_acc: bool = False) -> torch.Tensor:
    """Per token, the sum of its k rows in ascending expert order (moe_batch_invariant.py:276-320)."""
    H = expert_out.shape[1]
    out = torch.empty(p.T, H, dtype=torch.bfloat16, device=expert_out.device)
    _lib.check(
        _lib.lib().ix_moe_combine(expert_out.data_ptr(), p.combine_rows.data_ptr(), out.data_ptr(), p.T, H, p.k,
                                  int(fp32_acc), _lib.current_stream(expert_out.device)), "ix_moe_combine")
    return out


def combine_add_rms_norm(expert_out: torch.Tensor, p: Permutation, residual: torch.Tensor, weight: torch.Tensor,
                         eps: float, *, fp32_acc: bool = False, zero_centered: bool = True):
    """``combine`` followed by ``fused_add_rms_norm_gamma`` in one launch -> ``(y, h)``: ``h = bf16(combine + residual)``,
    ``y = norm(h)``, the bits of the two calls without the round trip of the combine's output. ``None`` when the kernel
    does not serve the width or k (the caller then makes the two calls)."""
    H = expert_out.shape[1]
    if (residual.shape != (p.T, H) or not residual.is_contiguous() or residual.dtype is not torch.bfloat16
            or weight.dtype is not torch.bfloat16 or not weight.is_contiguous() or not expert_out.is_contiguous()):
        return None
    _lib.require_device(expert_out, residual, weight)
    out = torch.empty(p.T, H, dtype=torch.bfloat16, device=expert_out.device)
    h = torch.empty_like(out)
    rc = _lib.check(
        _lib.lib().ix_moe_combine_add_rmsnorm(expert_out.data_ptr(), p.combine_rows.data_ptr(), p.k, int(fp32_acc),
                                              residual.data_ptr(), weight.data_ptr(), out.data_ptr(), h.data_ptr(), p.T,
                                              H, float(eps), int(zero_centered),
                                              _lib.current_stream(expert_out.device)), "ix_moe_combine_add_rmsnorm")
    return (out, h) if rc == _lib.IX_OK else None


def moe_ffn_forward(x: torch.Tensor, router_weight: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, k: int, *,
                    pre_softmax: bool = False, logit_bias: torch.Tensor | None = None,
                    scaling_factor: float | None = None, fp32_combine: bool = False, BM: int | None = None,
                    routing_out: list | None = None, add_norm: tuple | None = None,
                    packed: tuple | None = None):
    """Router GEMM (fp32) -> top-k -> permutation -> grouped experts -> combine. ``x [T, H]`` bf16.
    ``routing_out``: a list that receives this call's ``topk_idx [T, k]`` (for comparing composed models whose
    discrete choices must be like for like). ``add_norm = (residual, weight, eps)``: the layer's residual add and the
    next norm are folded into the combine's launch and ``(normed, h)`` is returned instead of the FFN output (the same
    bits as ``fused_add_rms_norm_gamma`` on it)."""
    logits = router_gemm(x, router_weight)
    if logits is None:
        raise RuntimeError("[isoexec-amd] router GEMM declined")
    if logit_bias is not None:
        logits = logits + logit_bias  # elementwise, per token
    idx, prob, p = route_and_permute(logits, k, pre_softmax=pre_softmax, scaling_factor=scaling_factor, BM=BM)
    if routing_out is not None:
        routing_out.append(idx)
    expert_out = experts_forward(x, w1, w2, p, packed=packed)
    if add_norm is None:
        return combine(expert_out, p, fp32_acc=fp32_combine)
    residual, norm_weight, eps = add_norm
    fused = combine_add_rms_norm(expert_out, p, residual, norm_weight, eps, fp32_acc=fp32_combine)
    if fused is not None:
        return fused
    from ..norms.fused_outnorm import fused_add_rms_norm_gamma

    return fused_add_rms_norm_gamma(combine(expert_out, p, fp32_acc=fp32_combine), residual, norm_weight, eps)
