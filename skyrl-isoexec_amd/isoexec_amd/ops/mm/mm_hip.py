"""Batch-invariant dense matmul on the fixed-K-order MFMA kernel.

Counterpart of the reference's global ``aten::mm/addmm/bmm`` override
(``ops/moe/moe_batch_invariant.py:422-473``) and of ``ops/mm/mm_cublaslt.py``: every
``F.linear`` of the model reaches one kernel whose per-element accumulation order does not
depend on M. On ROCm the dispatch key is still "CUDA".
"""

from __future__ import annotations

import torch

from ... import _lib

_LIBRARY = None
_COUNTS = {"mm": 0, "addmm": 0, "bmm": 0, "declined": 0}


def stats() -> dict:
    return dict(_COUNTS)


def linear_nt(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None, *, tile: int = 0,
              out_dtype: torch.dtype = torch.bfloat16, want_row_max: bool = False):
    """``x [M, K] @ weight [N, K]^T (+ bias)``, bf16 operands, fp32 accumulate; ``None`` if declined.

    ``out_dtype=torch.float32`` returns the fp32 accumulator unrounded. ``want_row_max`` also returns
    each row's exact maximum over the N outputs (taken in the kernel's epilogue), as ``(out, row_max)``.
    """
    _lib.require_device(x, weight, bias)
    if x.dtype is not torch.bfloat16 or weight.dtype is not torch.bfloat16:
        return None
    if x.ndim != 2 or weight.ndim != 2 or x.shape[1] != weight.shape[1]:
        raise RuntimeError(f"linear_nt shape mismatch {tuple(x.shape)} x {tuple(weight.shape)}")
    if x.stride(1) != 1 or weight.stride(1) != 1:
        return None
    m, k = x.shape
    n = weight.shape[0]
    out = torch.empty(m, n, dtype=out_dtype, device=x.device)
    if bias is not None and (bias.dtype is not torch.bfloat16 or not bias.is_contiguous()):
        return None
    L = _lib.lib()
    parts = None
    n_parts = 0
    if want_row_max:
        n_parts = int(L.ix_gemm_bf16_n_tiles(m, n, k, tile))
        parts = torch.empty(m, n_parts, dtype=torch.float32, device=x.device)
    stream = _lib.current_stream(x.device)
    rc = _lib.check(
        L.ix_gemm_bf16_nt(x.data_ptr(), x.stride(0), weight.data_ptr(), weight.stride(0), _lib.ptr(bias),
                          out.data_ptr(), _lib.dtype_code(out_dtype), out.stride(0), m, n, k, tile,
                          _lib.ptr(parts), n_parts, stream), "ix_gemm_bf16_nt")
    if rc != _lib.IX_OK:
        return None
    if not want_row_max:
        return out
    row_max = torch.empty(m, dtype=torch.float32, device=x.device)
    if m:
        _lib.check(L.ix_rowmax_reduce(parts.data_ptr(), n_parts, n_parts, m, row_max.data_ptr(), stream),
                   "ix_rowmax_reduce")
    return out, row_max


def router_gemm(x: torch.Tensor, weight: torch.Tensor):
    """Router gating logits in fp32. A bf16 router weight (exactly what an fp32 cast of a bf16
    checkpoint holds) multiplies exactly in the bf16 MFMA and is accumulated in fp32, so the bf16
    core with an fp32 store IS the fp32 gating product; an fp32 weight takes the fp32 kernel."""
    if weight.dtype is torch.bfloat16 and x.dtype is torch.bfloat16:
        return linear_nt(x, weight, out_dtype=torch.float32)
    return linear_f32_nt(x, weight.float())


def linear_f32_nt(x: torch.Tensor, weight: torch.Tensor):
    """Router gating: ``x [M, K]`` (bf16 or fp32) ``@ weight [N, K]^T`` (fp32) -> fp32."""
    _lib.require_device(x, weight)
    if weight.dtype is not torch.float32 or x.stride(1) != 1 or weight.stride(1) != 1:
        return None
    m, k = x.shape
    n = weight.shape[0]
    out = torch.empty(m, n, dtype=torch.float32, device=x.device)
    rc = _lib.check(
        _lib.lib().ix_gemm_f32_nt(x.data_ptr(), _lib.dtype_code(x.dtype), x.stride(0), weight.data_ptr(),
                                  weight.stride(0), out.data_ptr(), out.stride(0), m, n, k,
                                  _lib.current_stream(x.device)), "ix_gemm_f32_nt")
    return out if rc == _lib.IX_OK else None


def _as_nt(b: torch.Tensor):
    """``b [K, N]`` as a K-contiguous ``[N, K]`` matrix (free for the transposed view of a
    ``[N, K]`` weight, which is what ``F.linear`` hands to ``aten::mm``)."""
    bt = b.t()
    return bt if bt.stride(1) == 1 else bt.contiguous()


def mm_batch_invariant(a: torch.Tensor, b: torch.Tensor):
    out = None
    if a.dtype is torch.bfloat16 and b.dtype is torch.bfloat16:
        out = linear_nt(a if a.stride(1) == 1 else a.contiguous(), _as_nt(b))
    elif a.dtype is torch.float32 and b.dtype is torch.float32:
        out = linear_f32_nt(a if a.stride(1) == 1 else a.contiguous(), _as_nt(b))
    if out is None:
        _COUNTS["declined"] += 1
        raise RuntimeError(
            f"[isoexec-amd] mm override declined {tuple(a.shape)}x{tuple(b.shape)} {a.dtype}/{b.dtype}: "
            "no batch-invariant kernel for this signature")
    _COUNTS["mm"] += 1
    return out


def addmm_batch_invariant(bias, a, b, *, beta=1, alpha=1):
    if beta != 1 or alpha != 1 or bias.ndim != 1 or a.dtype is not torch.bfloat16:
        raise RuntimeError("[isoexec-amd] addmm override serves bias[N] + a@b with alpha=beta=1 in bf16 only")
    out = linear_nt(a if a.stride(1) == 1 else a.contiguous(), _as_nt(b), bias.contiguous())
    if out is None:
        _COUNTS["declined"] += 1
        raise RuntimeError("[isoexec-amd] addmm override declined")
    _COUNTS["addmm"] += 1
    return out


def bmm_batch_invariant(a, b):
    _COUNTS["bmm"] += 1
    return torch.stack([mm_batch_invariant(a[i], b[i]) for i in range(a.shape[0])])


def install_mm_override() -> bool:
    """Route ``aten::mm/addmm/bmm`` on device tensors to the kernel (moe_batch_invariant.py:453-464)."""
    global _LIBRARY
    if _LIBRARY is not None:
        return True
    _lib.lib()
    library = torch.library.Library("aten", "IMPL")
    library.impl("aten::mm", mm_batch_invariant, "CUDA")
    library.impl("aten::addmm", addmm_batch_invariant, "CUDA")
    library.impl("aten::bmm", bmm_batch_invariant, "CUDA")
    _LIBRARY = library
    return True


def uninstall_mm_override() -> None:
    global _LIBRARY
    _LIBRARY = None
