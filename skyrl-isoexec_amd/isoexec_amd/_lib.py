"""ctypes binding of ``libisoexec_hip.so`` (declared in ``include/isoexec_hip.h``).

The library is the product; there is no fallback. ``lib()`` raises if the shared object is
missing so a GPU box never silently serves an eager path.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_long, c_size_t, c_uint, c_uint64, c_void_p

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC_DIR = os.path.normpath(os.path.join(_PKG_DIR, "..", "csrc"))
LIB_PATH = os.path.join(CSRC_DIR, "libisoexec_hip.so")

IX_OK = 0
IX_DECLINED = 1
IX_ERR_SIZE = -3
DT_F32 = 0
DT_BF16 = 1

PRIM = {
    "exp": 0,
    "log": 1,
    "exp_fast": 2,
    "sigmoid": 3,
    "silu_div": 4,
    "softplus": 5,
    "rsqrt_ieee": 6,
    "round_bf16": 7,
    "exp2": 8,
}

P = c_void_p
# name -> (restype, argtypes); kept in header order so the export test can walk it.
SIGNATURES = {
    "ix_abi_version": (c_int, []),
    "ix_arch_tag": (c_char_p, []),
    "ix_prim_unary": (c_int, [c_int, P, P, c_long, P]),
    "ix_arch_selfcheck_workspace_bytes": (c_size_t, []),
    "ix_arch_selfcheck": (c_int, [P, c_size_t, P, P]),
    "ix_arch_selfcheck_probe": (c_int, [P, c_size_t, c_uint, P, P]),
    "ix_logprob_workspace_bytes": (c_size_t, [c_long, c_long, c_int]),
    "ix_logprob_rowinv_sampled": (
        c_int,
        [P, c_int, c_long, c_long, c_long, P, c_int, P, P, P, c_size_t, c_int, P, P],
    ),
    "ix_logprob_rowinv_full": (
        c_int,
        [P, c_int, c_long, c_long, c_long, c_int, P, c_long, P, P, c_size_t, c_int, P, P],
    ),
    "ix_rowmax_reduce": (c_int, [P, c_long, c_long, c_long, P, P]),
    "ix_rmsnorm_gamma": (c_int, [P, P, P, c_long, c_long, c_float, c_int, P]),
    "ix_gated_out_norm": (c_int, [P, P, c_long, P, P, c_long, c_long, c_long, c_float, c_int, P]),
    "ix_add_rmsnorm_gamma": (c_int, [P, P, P, P, P, c_long, c_long, c_float, c_int, P]),
    "ix_moe_combine_add_rmsnorm": (c_int, [P, P, c_long, c_int, P, P, P, P, c_long, c_long, c_float, c_int, P]),
    "ix_gemm_bf16_nt": (
        c_int,
        [P, c_long, P, c_long, P, P, c_int, c_long, c_long, c_long, c_long, c_int, P, c_long, P],
    ),
    "ix_gemm_bf16_n_tiles": (c_long, [c_long, c_long, c_long, c_int]),
    "ix_gemm_bf16_nt_batched": (
        c_int,
        [P, c_long, c_long, P, c_long, c_long, P, c_long, c_long, c_long, c_long, c_long, c_long, c_int, P],
    ),
    "ix_arena_create": (c_int, [c_size_t, P, P]),
    "ix_arena_base": (P, [P]),
    "ix_arena_bytes": (c_size_t, [P]),
    "ix_arena_is_mapped": (c_int, [P]),
    "ix_arena_release_memory": (c_int, [P]),
    "ix_arena_restore_memory": (c_int, [P, P]),
    "ix_arena_destroy": (c_int, [P]),
    "ix_gemm_decode_serves_shape": (c_int, [c_long, c_long]),
    "ix_gemm_pack_decode": (c_int, [P, c_long, P, c_long, c_long, P]),
    "ix_gemm_bf16_nt_decode": (c_int, [P, c_long, P, P, c_long, c_long, c_long, c_long, P]),
    "ix_gemm_f32_nt": (c_int, [P, c_int, c_long, P, c_long, P, c_long, c_long, c_long, c_long, P]),
    "ix_gdn_scan": (
        c_int,
        [P, P, P, P, P, P, c_int, c_long, c_long, c_long, P, P, P, c_long, c_long, c_long, c_long, c_long,
         c_long, c_float, c_int, P],
    ),
    "ix_gdn_l2norm": (c_int, [P, c_long, P, c_int, c_long, c_long, c_long, c_float, P]),
    "ix_gdn_cpr_scatter": (c_int, [P, c_long, P, c_long, P, P, P, P, P, P, P, P, P, c_int, c_long, c_long, c_long, c_long, c_long, c_long, P]),
    "ix_gdn_cpr_handoff": (c_int, [P, P, P, c_long, c_long, c_int, P]),
    "ix_gdn_resolve_rows": (c_int, [P, c_int, c_long, P, c_long, c_long, P, P, P, P, P]),
    "ix_gdn_gate": (c_int, [P, c_long, P, c_long, P, P, P, P, c_int, c_long, c_long, c_int, P]),
    "ix_gdn_decode_prep": (c_int, [P, c_long, P, c_long, P, c_long, P, P, P, P, P, P, P, P, P, c_long, c_long, c_long, c_long,
                                   c_long, c_long, c_int, c_float, P]),
    "ix_gdn_scan_gated_norm": (
        c_int,
        [P, P, P, P, P, P, c_long, c_long, c_long, P, P, P, c_long, c_long, c_long, c_long, c_long, c_float, c_int, P,
         c_long, P, c_float, c_int, P],
    ),
    "ix_gdn_conv": (c_int, [P, c_long, P, P, P, P, P, P, P, c_long, c_long, c_long, c_long, c_int, P]),
    "ix_gdn_conv_l2norm": (c_int, [P, c_long, P, P, P, P, P, P, P, c_long, c_long, c_long, c_long, c_int, c_long, c_long,
                                   c_float, P]),
    "ix_attn_varlen": (c_int, [P, c_long, P, P, c_long, P, P, P, P, c_long, c_long, c_long, c_long, c_long, c_float, P]),
    "ix_rope_inplace": (c_int, [P, c_long, P, P, c_long, P, c_long, c_long, c_long, c_long, P]),
    "ix_moe_router_topk": (c_int, [P, c_long, c_long, c_long, c_long, c_int, c_float, P, P, P, P, P]),
    "ix_moe_max_tiles": (c_long, [c_long, c_long, c_long, c_long]),
    "ix_moe_permute_scratch_ints": (c_size_t, [c_long, c_long]),
    "ix_moe_pick_bm": (c_int, [c_long, c_long, c_long]),
    "ix_moe_permute": (
        c_int,
        [P, P, c_long, c_long, c_long, c_long, P, P, P, P, P, P, c_long, P, P],
    ),
    "ix_moe_route_one_tile": (c_int, [P, c_long, c_long, c_long, c_long, c_int, c_float, c_long, P, P, P, P, P, P, P, P,
                                      c_long, P]),
    "ix_moe_block_map": (c_int, [P, c_int, c_long, c_long, c_long, P, P, c_long, P]),
    "ix_moe_permute_static_max_ints": (c_size_t, []),
    "ix_moe_permute_static_init": (c_int, []),
    "ix_moe_permute_static": (
        c_int,
        [P, P, c_long, c_long, c_long, c_long, P, P, P, P, P, P, c_long, P],
    ),
    "ix_moe_experts": (
        c_int,
        [P, c_long, P, P, P, P, P, c_long, c_long, P, P, c_long, c_long, c_long, c_long, P],
    ),
    "ix_moe_experts_tile": (
        c_int,
        [P, c_long, P, P, P, P, P, c_long, c_long, c_long, P, P, c_long, c_long, c_long, c_long, P],
    ),
    "ix_moe_pack_decode": (c_int, [P, P, P, P, c_long, c_long, c_long, P]),
    "ix_moe_experts_decode": (
        c_int,
        [P, c_long, P, P, P, P, P, c_long, P, P, c_long, c_long, c_long, c_long, P],
    ),
    "ix_moe_combine": (c_int, [P, P, P, c_long, c_long, c_long, c_int, P]),
    "ix_moe_combine_weighted": (c_int, [P, c_int, P, c_int, P, P, c_int, c_long, c_long, c_long, P]),
    "ix_digest_sums": (c_int, [P, c_int, c_long, c_uint64, P, c_int, P, c_size_t, P, P]),
    "ix_digest_segment_sums": (c_int, [P, c_int, c_long, c_long, c_long, c_uint64, c_uint64, P, c_size_t, P, P]),
    "ix_digest_workspace_words": (c_size_t, [c_long, c_long, c_int]),
}

_LIB = None
_DISABLED = None   # the reason, once the device self-check has failed: the library then serves nothing in this process


class IsoExecLibraryError(RuntimeError):
    pass


def lib() -> ctypes.CDLL:
    """Load (once) and return the shared library; raise loudly if it is not built."""
    global _LIB
    if _DISABLED is not None:
        raise IsoExecLibraryError(f"[isoexec-amd] the library is switched off for this process: {_DISABLED}")
    if _LIB is not None:
        return _LIB
    if not os.path.exists(LIB_PATH):
        raise IsoExecLibraryError(
            f"[isoexec-amd] {LIB_PATH} is missing: build it with `make -C {CSRC_DIR}` "
            "(or __graft_entry__.build()). There is no CPU or eager fallback."
        )
    handle = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(handle, name)  # AttributeError here means header and library disagree
        fn.restype = restype
        fn.argtypes = argtypes
    _LIB = handle
    return handle


def disable(reason: str) -> None:
    """Switch the library off for the rest of the process (a failed device self-check): every later ``lib()`` raises.
    There is no way back short of a new process, as for the reference's providers after a failed first-use check."""
    global _DISABLED
    _DISABLED = str(reason)


def disabled_reason():
    return _DISABLED


def check(rc: int, what: str) -> int:
    """Raise on an error code; return the code (0 launched, >0 declined) otherwise."""
    if rc < 0:
        raise IsoExecLibraryError(f"[isoexec-amd] {what} failed with code {rc}")
    return rc


def ptr(t) -> int | None:
    return None if t is None else t.data_ptr()


def current_stream(device=None) -> int:
    import torch

    return torch.cuda.current_stream(device).cuda_stream


def dtype_code(dtype) -> int:
    import torch

    if dtype is torch.float32:
        return DT_F32
    if dtype is torch.bfloat16:
        return DT_BF16
    raise IsoExecLibraryError(f"[isoexec-amd] unsupported dtype {dtype}")


def require_device(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise IsoExecLibraryError(
                f"[isoexec-amd] tensor on {t.device}: the HIP path only serves device tensors (no CPU fallback)"
            )


def prim_unary(name: str, x):
    """Elementwise device primitive (fp32 in, fp32 out) as the kernels evaluate it."""
    import torch

    require_device(x)
    xc = x.contiguous().to(torch.float32)
    y = torch.empty_like(xc)
    check(lib().ix_prim_unary(PRIM[name], xc.data_ptr(), y.data_ptr(), xc.numel(), current_stream(x.device)), name)
    return y
