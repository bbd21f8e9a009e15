"""Installing the file trace on the package's doors: every function a region of the registry is served by gets
``trace.wrap_region`` around it, so whatever kernel a side actually runs is what its trace records.

``install_debug_hooks()`` does nothing unless ``SKYRL_ISOEXEC_DEBUG_TRACE`` is set. A door is a module-level function
(or a method, ``"Class.method"``) named in ``DOORS`` by the module that defines it. Python binds imported functions by
value -- ``from .gdn_ops import gdn_l2norm`` leaves a second binding in the importing module -- so after wrapping the
definition the installer rebinds every other binding of the SAME function object it finds in the package's loaded
modules (the reference lists those namespaces by hand, isoexec/debug/install.py:107-186; here they are found).
A door must be the same mathematical point on both sides, or the comparison compares different quantities: the
table names ops, not runtimes. ``coverage()`` says, per registry region, which doors exist, which regions have only part
of the op behind a door and which have none, so that coverage never overstates itself (install.py:189-222, 271-281).
"""

from __future__ import annotations

import importlib
import sys
from typing import Callable, Dict, List, Optional, Tuple

from . import trace

_PKG = __name__.rsplit(".", 2)[0]  # "isoexec_amd"


def _first(out):
    """Doors that return ``(tensor, None)`` (the expert door's Megatron signature): the tensor is the region's output."""
    return out[0] if isinstance(out, tuple) and out else out


def _first_two(out):
    return tuple(out[:2])


# (region, module below the package, attribute, keyword arguments of wrap_region)
DOORS: Tuple[Tuple[str, str, str, dict], ...] = (
    ("attention.varlen", "ops.attention.varlen_attn", "varlen_attention", {}),
    ("gdn.conv", "ops.gdn.gdn_ops", "gdn_causal_conv", {}),
    ("gdn.conv", "ops.gdn.gdn_ops", "gdn_causal_conv_batched", {}),
    ("gdn.conv", "ops.gdn.gdn_ops", "conv_packed", {}),
    ("gdn.core", "ops.gdn.gdn_ops", "gdn_core", {}),
    ("gdn.core", "ops.gdn.gdn_ops", "gdn_recurrent", {}),
    ("gdn.core", "ops.gdn.gdn_ops", "gdn_cpr", {}),
    ("gdn.core", "ops.gdn.gdn_ops", "gdn_native_core", {}),
    ("gdn.core", "ops.gdn.gdn_ops", "gdn_recurrent_kernel", {}),
    ("gdn.core", "ops.gdn.gdn_ops", "gdn_native_core_kernel", {}),
    ("gdn.core", "ops.gdn.gdn_cpr", "gdn_cpr_fwd", {}),
    ("gdn.core", "ops.gdn.gdn_cpr", "gdn_native_cpr_fwd", {}),
    ("gdn.gating", "ops.gdn.gdn_ops", "gdn_gate_and_beta", {}),
    ("gdn.gating", "ops.gdn.gdn_ops", "gate_and_beta_fp32", {}),
    ("gdn.gating", "ops.gdn.gdn_cpr", "native_matched_prep", {}),
    ("gdn.l2norm", "ops.gdn.gdn_ops", "gdn_l2norm", {}),
    ("gdn.state", "ops.gdn.gdn_cpr", "chunk_boundary_states", {}),
    ("logprobs.log_softmax", "ops.logprobs.rowinv", "rowinv_sampled_logprobs", {}),
    ("logprobs.log_softmax", "ops.logprobs.rowinv", "rowinv_full_logprobs", {}),
    ("logprobs.log_softmax", "ops.logprobs.rowinv", "sampled_forward", {}),
    ("logprobs.log_softmax", "ops.logprobs.rowinv", "full_forward", {}),
    ("mm", "ops.mm.mm_hip", "linear_nt", {}),
    ("moe.blockmap", "ops.moe.moe_hip", "permute", {"out_fn": lambda p: p.tile_meta}),
    ("moe.combine", "ops.moe.moe_doors", "_deterministic_unpermute", {}),
    ("moe.combine", "ops.moe.moe_hip", "combine", {}),
    ("moe.dispatch", "ops.moe.moe_doors", "_dispatch_postprocess_fixed_shape", {}),
    ("moe.experts", "ops.moe.moe_doors", "_batched_experts_forward", {"out_fn": _first}),
    ("moe.experts", "ops.moe.moe_hip", "experts_forward", {}),
    ("moe.router", "ops.moe.moe_doors", "topk_router_routing", {}),
    # the router's decision: top-k expert ids and weights. route_and_permute calls router_topk for large batches; a region
    # that re-enters itself is recorded once, at the outside, so both sizes leave one record per call of the layer
    ("moe.router", "ops.moe.moe_hip", "route_and_permute", {"out_fn": _first_two}),
    ("moe.router", "ops.moe.moe_hip", "router_topk", {"out_fn": _first_two}),
    ("moe.router", "ops.moe.moe_hip", "fused_router_dense", {}),
    ("norms.gated_out", "ops.norms.fused_outnorm", "fused_gated_out_norm", {}),
    ("norms.rms", "ops.norms.fused_outnorm", "fused_rms_norm_gamma", {}),
    ("norms.rms", "ops.norms.fused_outnorm", "fused_add_rms_norm_gamma", {}),
    ("norms.rms", "ops.norms.fused_outnorm", "ZeroCenteredRMSNorm.forward", {}),
    ("rope.rope", "ops.rope.rope_hip", "apply_rope_", {}),
)

# Region -> why no door of its own.
NOT_HOOKED: Dict[str, str] = {
    "logprobs.lm_head_slice": "no callable of its own here: the LM head is one call of the mm door (region `mm`).",
    "moe.epilogue": "inside the first expert GEMM's kernel (SwiGLU and routing weight in its epilogue): its output is the "
                    "intermediate of the `moe.experts` door, which `experts_forward(..., return_inter=True)` exposes.",
    "moe.weights": "the stacked expert weights are the checkpoint's tensors, not the output of a call.",
}

# Regions whose doors cover only part of the op.
PARTIAL: Dict[str, str] = {
    "gdn.state": "read side only (chunk_boundary_states): the pools are advanced in place by the scan, there is no value "
                 "to digest at the write. The runtimes' per-layer records (`_Blocks.region_log`) see the state's effect.",
    "gdn.gating": "subsumed by the fused core when gating runs inside the scan's preparation (decode: ix_gdn_decode_prep).",
    "gdn.l2norm": "subsumed likewise in a decode step.",
    "moe.combine": "the runtimes fold combine + residual add + norm into one launch unless a region log is attached; with "
                   "the trace on they call the door.",
    "moe.blockmap": "a batch of at most one token tile computes its block map inside the router's launch "
                    "(route_and_permute); `permute` is the door of the larger ones.",
    "mm": "hooked, recorded only when SKYRL_ISOEXEC_DEBUG_REGIONS names it (every projection of every layer).",
}

_installed: List[Tuple[object, str, object]] = []  # (holder, name, what was bound there before)


def _resolve(module: str, attr: str):
    """(holder, name, current binding) of a module attribute or ``Class.method``; None if absent."""
    try:
        mod = importlib.import_module(f"{_PKG}.{module}")
    except Exception:  # noqa: BLE001 -- a module that does not import here is a skipped door, not a failure
        return None
    holder, name = mod, attr
    if "." in attr:
        cls_name, name = attr.split(".", 1)
        holder = getattr(mod, cls_name, None)
        if holder is None:
            return None
    if isinstance(holder, type):
        current = next((k.__dict__[name] for k in holder.__mro__ if name in k.__dict__), None)  # no descriptor protocol
    else:
        current = getattr(holder, name, None)
    return None if current is None else (holder, name, current)


def _rebind_elsewhere(fn: Callable, wrapped: Callable, skip) -> int:
    """Every other binding of ``fn`` itself in the package's loaded modules -> ``wrapped``."""
    n = 0
    for mod_name, mod in list(sys.modules.items()):
        if mod is None or not (mod_name == _PKG or mod_name.startswith(_PKG + ".")) or mod_name.startswith(__name__):
            continue
        for name, value in list(vars(mod).items()):
            if value is fn and (mod, name) != skip:
                setattr(mod, name, wrapped)
                _installed.append((mod, name, fn))
                n += 1
    return n


def install_debug_hooks() -> int:
    """Wrap every door whose region the trace wants. Returns the number of bindings changed (0 when tracing is off).
    Safe to call again (an already wrapped door is left alone) and after more modules were imported (their bindings of a
    wrapped door are caught up)."""
    if trace.get_tracer() is None:
        return 0
    changed = 0
    for region, module, attr, kw in DOORS:
        found = _resolve(module, attr)
        if found is None:
            continue
        holder, name, current = found
        raw = current.__func__ if isinstance(current, (staticmethod, classmethod)) else current
        if not callable(raw):
            continue
        inner = getattr(raw, "__wrapped__", None) if getattr(raw, "_ix_traced_region", None) else None
        if inner is not None:  # wrapped by an earlier call: only catch up on bindings imported since
            changed += _rebind_elsewhere(inner, raw, (holder, name))
            continue
        wrapped = trace.wrap_region(region, raw, **kw)
        if wrapped is raw:
            continue  # the allow list leaves this region out
        bound = staticmethod(wrapped) if isinstance(current, staticmethod) else (
            classmethod(wrapped) if isinstance(current, classmethod) else wrapped)
        setattr(holder, name, bound)
        _installed.append((holder, name, current))
        changed += 1
        if not isinstance(holder, type):
            changed += _rebind_elsewhere(raw, wrapped, (holder, name))
    return changed


def uninstall_debug_hooks() -> int:
    """Put back every binding ``install_debug_hooks`` changed."""
    n = len(_installed)
    while _installed:
        holder, name, before = _installed.pop()
        setattr(holder, name, before)
    return n


def coverage(regions: Optional[List[str]] = None) -> Dict[str, dict]:
    """Region -> {"status": hooked | partial | not_hooked | unknown, "doors": [...], "note": ...} for the registry's
    regions (or the given ones). ``unknown`` is a region the table says nothing about: a gap to close here."""
    if regions is None:
        from ..core.registry_build import build_registry

        regions = sorted(build_registry().ops)
    out: Dict[str, dict] = {}
    for region, module, attr, _kw in DOORS:
        entry = out.setdefault(region, {"status": "partial" if region in PARTIAL else "hooked", "doors": [],
                                        "note": PARTIAL.get(region)})
        entry["doors"].append(f"{module}:{attr}")
    for region, why in NOT_HOOKED.items():
        out.setdefault(region, {"status": "not_hooked", "doors": [], "note": why})
    for region in regions:
        out.setdefault(region, {"status": "unknown", "doors": [], "note": None})
    return out
