"""Debug aids for locating a trainer/engine mismatch: on-device digests of tensors (``thash``), per-region logs of them
with their in-process comparison (``regions``), the environment-switched file trace (``trace``) and the offline
comparison of two trace directories (``compare``; ``python -m isoexec_amd.debug A B``).

Nothing is imported until a name is asked for, so importing the package costs nothing in a run that never digests.
(The reference's ``isoexec/debug`` package re-exports its names lazily in the same way: debug/__init__.py:8-35.)
"""

_DIGEST_NAMES = ("tensor_digest", "digest_ladder", "ladder_for", "segment_axis", "segment_digests",
                 "first_divergent_segments", "iter_tensor_outputs", "digest_backend")
_REGION_NAMES = ("RegionLog", "wrap_region", "compare", "render", "ladder_verdict", "segment_note")
_TRACE_NAMES = ("Tracer", "get_tracer", "set_step", "set_case", "flush", "layer_context")

__all__ = sorted(_DIGEST_NAMES + _REGION_NAMES + _TRACE_NAMES + ("preload_digest",))


def __getattr__(name):
    if name in _DIGEST_NAMES or name == "preload_digest":
        from . import thash

        return thash.preload if name == "preload_digest" else getattr(thash, name)
    if name in _REGION_NAMES:
        from . import regions

        return getattr(regions, name)
    if name in _TRACE_NAMES:
        from . import trace

        return getattr(trace, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
