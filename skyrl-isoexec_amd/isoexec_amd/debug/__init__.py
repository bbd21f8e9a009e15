"""Debug aids for locating a trainer/engine mismatch: on-device digests of tensors (``thash``).

Nothing is imported until a name is asked for, so importing the package costs nothing in a run that never digests.
(The reference's ``isoexec/debug`` package re-exports the same digest names lazily: debug/__init__.py:8-35.)
"""

_DIGEST_NAMES = ("tensor_digest", "digest_ladder", "ladder_for", "segment_axis", "segment_digests",
                 "first_divergent_segments", "iter_tensor_outputs", "digest_backend")

__all__ = sorted(_DIGEST_NAMES + ("preload_digest",))


def __getattr__(name):
    if name in _DIGEST_NAMES or name == "preload_digest":
        from . import thash

        return thash.preload if name == "preload_digest" else getattr(thash, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
