"""Order-invariant 64-bit digests of device tensors, for comparing what two processes computed without moving it.

A digest is a position-weighted sum of the tensor's bit patterns modulo 2**64, finished with a header that folds in
the shape, the dtype and the truncation level. Integer addition is associative, so the value cannot depend on how
the sum was split over lanes and workgroups: equal logical contents give equal digests, on any device. Clearing the
low mantissa bits before summing gives a ladder of coarser digests; the finest rung at which two tensors still agree
brackets how far apart they are. Cutting the first axis with more than one row into slabs gives one digest per slab,
which locates a difference.

The names, arguments and values are those of the reference's ``isoexec/debug/thash.py`` (tensor_digest :251-266,
digest_ladder :269-301, segment_axis :304-315, segment_digests :318-354, iter_tensor_outputs :357-392). The sums are
computed by ``ix_digest_sums`` / ``ix_digest_segment_sums`` of the HIP library on the device that holds the tensor;
a tensor in host memory is refused (the library is the only backend), and so is an unsupported dtype.
"""

from __future__ import annotations

import ctypes
from typing import Dict, Iterable, List, Optional, Sequence, Tuple

import torch

from .._lib import IsoExecLibraryError, check, current_stream, lib

_WORD = (1 << 64) - 1
_GOLDEN = 0x9E3779B97F4A7C15
MAX_MASKS_PER_PASS = 8          # IX_DIGEST_MAX_MASKS
MAX_OUTPUT_DEPTH = 3
DEFAULT_CHUNK_NUMEL = 1 << 22   # accepted for compatibility; the device pass has no chunks


class _Kind:
    """How one dtype is digested: bytes per integer of its image, the mask that undoes the sign extension
    (None: all 64 bits), explicit mantissa bits (None: not a float), and the code the header carries."""

    __slots__ = ("elem_bytes", "width_mask", "mantissa", "code")

    def __init__(self, elem_bytes, width_mask, mantissa, code):
        self.elem_bytes, self.width_mask, self.mantissa, self.code = elem_bytes, width_mask, mantissa, code


def _kinds() -> Dict[torch.dtype, _Kind]:
    # (name, bytes, mask, mantissa bits) in the order that fixes the header's dtype codes: never reorder, only append
    rows = (
        ("bfloat16", 2, 0xFFFF, 7), ("float16", 2, 0xFFFF, 10), ("float32", 4, 0xFFFFFFFF, 23),
        ("float64", 8, None, 52), ("int8", 1, 0xFF, None), ("uint8", 1, 0xFF, None), ("int16", 2, 0xFFFF, None),
        ("int32", 4, 0xFFFFFFFF, None), ("int64", 8, None, None), ("bool", 1, 0x1, None),
        ("float8_e4m3fn", 1, 0xFF, 3), ("float8_e5m2", 1, 0xFF, 2), ("float8_e4m3fnuz", 1, 0xFF, 3),
        ("float8_e5m2fnuz", 1, 0xFF, 2), ("uint16", 2, 0xFFFF, None), ("uint32", 4, 0xFFFFFFFF, None),
        ("uint64", 8, None, None), ("complex64", 8, None, None), ("complex128", 8, None, None),
    )
    table = {}
    for position, (name, nbytes, mask, mantissa) in enumerate(rows):
        dtype = getattr(torch, name, None)
        if dtype is not None:
            table[dtype] = _Kind(nbytes, mask, mantissa, position + 1)
    return table


_KINDS = _kinds()

# mantissa bits -> the rungs recorded, finest first; about four bits apart, so a matching and a differing rung
# bracket the relative difference within a factor of 16
LADDER_BY_MANTISSA: Dict[int, Tuple[int, ...]] = {
    2: (1, 0),
    3: (2, 1, 0),
    7: (6, 4, 2, 0),
    10: (9, 7, 5, 3, 1, 0),
    23: (22, 18, 14, 10, 6, 2, 0),
    52: (48, 40, 32, 24, 16, 8, 0),
}
DEFAULT_LADDER: Tuple[int, ...] = (6, 4, 2, 0)


def _mix(z: int) -> int:
    """splitmix64's finaliser on a Python integer."""
    z &= _WORD
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _WORD
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _WORD
    return z ^ (z >> 31)


def _kind_of(t: torch.Tensor) -> _Kind:
    kind = _KINDS.get(t.dtype)
    if kind is None:
        raise TypeError(f"tensor_digest: unsupported dtype {t.dtype}")
    return kind


def mantissa_bits(dtype: torch.dtype) -> Optional[int]:
    kind = _KINDS.get(dtype)
    return None if kind is None else kind.mantissa


def ladder_for(dtype: torch.dtype) -> Tuple[int, ...]:
    """The truncation levels recorded for ``dtype``; none for a dtype without a mantissa."""
    bits = mantissa_bits(dtype)
    return () if bits is None else LADDER_BY_MANTISSA.get(bits, DEFAULT_LADDER)


def digest_backend(device) -> str:
    """Always ``"hip"``: there is one implementation. Raises if the library is not built."""
    lib()
    return "hip"


def preload(device=None) -> bool:
    """Load the library now rather than inside the first traced region. Nothing is compiled at run time."""
    lib()
    return True


def _mask_for(kind: _Kind, k: Optional[int]) -> Tuple[int, int]:
    """(the 64-bit mask applied to the sign-extended element, the mantissa bits kept or -1)."""
    mask = _WORD if kind.width_mask is None else kind.width_mask
    if kind.mantissa is None:
        return mask, -1
    if k is None or k >= kind.mantissa:
        return mask, kind.mantissa
    return mask & ~((1 << (kind.mantissa - k)) - 1), k


def _header(t: torch.Tensor, kind: _Kind, kept: int, seed: int) -> int:
    h = _mix(seed ^ _GOLDEN)
    h = _mix(h ^ (kept & 0xFF))
    h = _mix(h ^ _mix(kind.code))
    for extent in t.shape:
        h = _mix(h ^ ((extent + 1) & _WORD))
    return h


def _image(t: torch.Tensor) -> Tuple[torch.Tensor, int]:
    """(the tensor in logical row-major order on its device, how many integers its image has)."""
    if not t.is_cuda:
        raise IsoExecLibraryError(f"[isoexec-amd] digest of a tensor on {t.device}: digests are computed on the "
                                  "device that holds the tensor (no CPU fallback)")
    kind = _kind_of(t)
    flat = t.detach()
    if not flat.is_contiguous():
        flat = flat.contiguous()
    return flat, flat.numel() * flat.element_size() // kind.elem_bytes


def _words(device, count: int) -> torch.Tensor:
    return torch.empty(max(1, count), dtype=torch.int64, device=device)


def _read(out: torch.Tensor, count: int) -> List[int]:
    return [v & _WORD for v in out[:count].tolist()]


def _sums(flat: torch.Tensor, kind: _Kind, count: int, masks: Sequence[int], seed: int) -> List[int]:
    """One weighted sum per mask (at most eight), from a single pass over the data."""
    if not 1 <= len(masks) <= MAX_MASKS_PER_PASS:
        raise ValueError(f"{len(masks)} masks in one pass (1..{MAX_MASKS_PER_PASS})")
    handle = lib()
    need = handle.ix_digest_workspace_words(1, count, len(masks))
    work = _words(flat.device, need) if need else None
    out = _words(flat.device, len(masks))
    host_masks = (ctypes.c_uint64 * MAX_MASKS_PER_PASS)(*masks)
    salt = _mix(seed) ^ _GOLDEN
    with torch.cuda.device(flat.device):
        check(handle.ix_digest_sums(flat.data_ptr() if count else None, kind.elem_bytes, count, salt, host_masks,
                                    len(masks), None if work is None else work.data_ptr(), need, out.data_ptr(),
                                    current_stream(flat.device)), "ix_digest_sums")
    return _read(out, len(masks))


def tensor_digest(t: torch.Tensor, *, k: Optional[int] = None, seed: int = 0,
                  chunk_numel: int = DEFAULT_CHUNK_NUMEL) -> int:
    """The digest of ``t``'s logical contents; ``k`` first truncates float mantissas to k bits."""
    flat, count = _image(t)
    kind = _kind_of(t)
    mask, kept = _mask_for(kind, k)
    (body,) = _sums(flat, kind, count, [mask], seed)
    return _mix(body ^ _header(t, kind, kept, seed))


def digest_ladder(t: torch.Tensor, ks: Optional[Sequence[int]] = None, *, seed: int = 0,
                  chunk_numel: int = DEFAULT_CHUNK_NUMEL) -> Dict[str, str]:
    """``{"full": hex, "k6": hex, ...}``: full precision and every rung, all from one pass over the tensor. A dtype
    without a mantissa gets ``"full"`` only; rungs at or above the mantissa width are dropped. The bound a ladder
    gives is a maximum over elements: when many elements differ every rung breaks and it bounds nothing."""
    flat, count = _image(t)
    kind = _kind_of(t)
    levels: List[Optional[int]] = [None]
    if kind.mantissa is not None:
        levels.extend(k for k in (ladder_for(t.dtype) if ks is None else ks) if 0 <= k < kind.mantissa)
    out: Dict[str, str] = {}
    for first in range(0, len(levels), MAX_MASKS_PER_PASS):
        window = levels[first:first + MAX_MASKS_PER_PASS]
        plan = [_mask_for(kind, k) for k in window]
        bodies = _sums(flat, kind, count, [mask for mask, _ in plan], seed)
        for k, (_, kept), body in zip(window, plan, bodies):
            out["full" if k is None else f"k{k}"] = f"{_mix(body ^ _header(t, kind, kept, seed)):016x}"
    return out


def segment_axis(t: torch.Tensor) -> int:
    """The axis ``segment_digests`` cuts: the first whose extent exceeds 1 (0 if there is none). Everything in
    front of it has extent 1, so slabs of it are contiguous runs of the row-major image."""
    for axis, extent in enumerate(t.shape):
        if extent > 1:
            return axis
    return 0


def segment_digests(t: torch.Tensor, *, rows_per_segment: int = 1024, k: Optional[int] = None, seed: int = 0,
                    chunk_numel: int = DEFAULT_CHUNK_NUMEL) -> List[str]:
    """One digest per slab of ``rows_per_segment`` rows of ``segment_axis(t)``, every slab from one launch. A
    slab's weights count from the slab's start and are salted by its absolute offset, so slab i of one tensor is
    comparable with slab i of another of the same shape."""
    if t.dim() == 0 or t.numel() == 0:
        return [f"{tensor_digest(t, k=k, seed=seed):016x}"]
    flat, count = _image(t)
    kind = _kind_of(t)
    mask, kept = _mask_for(kind, k)
    rows = t.shape[segment_axis(t)]
    per = max(1, rows_per_segment)
    seg_numel = per * (count // rows)
    nseg = -(-rows // per)
    handle = lib()
    need = handle.ix_digest_workspace_words(nseg, seg_numel, 1)
    work = _words(flat.device, need) if need else None
    out = _words(flat.device, nseg)
    with torch.cuda.device(flat.device):
        check(handle.ix_digest_segment_sums(flat.data_ptr(), kind.elem_bytes, count, nseg, seg_numel, seed & _WORD,
                                            mask, None if work is None else work.data_ptr(), need, out.data_ptr(),
                                            current_stream(flat.device)), "ix_digest_segment_sums")
    head = _header(t, kind, kept, seed)
    return [f"{_mix(body ^ _mix(head ^ (s + 1))):016x}" for s, body in enumerate(_read(out, nseg))]


def first_divergent_segments(mine: Sequence[str], theirs: Sequence[str]) -> List[int]:
    """Indices at which two lists of slab digests of equal length differ (a length mismatch is every index)."""
    if len(mine) != len(theirs):
        return list(range(max(len(mine), len(theirs))))
    return [i for i, (a, b) in enumerate(zip(mine, theirs)) if a != b]


def iter_tensor_outputs(out, *, max_depth: int = MAX_OUTPUT_DEPTH) -> Iterable[Tuple[str, Optional[torch.Tensor]]]:
    """The tensors inside a region's return value as ``(path, tensor)``: a bare tensor is ``"0"``, members of
    tuples, lists and dicts get dotted paths (``"1.0"``, ``"aux.0"``), other leaves are skipped. A container met at
    ``max_depth`` is reported as ``(path, None)`` rather than dropped."""
    if isinstance(out, torch.Tensor):
        yield "0", out
        return
    pending = [("", out, 0)]
    while pending:
        path, node, depth = pending.pop(0)
        if isinstance(node, torch.Tensor):
            yield path, node
            continue
        if isinstance(node, dict):
            members = list(node.items())
        elif isinstance(node, (list, tuple)):
            members = list(enumerate(node))
        else:
            continue
        if depth >= max_depth:
            yield path, None
            continue
        children = [(f"{path}.{key}" if path else str(key), value, depth + 1) for key, value in members]
        pending[0:0] = children      # depth first, members in order
