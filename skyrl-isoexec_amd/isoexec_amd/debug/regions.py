"""Where two runs first disagree: per-region digests recorded in execution order, and their comparison.

A ``RegionLog`` belongs to one side (the trainer, the engine). Code that wants to be comparable calls
``log.record(region, output, layer=...)`` at the same points on both sides; each tensor of the output is reduced on the
device to a 64-bit digest (optionally with its mantissa ladder and per-slab digests), so a recorded run costs one pass
over each output and moves a few bytes to the host. ``compare`` pairs the records of two logs by (region, layer, output
path, occurrence) and reports every pair that differs, earliest first, with what the ladder says about the size of
the difference and what the slabs say about where it is.

This is the in-process core of the reference's debug mode: its capture layer writes the same kind of record to JSONL
files per process (isoexec/debug/trace.py:200-262) and an offline tool compares them (isoexec/debug/compare.py:123-181,
291-470). The record fields, the ladder verdict and the slab note keep the reference's meaning. ``debug.trace`` puts
the environment switches and the per-process files on top of this log, ``debug.compare`` is the offline tool.
"""

from __future__ import annotations

import json
from typing import Callable, Dict, List, Optional, Tuple

import torch

from . import thash
from .compare import ladder_verdict, segment_note  # noqa: F401 -- the verdicts are shared with the offline tool

FORMAT_VERSION = 3


def _capturing() -> bool:
    """A digest is read back by the host, which a stream under graph capture cannot serve."""
    return torch.cuda.is_available() and torch.cuda.is_current_stream_capturing()


class RegionLog:
    """The records of one side, in the order they were made."""

    def __init__(self, side: str, *, ladder: bool = False, segment_rows: int = 0) -> None:
        self.side = side
        self.ladder = bool(ladder)
        self.segment_rows = max(0, int(segment_rows))
        self.records: List[dict] = []
        self.capture_skipped = 0
        self._calls: Dict[Tuple[str, Optional[int]], int] = {}

    # -- recording
    def _describe(self, rec: dict, t: torch.Tensor) -> dict:
        rec["shape"] = list(t.shape)
        rec["dtype"] = str(t.dtype).replace("torch.", "")
        try:
            if self.ladder:
                rungs = thash.digest_ladder(t)
                rec["digest"] = rungs.pop("full")
                rec["ladder"] = rungs
            else:
                rec["digest"] = f"{thash.tensor_digest(t):016x}"
            if self.segment_rows and t.dim() > 0:
                rec["segments"] = thash.segment_digests(t, rows_per_segment=self.segment_rows)
                rec["seg_rows"] = self.segment_rows
                rec["seg_axis"] = thash.segment_axis(t)
        except Exception as exc:  # noqa: BLE001 -- an output that cannot be digested is reported, never dropped
            for key in ("digest", "ladder", "segments"):
                rec.pop(key, None)
            rec["unrecordable"] = f"{type(exc).__name__}: {exc}"
        return rec

    def record(self, region: str, out, *, layer: Optional[int] = None, case: Optional[str] = None) -> None:
        """Digest every tensor inside ``out`` (a tensor, or tuples / lists / dicts of them)."""
        if _capturing():
            self.capture_skipped += 1
            return
        call = self._calls.get((region, layer), 0) + 1
        self._calls[(region, layer)] = call
        made = []
        for path, t in thash.iter_tensor_outputs(out):
            rec = {"v": FORMAT_VERSION, "region": region, "case": case, "side": self.side, "layer": layer,
                   "call": call, "out": path}
            if t is None:
                rec["unrecordable"] = f"nested output deeper than {thash.MAX_OUTPUT_DEPTH} levels"
            else:
                self._describe(rec, t)
            made.append(rec)
        if not made:
            made.append({"v": FORMAT_VERSION, "region": region, "case": case, "side": self.side, "layer": layer,
                         "call": call, "out": "0", "unrecordable": f"no tensor outputs (got {type(out).__name__})"})
        for rec in made:
            rec["seq"] = len(self.records) + 1
            self.records.append(rec)

    def next_call(self, region: str, layer: Optional[int] = None) -> int:
        """The number the next call of ``region`` at ``layer`` will carry."""
        return self._calls.get((region, layer), 0) + 1

    def skip(self, region: str, layer: Optional[int] = None) -> int:
        """Count a call of ``region`` without digesting it (a caller that records only some calls keeps the call
        numbers of the others honest this way). Returns the call's number."""
        call = self._calls.get((region, layer), 0) + 1
        self._calls[(region, layer)] = call
        return call

    # -- persistence (one JSON object per line)
    def dump(self, path: str) -> None:
        with open(path, "w") as fh:
            for rec in self.records:
                fh.write(json.dumps(rec, sort_keys=True) + "\n")

    @classmethod
    def load(cls, path: str, side: Optional[str] = None) -> "RegionLog":
        with open(path) as fh:
            records = [json.loads(line) for line in fh if line.strip()]
        log = cls(side or (records[0]["side"] if records else "unknown"))
        log.records = records
        log.ladder = any("ladder" in r for r in records)
        log.segment_rows = max((int(r.get("seg_rows") or 0) for r in records), default=0)
        return log


def wrap_region(log: Optional[RegionLog], region: str, fn: Callable, *, layer: Optional[int] = None) -> Callable:
    """``fn`` itself when there is no log; otherwise ``fn`` with its return value recorded under ``region``."""
    if log is None:
        return fn

    def recorded(*args, **kwargs):
        out = fn(*args, **kwargs)
        log.record(region, out, layer=layer)
        return out

    recorded.__wrapped__ = fn
    return recorded


def _pairing_key(rec: dict) -> tuple:
    return rec["region"], rec.get("layer"), rec.get("out"), rec.get("call")


def compare(mine: RegionLog, theirs: RegionLog) -> dict:
    """Pair the records of two logs and list the pairs that differ in ``mine``'s execution order.

    ``mismatches`` holds one entry per differing pair: the key, both digests, shapes, the ladder verdict and the slab
    note; ``first`` is the earliest of them (None when everything paired agrees); ``unpaired`` lists keys present on
    one side only; ``unrecordable`` the records that carry no digest. A pair whose shapes or dtypes differ is reported
    as a mismatch of kind "layout": the digest folds both, so such a pair could never agree."""
    other = {_pairing_key(rec): rec for rec in theirs.records}
    seen, mismatches, unrecordable, matched = set(), [], [], 0
    for rec in mine.records:
        key = _pairing_key(rec)
        seen.add(key)
        twin = other.get(key)
        if twin is None:
            continue
        if "digest" not in rec or "digest" not in twin:
            unrecordable.append({"key": key, mine.side: rec.get("unrecordable"), theirs.side: twin.get("unrecordable")})
            continue
        if rec["digest"] == twin["digest"]:
            matched += 1
            continue
        entry = {"region": rec["region"], "layer": rec.get("layer"), "out": rec.get("out"), "call": rec.get("call"),
                 "seq": rec.get("seq"), "digests": (rec["digest"], twin["digest"]),
                 "shapes": (rec.get("shape"), twin.get("shape"))}
        if rec.get("shape") != twin.get("shape") or rec.get("dtype") != twin.get("dtype"):
            entry["kind"] = "layout"
            entry["magnitude"] = "not comparable: shape or dtype differs, and the digest folds both"
        else:
            entry["kind"] = "value"
            entry["agree_k"], entry["magnitude"] = ladder_verdict(rec, twin)
            entry["segments"] = segment_note(rec, twin)
        mismatches.append(entry)
    unpaired = sorted(set(other) ^ seen, key=repr)
    return {"sides": (mine.side, theirs.side), "matched": matched, "mismatches": mismatches,
            "first": mismatches[0] if mismatches else None, "unpaired": unpaired, "unrecordable": unrecordable,
            "capture_skipped": (mine.capture_skipped, theirs.capture_skipped)}


def render(report: dict) -> str:
    """A few lines of text for a report of ``compare``."""
    a, b = report["sides"]
    lines = [f"{a} vs {b}: {report['matched']} region outputs agree, {len(report['mismatches'])} differ, "
             f"{len(report['unpaired'])} on one side only"]
    first = report["first"]
    if first is None:
        lines.append("no divergence in what both sides recorded")
    else:
        where = first["region"] + ("" if first["layer"] is None else f" @ layer {first['layer']}")
        lines.append(f"first divergence: {where}, output {first['out']}, call {first['call']} ({first['kind']})")
        lines.append(f"  magnitude: {first['magnitude']}")
        if first.get("segments"):
            lines.append(f"  segments: {first['segments']}")
    if any(report["capture_skipped"]):
        lines.append(f"records skipped under graph capture: {report['capture_skipped']}")
    return "\n".join(lines)
