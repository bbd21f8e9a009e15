#!/usr/bin/env python3
"""Offline comparison of two trace directories: where did the trainer and the engine first disagree?

    python -m isoexec_amd.debug TRACE_A TRACE_B [--regions r1,r2] [--layers N] [--case-a C] [--case-b C] [--json OUT]
    python path/to/compare.py TRACE_A TRACE_B            # the file has no imports beyond the standard library

A trace directory holds what ``debug.trace`` wrote: one ``*.jsonl`` file of records per process and one
``manifest-*.json`` beside it. Records are grouped by (region, layer, output path, rank), the two sides' groups are
aligned on ``step`` (else ``call``, else position), and every aligned pair is judged: equal digests agree; different
shapes or dtypes are a layout divergence; different digests a value divergence with the mantissa ladder's bound on its
size and the row slabs' note on its place; a record on one side only is an absent one. Divergences are ordered by when
the first side executed them, so the first one listed is the origin and later ones in the same rank are marked as
possibly inherited from it.

Exit status: 0 nothing diverges, 2 a divergence, 3 inconclusive (the two sides sampled disjoint sets of records, or
nothing could be paired), 1 unusable input.

Counterpart of the reference's comparator (isoexec/debug/compare.py:36-77 loading, :88-122 grouping and alignment,
:128-181 verdicts, :291-493 comparison, :707-742 command line); the exit codes and the record fields keep its meaning.
"""

from __future__ import annotations

import argparse
import glob
import json
import os
import sys
from typing import Dict, Iterable, List, Optional, Sequence, Tuple

FORMAT_VERSION = 3
STATUS_EXIT = {"clean": 0, "divergent": 2, "inconclusive": 3}


class BadTrace(Exception):
    """A directory that cannot be compared: missing, empty, malformed or of another format version."""


# ---- verdicts on one pair of records ---------------------------------------------------------------------------------

def ladder_verdict(a: dict, b: dict) -> Tuple[Optional[int], str]:
    """(the finest rung at which two records agree, what that says about the size of the difference). The bound is
    a maximum over elements, relative; a ladder that differs at every rung bounds nothing and is not called large."""
    la, lb = a.get("ladder") or {}, b.get("ladder") or {}
    shared = sorted((int(name[1:]) for name in set(la) & set(lb) if name.startswith("k")), reverse=True)
    if not shared:
        return None, "unknown (no ladder recorded on both sides)"
    agree = next((k for k in shared if la[f"k{k}"] == lb[f"k{k}"]), None)
    if agree is None:
        return None, ("not bounded by the ladder: differs at every rung down to k=0 (a sign or exponent difference, or "
                      "small differences in enough elements that some straddle every truncation boundary)")
    finer = [k for k in shared if k > agree]
    if not finer:
        return agree, f"< 2^-{agree} relative, max over elements (agrees at the finest rung recorded)"
    return agree, (f"between ~2^-{min(finer)} and 2^-{agree} relative, max over elements (the upper end is a bound, the "
                   f"lower end holds if no element straddles the k={min(finer)} boundary)")


def differing_segments(mine: Sequence[str], theirs: Sequence[str]) -> List[int]:
    """Indices at which two lists of slab digests differ (a length mismatch is every index)."""
    if len(mine) != len(theirs):
        return list(range(max(len(mine), len(theirs))))
    return [i for i, (x, y) in enumerate(zip(mine, theirs)) if x != y]


def segment_note(a: dict, b: dict) -> Optional[str]:
    """Which slabs of rows differ, when both records carry slab digests of the same count."""
    sa, sb = a.get("segments"), b.get("segments")
    if not sa or not sb or len(sa) != len(sb):
        return None
    differing = differing_segments(sa, sb)
    if not differing:
        return f"all {len(sa)} row segments match (the difference is below segment resolution)"
    if len(differing) == len(sa):
        return f"all {len(sa)} row segments differ: a whole-tensor difference, not one confined to some rows"
    rows = a.get("seg_rows") or 0
    first = differing[0]
    span = f", rows {first * rows}..{(first + 1) * rows - 1}" if rows else ""
    return f"{len(differing)} of {len(sa)} row segments differ (first: segment {first}{span})"


# ---- loading ---------------------------------------------------------------------------------------------------------

def load_dir(path: str) -> List[dict]:
    """Every record of every ``*.jsonl`` file of a trace directory (a single file is taken as it is). A truncated last
    line -- a process killed in the middle of a write -- is dropped; a malformed line elsewhere is an error."""
    files = [path] if os.path.isfile(path) else sorted(glob.glob(os.path.join(path, "*.jsonl")))
    if not files:
        raise BadTrace(f"{path}: no *.jsonl trace files")
    records: List[dict] = []
    for name in files:
        with open(name) as fh:
            lines = fh.read().split("\n")
        body = [(i, ln) for i, ln in enumerate(lines, 1) if ln.strip()]
        for pos, (lineno, ln) in enumerate(body):
            try:
                rec = json.loads(ln)
            except ValueError as exc:
                if pos == len(body) - 1:
                    break
                raise BadTrace(f"{name}:{lineno}: not JSON ({exc})") from None
            if not isinstance(rec, dict) or "region" not in rec:
                raise BadTrace(f"{name}:{lineno}: not a trace record")
            if rec.get("v") != FORMAT_VERSION:
                raise BadTrace(f"{name}:{lineno}: record format {rec.get('v')!r}, this tool reads {FORMAT_VERSION}")
            rec["_file"] = os.path.basename(name)
            records.append(rec)
    if not records:
        raise BadTrace(f"{path}: trace files hold no records")
    return records


def load_manifests(path: str) -> List[dict]:
    """The ``manifest-*.json`` files of a directory (none for a single file or an old trace: the comparison then works
    from the records alone)."""
    out = []
    if os.path.isdir(path):
        for name in sorted(glob.glob(os.path.join(path, "manifest-*.json"))):
            try:
                with open(name) as fh:
                    out.append(json.load(fh))
            except ValueError as exc:
                raise BadTrace(f"{name}: not JSON ({exc})") from None
    return out


# ---- comparison ------------------------------------------------------------------------------------------------------

def _layer(rec: dict, layers: Optional[int]) -> Optional[int]:
    if rec.get("layer") is not None:
        return rec["layer"]
    return (rec.get("call", 1) - 1) % layers if layers else None


def _groups(recs: Iterable[dict], case: Optional[str], layers: Optional[int], regions) -> Dict[tuple, List[dict]]:
    out: Dict[tuple, List[dict]] = {}
    for rec in recs:
        if (case and rec.get("case") != case) or (regions and rec["region"] not in regions):
            continue
        out.setdefault((rec["region"], _layer(rec, layers), str(rec.get("out", "0")), rec.get("rank")), []).append(rec)
    for group in out.values():
        group.sort(key=lambda r: (r.get("ts") or 0.0, r.get("seq") or 0))
    return out


def _align(ga: List[dict], gb: List[dict]) -> Tuple[List[Tuple[Optional[dict], Optional[dict]]], str]:
    """Pairs of records of two groups. A field that both sides hold and that is unique within each group is a key, so a
    record missing on one side leaves a hole instead of shifting every later pair; position is the last resort."""
    for field in ("step", "call"):
        ka, kb = [r.get(field) for r in ga], [r.get(field) for r in gb]
        if None not in ka and None not in kb and len(set(ka)) == len(ka) and len(set(kb)) == len(kb):
            da, db = dict(zip(ka, ga)), dict(zip(kb, gb))
            return [(da.get(k), db.get(k)) for k in sorted(set(ka) | set(kb))], field
    n = max(len(ga), len(gb))
    return [(ga[i] if i < len(ga) else None, gb[i] if i < len(gb) else None) for i in range(n)], "position"


def _coverage(recs: List[dict], manifests: List[dict]) -> dict:
    steps = {r["step"] for r in recs if r.get("step") is not None}
    seen = set()
    for m in manifests:
        seen.update(m.get("steps_seen") or [])
    labels = {m.get("side") for m in manifests} | {r.get("side") for r in recs}
    labels.discard(None)
    return {
        "label": "/".join(sorted(labels)) or "?",
        "records": len(recs),
        "ranks": sorted({r.get("rank") for r in recs}, key=str),
        "sample": max([int(m.get("sample") or 1) for m in manifests] or [1]),
        "step_signal": bool(steps) or any(m.get("step_signal") for m in manifests),
        "steps_recorded": sorted(steps),
        "steps_not_observed": sorted(seen - steps),
        "ladder": any("ladder" in r for r in recs),
        "segment_rows": max([int(r.get("seg_rows") or 0) for r in recs] or [0]),
        "capture_skipped": sum(int(m.get("capture_skipped") or 0) for m in manifests),
        "digest_backend": sorted({m.get("digest_backend") for m in manifests if m.get("digest_backend")}),
    }


def _disjoint(ca: dict, cb: dict) -> Optional[str]:
    if ca["sample"] <= 1 and cb["sample"] <= 1:
        return None
    if ca["step_signal"] != cb["step_signal"]:
        keyed, counted = ("A", "B") if ca["step_signal"] else ("B", "A")
        return (f"side {keyed} records every Nth step and side {counted} every Nth call of a region: they chose their "
                "records by different rules")
    sa, sb = set(ca["steps_recorded"]), set(cb["steps_recorded"])
    if sa and sb and not sa & sb:
        return "the two sides recorded disjoint sets of steps"
    return None


def _when(entry: dict) -> tuple:
    ts = entry.get("ts")
    return (ts is None, ts or 0.0, entry.get("seq") or 0, entry.get("step") or 0,
            entry["layer"] if entry.get("layer") is not None else 1 << 30, entry["out"], entry["region"])


def compare_records(recs_a: List[dict], recs_b: List[dict], *, case_a: Optional[str] = None, case_b: Optional[str] = None,
                    layers: Optional[int] = None, regions=None, manifests_a: Optional[List[dict]] = None,
                    manifests_b: Optional[List[dict]] = None) -> dict:
    """The report on two sides' records (see the module's text for the rules)."""
    cov_a, cov_b = _coverage(recs_a, manifests_a or []), _coverage(recs_b, manifests_b or [])
    ga, gb = _groups(recs_a, case_a, layers, regions), _groups(recs_b, case_b, layers, regions)
    per_region: Dict[str, dict] = {}
    divergences, unrecordable = [], []
    paired = 0
    for key in sorted(set(ga) & set(gb), key=repr):
        region, layer, out, rank = key
        stat = per_region.setdefault(region, {"compared": 0, "matched": 0, "mismatched": 0, "absent": 0,
                                              "unrecordable": 0, "aligned_on": set()})
        pairs, how = _align(ga[key], gb[key])
        stat["aligned_on"].add(how)
        for ra, rb in pairs:
            anchor = ra or rb
            base = {"region": region, "layer": layer, "out": out, "rank": rank, "step": anchor.get("step"),
                    "call": anchor.get("call"), "ts": (ra or {}).get("ts"), "seq": (ra or {}).get("seq")}
            if ra is None or rb is None:
                stat["absent"] += 1
                divergences.append(dict(base, kind="absent", magnitude=f"recorded by side {'B' if ra is None else 'A'} only"))
                continue
            stat["compared"] += 1
            paired += 1
            if "digest" not in ra or "digest" not in rb:
                stat["unrecordable"] += 1
                unrecordable.append(dict(base, a=ra.get("unrecordable"), b=rb.get("unrecordable")))
            elif ra.get("shape") != rb.get("shape") or ra.get("dtype") != rb.get("dtype"):
                stat["mismatched"] += 1
                divergences.append(dict(base, kind="layout", magnitude=f"{ra.get('shape')} {ra.get('dtype')} vs "
                                                                          f"{rb.get('shape')} {rb.get('dtype')}"))
            elif ra["digest"] == rb["digest"]:
                stat["matched"] += 1
            else:
                stat["mismatched"] += 1
                agree_k, magnitude = ladder_verdict(ra, rb)
                divergences.append(dict(base, kind="value", digests=[ra["digest"], rb["digest"]], agree_k=agree_k,
                                        magnitude=magnitude, segments=segment_note(ra, rb)))
    divergences.sort(key=_when)
    origin_of_rank: Dict[object, dict] = {}
    for entry in divergences:
        origin_of_rank.setdefault(entry["rank"], entry)
    for entry in divergences:
        entry["inherited"] = entry is not origin_of_rank[entry["rank"]]
    for stat in per_region.values():
        stat["aligned_on"] = sorted(stat["aligned_on"])
    only_a, only_b = sorted(set(ga) - set(gb), key=repr), sorted(set(gb) - set(ga), key=repr)
    ranks_differ = cov_a["ranks"] != cov_b["ranks"]
    reason = _disjoint(cov_a, cov_b)
    if reason is None and paired == 0:
        reason = "no record of one side has a counterpart on the other (other regions, layers, ranks or cases)"
    if reason is None and ranks_differ and not divergences:
        reason = f"side A holds ranks {cov_a['ranks']} and side B ranks {cov_b['ranks']}: some ranks have nothing to be compared with"
    status = "inconclusive" if reason else ("divergent" if divergences else "clean")
    return {"format_version": FORMAT_VERSION, "status": status, "inconclusive_because": reason,
            "sides": {"a": cov_a, "b": cov_b}, "regions": per_region, "paired": paired,
            "first_divergence": divergences[0] if divergences else None,
            "origins": [origin_of_rank[r] for r in sorted(origin_of_rank, key=str)], "divergences": divergences,
            "unrecordable": unrecordable, "keys_only_in_a": [list(k) for k in only_a],
            "keys_only_in_b": [list(k) for k in only_b]}


def compare_dirs(dir_a: str, dir_b: str, **kwargs) -> dict:
    return compare_records(load_dir(dir_a), load_dir(dir_b), manifests_a=load_manifests(dir_a),
                           manifests_b=load_manifests(dir_b), **kwargs)


# ---- text ------------------------------------------------------------------------------------------------------------

def _place(entry: dict) -> str:
    where = entry["region"] + ("" if entry["layer"] is None else f" @ layer {entry['layer']}")
    keys = ", ".join(f"{name} {entry[name]}" for name in ("rank", "step", "call") if entry.get(name) is not None)
    return f"{where}, output {entry['out']}" + (f" ({keys})" if keys else "")


def render_text(report: dict, max_listed: int = 12) -> str:
    a, b = report["sides"]["a"], report["sides"]["b"]
    lines = [f"A = {a['label']}: {a['records']} records, ranks {a['ranks']}, every {a['sample']} "
             f"{'steps' if a['step_signal'] else 'calls'};  B = {b['label']}: {b['records']} records, ranks {b['ranks']}, "
             f"every {b['sample']} {'steps' if b['step_signal'] else 'calls'}"]
    if a["digest_backend"] and b["digest_backend"] and a["digest_backend"] != b["digest_backend"]:
        lines.append(f"WARNING: digest backends differ ({a['digest_backend']} vs {b['digest_backend']}): digests of equal "
                     "tensors may not be equal")
    width = max([len(name) for name in report["regions"]] + [6])
    lines.append(f"{'region':<{width}}  compared  matched  differ  absent  undigested  aligned on")
    for name in sorted(report["regions"]):
        s = report["regions"][name]
        lines.append(f"{name:<{width}}  {s['compared']:>8}  {s['matched']:>7}  {s['mismatched']:>6}  {s['absent']:>6}  "
                     f"{s['unrecordable']:>10}  {','.join(s['aligned_on'])}")
    for side, keys in (("A", report["keys_only_in_a"]), ("B", report["keys_only_in_b"])):
        if keys:
            shown = "; ".join(f"{k[0]}@{k[1]} out {k[2]} rank {k[3]}" for k in keys[:4])
            lines.append(f"recorded by side {side} only: {len(keys)} (region, layer, output, rank) groups, e.g. {shown}")
    for side, cov in (("A", a), ("B", b)):
        if cov["steps_not_observed"]:
            lines.append(f"side {side} saw steps it did not record (sampling): {cov['steps_not_observed'][:16]}")
        if cov["capture_skipped"]:
            lines.append(f"side {side} skipped {cov['capture_skipped']} records under graph capture")
    if report["status"] == "inconclusive":
        lines.append(f"INCONCLUSIVE: {report['inconclusive_because']}")
    first = report["first_divergence"]
    if first is None:
        if report["status"] == "clean":
            lines.append(f"CLEAN: {report['paired']} paired region outputs, none differs")
    else:
        lines.append(f"FIRST DIVERGENCE ({first['kind']}): {_place(first)}")
        lines.append(f"  magnitude: {first['magnitude']}")
        if first.get("segments"):
            lines.append(f"  where: {first['segments']}")
        later = [d for d in report["divergences"] if d is not first]
        if later:
            lines.append(f"{len(later)} later divergences ({sum(d['inherited'] for d in later)} possibly inherited from an "
                         "earlier one of their rank):")
            for d in later[:max_listed]:
                lines.append(f"  {d['kind']:<6} {_place(d)}: {d['magnitude'][:80]}")
            if len(later) > max_listed:
                lines.append(f"  ... and {len(later) - max_listed} more")
    if report["unrecordable"]:
        lines.append(f"{len(report['unrecordable'])} paired outputs carry no digest on at least one side "
                     f"(first: {_place(report['unrecordable'][0])})")
    return "\n".join(lines)


# ---- command line ----------------------------------------------------------------------------------------------------

def main(argv=None) -> int:
    p = argparse.ArgumentParser(prog="isoexec_amd.debug", description=__doc__.splitlines()[0])
    p.add_argument("dir_a", help="first trace directory (say, the trainer's)")
    p.add_argument("dir_b", help="second trace directory (say, the engine's)")
    p.add_argument("--case-a", default=None, help="compare only A's records of this case")
    p.add_argument("--case-b", default=None, help="compare only B's records of this case")
    p.add_argument("--layers", type=int, default=None, help="layers per forward: folds the call count into a layer "
                                                            "for records that carry none")
    p.add_argument("--regions", default=None, help="comma-separated regions to compare (default: all)")
    p.add_argument("--json", dest="json_out", default=None, help="also write the whole report here as JSON")
    args = p.parse_args(argv)
    try:
        report = compare_dirs(args.dir_a, args.dir_b, case_a=args.case_a, case_b=args.case_b, layers=args.layers,
                              regions=set(args.regions.split(",")) if args.regions else None)
    except (BadTrace, OSError) as exc:
        print(f"compare: {exc}", file=sys.stderr)
        return 1
    print(render_text(report))
    if args.json_out:
        with open(args.json_out, "w") as fh:
            json.dump(report, fh, indent=1, default=str)
    return STATUS_EXIT[report["status"]]


if __name__ == "__main__":
    sys.exit(main())
