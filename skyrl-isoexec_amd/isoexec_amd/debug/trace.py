"""File trace of a run's region outputs, switched on from the environment.

Nothing happens unless ``SKYRL_ISOEXEC_DEBUG_TRACE`` names a directory: ``get_tracer()`` is then ``None`` and
``wrap_region`` returns the function it was given. With the switch set, every process writes its records to
``{dir}/{side}-r{rank}-{host}-{pid}.jsonl`` (one JSON object per line, appended in bursts) and keeps
``manifest-{side}-r{rank}-{host}-{pid}.json`` beside it up to date; two such directories are what
``python -m isoexec_amd.debug A B`` compares.

Switches, read once when the tracer is first asked for (same names and meaning as the reference's capture layer,
isoexec/debug/trace.py:7-16):

  SKYRL_ISOEXEC_DEBUG_TRACE     directory to write into (the master switch)
  SKYRL_ISOEXEC_DEBUG_SIDE      "trainer" | "engine": labels the records and names the file (default "unknown")
  SKYRL_ISOEXEC_DEBUG_SAMPLE    N: record every Nth step once ``set_step`` has been called, else every Nth call of a
                                region (default 1). Both sides must choose by the same rule to be comparable.
  SKYRL_ISOEXEC_DEBUG_LADDER    "1": also the mantissa ladder of every output (bounds the size of a difference)
  SKYRL_ISOEXEC_DEBUG_SEGMENTS  R: also one digest per R rows of the first non-unit dimension (places a difference)
  SKYRL_ISOEXEC_DEBUG_REGIONS   comma-separated allow list; default: every region except the high-volume ones
  SKYRL_ISOEXEC_DEBUG_RING      records held in memory before they are appended to the file (default 4096)

The digesting itself is ``regions.RegionLog``'s: one pass over each output on the device, a few bytes to the host.
Records made while the stream is being captured into a graph are skipped and counted (a digest is read back by the
host, which a capture cannot serve).
"""

from __future__ import annotations

import atexit
import json
import os
import socket
import threading
import time
from typing import Callable, List, Optional

from .compare import FORMAT_VERSION

ENV_TRACE = "SKYRL_ISOEXEC_DEBUG_TRACE"
ENV_SIDE = "SKYRL_ISOEXEC_DEBUG_SIDE"
ENV_SAMPLE = "SKYRL_ISOEXEC_DEBUG_SAMPLE"
ENV_LADDER = "SKYRL_ISOEXEC_DEBUG_LADDER"
ENV_SEGMENTS = "SKYRL_ISOEXEC_DEBUG_SEGMENTS"
ENV_REGIONS = "SKYRL_ISOEXEC_DEBUG_REGIONS"
ENV_RING = "SKYRL_ISOEXEC_DEBUG_RING"

# recorded only when the allow list names them: a matrix product runs once per projection per layer per micro-batch
HIGH_VOLUME_REGIONS = frozenset({"mm"})

_lock = threading.Lock()
_tracer: Optional["Tracer"] = None
_tracer_resolved = False


def enabled() -> bool:
    return bool(os.environ.get(ENV_TRACE))


def _int_env(name: str, default: int, least: int) -> int:
    raw = os.environ.get(name, "")
    try:
        return max(least, int(raw)) if raw.strip() else default
    except ValueError:
        raise ValueError(f"{name}={raw!r} is not an integer") from None


def process_rank() -> int:
    """This process's rank as the launcher exported it (0 for a process started alone)."""
    for name in ("RANK", "LOCAL_RANK"):
        raw = os.environ.get(name, "")
        if raw.strip().isdigit():
            return int(raw)
    return 0


class Tracer:
    """One process's trace: samples, digests through a ``RegionLog``, buffers, appends to its file.

    ``digest_log`` may be handed in (any object with ``record``, ``next_call``, ``skip``, ``records`` and ``capture_skipped`` as
    ``RegionLog`` has them); by default a ``RegionLog`` is made on first use, which is when the device digest is loaded.
    """

    def __init__(self, trace_dir: str, *, side: str = "unknown", sample: int = 1, ladder: bool = False,
                 segment_rows: int = 0, regions: Optional[List[str]] = None, ring: int = 4096,
                 rank: Optional[int] = None, digest_log=None) -> None:
        self.dir = trace_dir
        self.side = side
        self.sample = max(1, int(sample))
        self.ladder = bool(ladder)
        self.segment_rows = max(0, int(segment_rows))
        self.regions = frozenset(regions) if regions else None
        self.ring = max(1, int(ring))
        self.rank = process_rank() if rank is None else int(rank)
        self.host = socket.gethostname().split(".")[0] or "host"
        self.pid = os.getpid()
        stem = f"{self.side}-r{self.rank}-{self.host}-{self.pid}"
        os.makedirs(self.dir, exist_ok=True)
        self.path = os.path.join(self.dir, stem + ".jsonl")
        self.manifest_path = os.path.join(self.dir, f"manifest-{stem}.json")
        self.step: Optional[int] = None
        self.case: Optional[str] = None
        self.started = time.time()
        self.written = 0
        self._log = digest_log
        self._buf: List[dict] = []
        self._seq = 0
        self._steps_seen: set = set()
        self._steps_recorded: set = set()
        self._depth: dict = {}
        self._local = threading.local()
        self._io = threading.Lock()
        self.write_manifest()

    @classmethod
    def from_env(cls) -> Optional["Tracer"]:
        trace_dir = os.environ.get(ENV_TRACE, "")
        if not trace_dir:
            return None
        allow = [r.strip() for r in os.environ.get(ENV_REGIONS, "").split(",") if r.strip()]
        return cls(trace_dir, side=os.environ.get(ENV_SIDE, "unknown") or "unknown", sample=_int_env(ENV_SAMPLE, 1, 1),
                   ladder=os.environ.get(ENV_LADDER, "") == "1", segment_rows=_int_env(ENV_SEGMENTS, 0, 0),
                   regions=allow or None, ring=_int_env(ENV_RING, 4096, 1))

    # -- what is recorded
    def wants(self, region: str) -> bool:
        if self.regions is not None:
            return region in self.regions
        return region not in HIGH_VOLUME_REGIONS

    def set_step(self, step: int) -> None:
        self.step = int(step)
        self._steps_seen.add(self.step)

    def _sampled(self, call: int) -> bool:
        if self.step is not None:
            return self.step % self.sample == 0
        return (call - 1) % self.sample == 0

    def current_layer(self) -> Optional[int]:
        return getattr(self._local, "layer", None)

    def _digest_log(self):
        if self._log is None:
            from .regions import RegionLog

            self._log = RegionLog(self.side, ladder=self.ladder, segment_rows=self.segment_rows)
        return self._log

    def record(self, region: str, out, *, layer: Optional[int] = None, case: Optional[str] = None) -> None:
        """Digest ``out`` under ``region`` if the allow list and the sampling rule select this call."""
        if not self.wants(region):
            return
        layer_src = "caller" if layer is not None else None
        if layer is None and self.current_layer() is not None:
            layer, layer_src = self.current_layer(), "context"
        log = self._digest_log()
        # the log numbers the calls of (region, layer); a call that is not sampled still takes its number
        if not self._sampled(log.next_call(region, layer)):
            log.skip(region, layer)
            return
        log.record(region, out, layer=layer, case=case if case is not None else self.case)
        made, log.records = log.records, []
        now = time.time()
        with self._io:
            for rec in made:
                self._seq += 1
                rec.update(seq=self._seq, ts=now, rank=self.rank, pid=self.pid, step=self.step, layer_src=layer_src)
                self._buf.append(rec)
            if made and self.step is not None:
                self._steps_recorded.add(self.step)
            full = len(self._buf) >= self.ring
        if full:
            self.flush()

    # -- files
    def manifest(self) -> dict:
        log = self._log
        backend = None
        if log is not None and type(log).__module__.endswith("regions"):
            from . import thash

            backend = thash.digest_backend(None)
        return {"v": FORMAT_VERSION, "side": self.side, "rank": self.rank, "host": self.host, "pid": self.pid,
                "file": os.path.basename(self.path), "started": self.started, "updated": time.time(),
                "sample": self.sample, "ladder": self.ladder, "segment_rows": self.segment_rows,
                "regions": sorted(self.regions) if self.regions is not None else None,
                "step_signal": bool(self._steps_seen), "steps_seen": sorted(self._steps_seen),
                "steps_recorded": sorted(self._steps_recorded), "records": self.written + len(self._buf),
                "capture_skipped": int(getattr(log, "capture_skipped", 0) or 0), "digest_backend": backend}

    def write_manifest(self) -> None:
        tmp = self.manifest_path + ".tmp"
        with open(tmp, "w") as fh:
            json.dump(self.manifest(), fh, indent=1, sort_keys=True)
        os.replace(tmp, self.manifest_path)  # a reader never sees half a manifest

    def flush(self) -> None:
        """Append what is buffered to the file and bring the manifest up to date."""
        with self._io:
            pending, self._buf = self._buf, []
            if pending:
                with open(self.path, "a") as fh:
                    fh.write("".join(json.dumps(rec, sort_keys=True) + "\n" for rec in pending))
                self.written += len(pending)
            self.write_manifest()


def get_tracer() -> Optional[Tracer]:
    """The process's tracer, made from the environment on the first call; ``None`` when tracing is off."""
    global _tracer, _tracer_resolved
    if _tracer_resolved:
        return _tracer
    with _lock:
        if not _tracer_resolved:
            _tracer = Tracer.from_env()
            if _tracer is not None:
                atexit.register(_tracer.flush)
            _tracer_resolved = True
    return _tracer


def set_step(step: int) -> None:
    """Tell the trace which training step (or engine request round) the following records belong to. With a sample
    rate above 1 it has to be called on BOTH sides, or the sides choose their records by different rules."""
    tracer = get_tracer()
    if tracer is not None:
        tracer.set_step(step)


def set_case(case: Optional[str]) -> None:
    """Label the following records (``--case-a`` / ``--case-b`` of the comparison select by it)."""
    tracer = get_tracer()
    if tracer is not None:
        tracer.case = case


def flush() -> None:
    tracer = get_tracer()
    if tracer is not None:
        tracer.flush()


def _forget_for_tests() -> None:
    global _tracer, _tracer_resolved
    with _lock:
        if _tracer is not None:
            atexit.unregister(_tracer.flush)
        _tracer, _tracer_resolved = None, False


class layer_context:
    """``with layer_context(i):`` -- records made inside carry layer ``i`` unless their caller names one."""

    def __init__(self, layer: Optional[int]) -> None:
        self.layer = layer
        self._before = None
        self._tracer = get_tracer()

    def __enter__(self):
        if self._tracer is not None:
            self._before = self._tracer.current_layer()
            self._tracer._local.layer = self.layer
        return self

    def __exit__(self, *exc):
        if self._tracer is not None:
            self._tracer._local.layer = self._before
        return False


def wrap_region(region: str, fn: Callable, *, layer: Optional[int] = None,
                out_fn: Optional[Callable] = None) -> Callable:
    """``fn`` itself when tracing is off or the allow list leaves ``region`` out; otherwise ``fn`` with the return value
    of every outermost call recorded (a region that calls itself is recorded once, at the outside). ``out_fn`` picks
    what to digest out of the return value.  (isoexec/debug/trace.py:357-400 has the same contract.)"""
    tracer = get_tracer()
    if tracer is None or not tracer.wants(region) or getattr(fn, "_ix_traced_region", None) == region:
        return fn

    def traced(*args, **kwargs):
        depth = tracer._depth.get(region, 0)
        tracer._depth[region] = depth + 1
        try:
            out = fn(*args, **kwargs)
        finally:
            tracer._depth[region] = depth
        if depth == 0:
            tracer.record(region, out if out_fn is None else out_fn(out), layer=layer)
        return out

    traced.__wrapped__ = fn
    traced._ix_traced_region = region
    return traced
