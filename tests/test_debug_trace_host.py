"""The file trace and the offline comparison of two trace directories, on the host (no GPU): the tracer's plumbing
with a stand-in for the device digest, and the comparator on handmade directories. What the comparator promises
follows the reference's tool (isoexec/debug/compare.py:5 exit codes; :104-120 alignment on step, call, position;
:258-270 disjoint sampling is inconclusive; :457-468 causal order of divergences)."""

import json
import os
import subprocess
import sys

import pytest

from isoexec_amd.debug import compare as C
from isoexec_amd.debug import trace as T

PKG_PARENT = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "skyrl-isoexec_amd")


class HostLog:
    """Stands in for RegionLog: 'digests' a Python value by its repr, numbers calls the same way."""

    def __init__(self):
        self.records, self.capture_skipped, self._calls = [], 0, {}

    def next_call(self, region, layer=None):
        return self._calls.get((region, layer), 0) + 1

    def skip(self, region, layer=None):
        self._calls[(region, layer)] = self.next_call(region, layer)

    def record(self, region, out, *, layer=None, case=None):
        call = self.next_call(region, layer)
        self._calls[(region, layer)] = call
        self.records.append({"v": C.FORMAT_VERSION, "region": region, "case": case, "side": "x", "layer": layer,
                             "call": call, "out": "0", "shape": [1], "dtype": "host", "digest": repr(out)})


def make_tracer(tmp_path, name="t", **kw):
    kw.setdefault("digest_log", HostLog())
    return T.Tracer(str(tmp_path / name), **kw)


# ---- the tracer ------------------------------------------------------------------------------------------------------

def test_file_names_manifest_and_ring(tmp_path):
    tr = make_tracer(tmp_path, side="trainer", ring=3, rank=2)
    assert os.path.basename(tr.path).startswith("trainer-r2-") and tr.path.endswith(f"-{os.getpid()}.jsonl")
    assert os.path.basename(tr.manifest_path).startswith("manifest-trainer-r2-")
    assert json.load(open(tr.manifest_path))["records"] == 0          # the manifest exists before any record
    tr.record("gdn.core", 1.0, layer=0)
    tr.record("gdn.core", 2.0, layer=1)
    assert not os.path.exists(tr.path)                                 # two records: still in memory
    tr.record("moe.combine", 3.0, layer=1)
    got = [json.loads(ln) for ln in open(tr.path)]                     # the third filled the ring
    assert [r["seq"] for r in got] == [1, 2, 3] and got[2]["region"] == "moe.combine"
    assert all(r["rank"] == 2 and r["pid"] == os.getpid() and r["layer_src"] == "caller" and r["ts"] > 0 for r in got)
    tr.record("gdn.core", 4.0, layer=0)
    tr.flush()
    assert len(open(tr.path).read().splitlines()) == 4
    man = json.load(open(tr.manifest_path))
    assert man["records"] == 4 and man["side"] == "trainer" and man["sample"] == 1 and man["step_signal"] is False
    assert C.load_dir(tr.dir)[3]["call"] == 2 and C.load_manifests(tr.dir)[0]["file"] == os.path.basename(tr.path)


def test_sampling_by_call_then_by_step(tmp_path):
    tr = make_tracer(tmp_path, sample=3)
    for i in range(7):
        tr.record("gdn.core", float(i), layer=0)
    tr.flush()
    assert [r["call"] for r in C.load_dir(tr.dir)] == [1, 4, 7]       # every third call, numbers of the others kept
    tr2 = make_tracer(tmp_path, "t2", sample=2)
    for step in range(5):
        tr2.set_step(step)
        tr2.record("gdn.core", float(step), layer=0)
        tr2.record("gdn.core", float(step) + 0.5, layer=0)
    tr2.flush()
    recs = C.load_dir(tr2.dir)
    assert [r["step"] for r in recs] == [0, 0, 2, 2, 4, 4] and [r["call"] for r in recs] == [1, 2, 5, 6, 9, 10]
    man = C.load_manifests(tr2.dir)[0]
    assert man["step_signal"] and man["steps_seen"] == [0, 1, 2, 3, 4] and man["steps_recorded"] == [0, 2, 4]


def test_allow_list_and_high_volume_default(tmp_path):
    tr = make_tracer(tmp_path)
    assert tr.wants("gdn.core") and not tr.wants("mm")
    tr.record("mm", 1.0)
    tr.flush()
    assert not os.path.exists(tr.path)
    tr2 = make_tracer(tmp_path, "t2", regions=["mm"])
    assert tr2.wants("mm") and not tr2.wants("gdn.core")


def test_env_switches_wrap_region_and_layer_context(tmp_path, monkeypatch):
    T._forget_for_tests()
    monkeypatch.delenv(T.ENV_TRACE, raising=False)
    fn = lambda x: x  # noqa: E731
    assert T.get_tracer() is None and T.wrap_region("gdn.core", fn) is fn          # off: nothing is installed
    T.set_step(3), T.flush()                                                         # and the calls cost nothing

    T._forget_for_tests()
    monkeypatch.setenv(T.ENV_TRACE, str(tmp_path / "env"))
    monkeypatch.setenv(T.ENV_SIDE, "engine")
    monkeypatch.setenv(T.ENV_SAMPLE, "1")
    monkeypatch.setenv(T.ENV_SEGMENTS, "64")
    monkeypatch.setenv(T.ENV_LADDER, "1")
    monkeypatch.setenv(T.ENV_RING, "100")
    monkeypatch.setenv("RANK", "5")
    tr = T.get_tracer()
    try:
        assert tr is T.get_tracer() and (tr.side, tr.rank, tr.segment_rows, tr.ladder, tr.ring) == ("engine", 5, 64, True, 100)
        tr._log = HostLog()

        def outer(n):
            return n if n == 0 else inner(n - 1) + 1

        inner = T.wrap_region("gdn.core", outer)
        assert T.wrap_region("gdn.core", inner) is inner                             # not wrapped twice
        assert T.wrap_region("mm", fn) is fn                                         # not on the allow list: untouched
        outer = inner                                                                # the region now calls itself
        with T.layer_context(7):
            assert inner(3) == 3
        picked = T.wrap_region("moe.router", lambda: ("idx", "prob"), out_fn=lambda out: out[1])
        picked()
        T.set_case("prefill")
        T.wrap_region("moe.combine", fn, layer=2)(1.5)
        T.flush()
        recs = C.load_dir(tr.dir)
        assert [(r["region"], r["layer"], r["layer_src"], r["digest"], r["case"]) for r in recs] == [
            ("gdn.core", 7, "context", "3", None), ("moe.router", None, None, "'prob'", None),
            ("moe.combine", 2, "caller", "1.5", "prefill")]                          # recursion recorded once, outside
    finally:
        T._forget_for_tests()
    monkeypatch.setenv(T.ENV_SAMPLE, "many")
    with pytest.raises(ValueError, match="SKYRL_ISOEXEC_DEBUG_SAMPLE"):
        T.get_tracer()
    T._forget_for_tests()


# ---- the comparator --------------------------------------------------------------------------------------------------

def rec(region, layer, digest, *, call=1, step=None, ts=0.0, out="0", rank=0, shape=(4, 8), **extra):
    return dict({"v": C.FORMAT_VERSION, "region": region, "layer": layer, "out": out, "call": call, "step": step,
                 "rank": rank, "ts": ts, "shape": list(shape), "dtype": "bfloat16", "digest": digest}, **extra)


def write_dir(tmp_path, name, records, side, manifest=None):
    d = tmp_path / name
    d.mkdir()
    with open(d / f"{side}-r0-h-1.jsonl", "w") as fh:
        for i, r in enumerate(records):
            fh.write(json.dumps(dict(r, side=side, seq=i + 1)) + "\n")
    if manifest is not None:
        with open(d / f"manifest-{side}-r0-h-1.json", "w") as fh:
            json.dump(dict({"v": C.FORMAT_VERSION, "side": side, "sample": 1}, **manifest), fh)
    return str(d)


def forward(digests, t0=0.0):
    """Records of one pass over two layers in execution order; `digests` maps (region, layer) -> digest."""
    order = [("gdn.core", 0), ("moe.combine", 0), ("gdn.core", 1), ("moe.combine", 1)]
    return [rec(r, l, digests.get((r, l), f"{r}{l}"), ts=t0 + i) for i, (r, l) in enumerate(order)]


def test_clean_and_divergent_directories(tmp_path, capsys):
    a = write_dir(tmp_path, "a", forward({}), "trainer", {})
    b = write_dir(tmp_path, "b", forward({}), "engine", {})
    assert C.main([a, b]) == 0
    assert "CLEAN: 4 paired region outputs" in capsys.readouterr().out
    # the engine differs from moe.combine@0 on; gdn.core@1 inherits it
    c = write_dir(tmp_path, "c", forward({("moe.combine", 0): "XX", ("gdn.core", 1): "YY"}), "engine", {})
    out_json = str(tmp_path / "rep.json")
    assert C.main([a, c, "--json", out_json]) == 2
    text = capsys.readouterr().out
    assert "FIRST DIVERGENCE (value): moe.combine @ layer 0" in text and "1 later divergences (1 possibly inherited" in text
    rep = json.load(open(out_json))
    assert rep["status"] == "divergent" and rep["first_divergence"]["digests"] == ["moe.combine0", "XX"]
    assert [d["inherited"] for d in rep["divergences"]] == [False, True]
    assert rep["regions"]["gdn.core"] == {"compared": 2, "matched": 1, "mismatched": 1, "absent": 0, "unrecordable": 0,
                                          "aligned_on": ["call"]}
    assert C.main([a, c, "--regions", "gdn.core"]) == 2
    assert "FIRST DIVERGENCE (value): gdn.core @ layer 1" in capsys.readouterr().out


def test_alignment_on_step_leaves_a_hole_instead_of_shifting(tmp_path):
    a = [rec("gdn.core", 0, f"s{s}", call=s + 1, step=s, ts=s) for s in range(4)]
    b = [r for r in a if r["step"] != 1]                                # the engine never recorded step 1
    rep = C.compare_records(a, [dict(r, call=i + 1) for i, r in enumerate(b)])
    assert rep["regions"]["gdn.core"]["aligned_on"] == ["step"] and rep["regions"]["gdn.core"]["matched"] == 3
    assert [(d["kind"], d["step"]) for d in rep["divergences"]] == [("absent", 1)] and rep["status"] == "divergent"
    # without the step signal the call numbers pair; without either, position does (and shifts)
    rep = C.compare_records([dict(r, step=None) for r in a], [dict(r, step=None) for r in a])
    assert rep["regions"]["gdn.core"]["aligned_on"] == ["call"] and rep["status"] == "clean"
    rep = C.compare_records([dict(r, step=None, call=1) for r in a], [dict(r, step=None, call=1) for r in b])
    assert rep["regions"]["gdn.core"]["aligned_on"] == ["position"]


def test_layout_ladder_segments_and_layer_folding(tmp_path):
    la = {"k7": "a7", "k4": "a4", "k0": "a0"}
    a = [rec("gdn.core", None, "aa", call=c, ladder=la, segments=["s0", "s1", "s2", "s3"], seg_rows=16) for c in (1, 2, 3, 4)]
    b = [dict(r) for r in a]
    b[3] = dict(b[3], digest="ab", ladder=dict(la, k7="b7"), segments=["s0", "s1", "XX", "s3"])
    b[1] = dict(b[1], shape=[1, 4, 8])
    rep = C.compare_records(a, b, layers=2)                             # calls 1,3 -> layer 0; calls 2,4 -> layer 1
    kinds = {(d["layer"], d["call"]): d for d in rep["divergences"]}
    assert set(kinds) == {(1, 2), (1, 4)} and kinds[(1, 2)]["kind"] == "layout"
    value = kinds[(1, 4)]
    assert value["agree_k"] == 4 and value["magnitude"].startswith("between ~2^-7 and 2^-4")
    assert value["segments"] == "1 of 4 row segments differ (first: segment 2, rows 32..47)"


def test_disjoint_sampling_and_nothing_paired_are_inconclusive(tmp_path, capsys):
    a = write_dir(tmp_path, "a", [rec("gdn.core", 0, "x", step=0), rec("gdn.core", 0, "y", call=2, step=2)], "trainer",
                  {"sample": 2, "step_signal": True})
    b = write_dir(tmp_path, "b", [rec("gdn.core", 0, "x", call=1), rec("gdn.core", 0, "z", call=3)], "engine", {"sample": 2})
    assert C.main([a, b]) == 3
    assert "INCONCLUSIVE: side A records every Nth step and side B every Nth call" in capsys.readouterr().out
    c = write_dir(tmp_path, "c", [rec("gdn.core", 0, "x", step=1), rec("gdn.core", 0, "y", call=2, step=3)], "engine",
                  {"sample": 2, "step_signal": True})
    assert C.main([a, c]) == 3 and "disjoint sets of steps" in capsys.readouterr().out
    d = write_dir(tmp_path, "d", [rec("attention.varlen", 3, "x")], "engine", {})
    e = write_dir(tmp_path, "e", [rec("gdn.core", 0, "x")], "trainer", {})
    assert C.main([e, d]) == 3 and "no record of one side has a counterpart" in capsys.readouterr().out


def test_bad_input_exits_1_and_a_torn_last_line_is_tolerated(tmp_path, capsys):
    good = write_dir(tmp_path, "good", forward({}), "trainer", {})
    assert C.main([good, str(tmp_path / "missing")]) == 1
    assert "no *.jsonl trace files" in capsys.readouterr().err
    old = write_dir(tmp_path, "old", [dict(r, v=2) for r in forward({})], "engine")
    assert C.main([good, old]) == 1 and "record format 2" in capsys.readouterr().err
    torn = write_dir(tmp_path, "torn", forward({}), "engine")
    with open(os.path.join(torn, "engine-r0-h-1.jsonl"), "a") as fh:
        fh.write('{"v": 3, "region": "gdn.co')                          # the process died inside a write
    assert C.main([good, torn]) == 0
    capsys.readouterr()
    with open(os.path.join(torn, "engine-r0-h-1.jsonl"), "a") as fh:
        fh.write('\n' + json.dumps(rec("gdn.core", 0, "late", call=9)) + "\n")
    assert C.main([good, torn]) == 1 and "not JSON" in capsys.readouterr().err   # torn in the middle is damage


def test_undigested_outputs_are_counted_not_compared():
    a = [rec("gdn.core", 0, "aa"), {k: v for k, v in rec("moe.combine", 0, "", unrecordable="ValueError: host tensor").items()
                                    if k != "digest"}]
    rep = C.compare_records(a, [dict(r) for r in a])
    assert rep["status"] == "clean" and rep["regions"]["moe.combine"]["unrecordable"] == 1 and len(rep["unrecordable"]) == 1
    assert "carry no digest" in C.render_text(rep)


def test_the_tool_runs_on_the_standard_library_alone(tmp_path):
    a = write_dir(tmp_path, "a", forward({}), "trainer", {})
    b = write_dir(tmp_path, "b", forward({("gdn.core", 1): "ZZ"}), "engine", {})
    by_path = subprocess.run([sys.executable, C.__file__, a, b], capture_output=True, text=True)
    assert by_path.returncode == 2 and "FIRST DIVERGENCE (value): gdn.core @ layer 1" in by_path.stdout
    probe = ("import sys, runpy\nsys.argv = ['isoexec_amd.debug', %r, %r]\n"
             "try:\n    runpy.run_module('isoexec_amd.debug', run_name='__main__')\n"
             "except SystemExit as e:\n    code = e.code\n"
             "assert 'torch' not in sys.modules and 'numpy' not in sys.modules, sorted(sys.modules)\nsys.exit(code)\n") % (a, a)
    as_module = subprocess.run([sys.executable, "-c", probe], capture_output=True, text=True,
                               env=dict(os.environ, PYTHONPATH=PKG_PARENT))
    assert as_module.returncode == 0, as_module.stderr
    assert "CLEAN" in as_module.stdout


# ---- the installer ---------------------------------------------------------------------------------------------------

def test_every_registry_region_is_accounted_for():
    from isoexec_amd.debug import install

    cov = install.coverage()
    assert not [r for r, e in cov.items() if e["status"] == "unknown"]
    assert cov["gdn.core"]["status"] == "hooked" and "ops.gdn.gdn_ops:gdn_recurrent_kernel" in cov["gdn.core"]["doors"]
    assert cov["gdn.state"]["status"] == "partial" and cov["moe.weights"]["status"] == "not_hooked" and cov["moe.weights"]["note"]
    assert install.coverage(["made.up"])["made.up"]["status"] == "unknown"
    for region, module, attr, _ in install.DOORS:                      # every door of the table exists
        assert install._resolve(module, attr) is not None, (region, module, attr)


def test_install_wraps_the_definition_and_every_imported_binding(tmp_path, monkeypatch):
    from isoexec_amd.debug import install
    from isoexec_amd.ops.norms import fused_outnorm
    from isoexec_amd.runtimes import hybrid

    T._forget_for_tests()
    monkeypatch.delenv(T.ENV_TRACE, raising=False)
    assert install.install_debug_hooks() == 0                          # tracing off: nothing is touched
    original = fused_outnorm.fused_rms_norm_gamma
    assert hybrid.fused_rms_norm_gamma is original

    T._forget_for_tests()
    monkeypatch.setenv(T.ENV_TRACE, str(tmp_path / "t"))
    monkeypatch.setenv(T.ENV_SIDE, "trainer")
    try:
        T.get_tracer()._log = HostLog()
        changed = install.install_debug_hooks()
        wrapped = fused_outnorm.fused_rms_norm_gamma
        assert changed > len(install.DOORS) // 2 and wrapped is not original and wrapped.__wrapped__ is original
        assert hybrid.fused_rms_norm_gamma is wrapped                  # the binding `from ... import` left behind
        assert fused_outnorm.ZeroCenteredRMSNorm.forward._ix_traced_region == "norms.rms"
        from isoexec_amd.ops.mm import mm_hip

        assert not hasattr(mm_hip.linear_nt, "_ix_traced_region")      # `mm` is off unless the allow list names it
        assert install.install_debug_hooks() == 0                      # a second call finds everything wrapped
        monkeypatch.setattr(fused_outnorm, "fused_rms_norm_gamma", lambda x, w, eps, **kw: ("normed", x))
        T.wrap_region("norms.rms", fused_outnorm.fused_rms_norm_gamma)("x", None, 1e-6)
        T.flush()
        assert [r["region"] for r in C.load_dir(str(tmp_path / "t"))] == ["norms.rms"]
    finally:
        monkeypatch.undo()
        assert install.uninstall_debug_hooks() > 0
        T._forget_for_tests()
    assert fused_outnorm.fused_rms_norm_gamma is original and hybrid.fused_rms_norm_gamma is original
    assert not hasattr(fused_outnorm.ZeroCenteredRMSNorm.forward, "_ix_traced_region")
