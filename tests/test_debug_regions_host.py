"""The comparison half of the region log on handmade records (no GPU): pairing, the ladder verdict, the slab note,
the text report and the JSONL round trip. The verdict wording follows what the reference's comparator promises
(isoexec/debug/compare.py:123-181): a bound is a maximum over elements, and a saturated ladder is not called large."""

from isoexec_amd.debug import regions as R


def rec(region, layer, digest, *, out="0", call=1, shape=(4, 8), ladder=None, segments=None, seg_rows=0, side="a"):
    r = {"v": R.FORMAT_VERSION, "region": region, "layer": layer, "out": out, "call": call, "side": side,
         "shape": list(shape), "dtype": "bfloat16", "digest": digest}
    if ladder is not None:
        r["ladder"] = ladder
    if segments is not None:
        r["segments"], r["seg_rows"], r["seg_axis"] = segments, seg_rows, 0
    return r


def log_of(side, records):
    log = R.RegionLog(side)
    for i, r in enumerate(records):
        r = dict(r, side=side, seq=i + 1)
        log.records.append(r)
    return log


def test_equal_logs_have_no_divergence():
    records = [rec("gdn.core", 0, "aa"), rec("moe.combine", 0, "bb"), rec("gdn.core", 1, "cc")]
    report = R.compare(log_of("trainer", records), log_of("engine", records))
    assert report["matched"] == 3 and report["mismatches"] == [] and report["first"] is None
    assert "no divergence" in R.render(report)


def test_first_divergence_is_the_earliest_in_execution_order():
    a = [rec("gdn.core", 0, "aa"), rec("moe.combine", 0, "bb"), rec("gdn.core", 1, "cc"), rec("moe.combine", 1, "dd")]
    b = [rec("gdn.core", 0, "aa"), rec("moe.combine", 0, "b0"), rec("gdn.core", 1, "c0"), rec("moe.combine", 1, "dd")]
    report = R.compare(log_of("trainer", a), log_of("engine", b))
    assert report["matched"] == 2 and len(report["mismatches"]) == 2
    first = report["first"]
    assert (first["region"], first["layer"], first["kind"]) == ("moe.combine", 0, "value")
    assert first["digests"] == ("bb", "b0") and first["agree_k"] is None and first["magnitude"].startswith("unknown")
    text = R.render(report)
    assert "first divergence: moe.combine @ layer 0" in text and "2 differ" in text


def test_records_pair_by_occurrence_and_output_path():
    a = [rec("norms.rms", 0, "x0", out="0"), rec("norms.rms", 0, "h0", out="1"), rec("norms.rms", 0, "x1", call=2)]
    b = [rec("norms.rms", 0, "x0", out="0"), rec("norms.rms", 0, "hZ", out="1"), rec("norms.rms", 0, "x1", call=2),
         rec("norms.rms", 0, "extra", call=3)]
    report = R.compare(log_of("a", a), log_of("b", b))
    assert report["matched"] == 2 and [m["out"] for m in report["mismatches"]] == ["1"]
    assert report["unpaired"] == [("norms.rms", 0, "0", 3)]


def test_layout_difference_is_named_as_such():
    report = R.compare(log_of("a", [rec("gdn.core", 0, "aa", shape=(1, 4, 8))]), log_of("b", [rec("gdn.core", 0, "ab", shape=(4, 8))]))
    assert report["first"]["kind"] == "layout" and "not comparable" in report["first"]["magnitude"]


def test_ladder_verdicts():
    full = {"k6": "1", "k4": "2", "k2": "3", "k0": "4"}
    # agree from k4 down, differ at k6: the difference is below 2^-4 and (probably) above 2^-6
    agree, text = R.ladder_verdict({"ladder": full}, {"ladder": dict(full, k6="x")})
    assert agree == 4 and "2^-6" in text and "2^-4" in text
    # agree at every rung: below the finest rung recorded
    agree, text = R.ladder_verdict({"ladder": full}, {"ladder": dict(full)})
    assert agree == 6 and text.startswith("< 2^-6")
    # differ at every rung: nothing is bounded, and nothing is called large
    agree, text = R.ladder_verdict({"ladder": full}, {"ladder": {k: v + "'" for k, v in full.items()}})
    assert agree is None and "not bounded" in text and "large" not in text
    assert R.ladder_verdict({}, {"ladder": full})[1].startswith("unknown")


def test_segment_notes():
    base = ["s0", "s1", "s2", "s3"]
    a = rec("gdn.core", 0, "aa", segments=base, seg_rows=16)
    assert R.segment_note(a, rec("gdn.core", 0, "ab", segments=["s0", "s1", "XX", "s3"], seg_rows=16)) == \
        "1 of 4 row segments differ (first: segment 2, rows 32..47)"
    assert "whole-tensor" in R.segment_note(a, rec("gdn.core", 0, "ab", segments=["a", "b", "c", "d"], seg_rows=16))
    assert "below segment resolution" in R.segment_note(a, rec("gdn.core", 0, "ab", segments=list(base), seg_rows=16))
    assert R.segment_note(a, rec("gdn.core", 0, "ab")) is None
    assert R.segment_note(a, rec("gdn.core", 0, "ab", segments=["s0"], seg_rows=64)) is None


def test_unrecordable_outputs_are_listed_not_compared():
    broken = {"v": 3, "region": "moe.router", "layer": 0, "out": "0", "call": 1, "unrecordable": "TypeError: nope"}
    report = R.compare(log_of("a", [broken]), log_of("b", [rec("moe.router", 0, "aa")]))
    assert report["matched"] == 0 and report["mismatches"] == [] and len(report["unrecordable"]) == 1


def test_jsonl_round_trip(tmp_path):
    log = log_of("trainer", [rec("gdn.core", 0, "aa", ladder={"k6": "1"}, segments=["s"], seg_rows=8), rec("moe.combine", 0, "bb")])
    path = tmp_path / "trainer.jsonl"
    log.dump(str(path))
    back = R.RegionLog.load(str(path))
    assert back.side == "trainer" and back.records == log.records and back.ladder and back.segment_rows == 8


def test_wrap_region_without_a_log_is_the_function_itself():
    fn = lambda x: x
    assert R.wrap_region(None, "gdn.core", fn) is fn
