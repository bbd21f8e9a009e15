"""Region logs on the hybrid model: the trainer's pass over the prompts and the engine's prefill agree at every
recorded region; a changed weight or a changed token is found at the first region it reaches, with the rows it
touches; nothing is read back while a decode step is being captured into a graph."""

import pytest
import torch

from isoexec_amd.debug.regions import RegionLog, compare, render, wrap_region
from test_gpu_hybrid import DEV, small_config

pytestmark = pytest.mark.gpu


def setup(seed=0, prompt_lens=(37, 5, 64, 1, 90)):
    from isoexec_amd.runtimes.hybrid import HybridWeights, RolloutEngine, TrainerModel

    cfg = small_config()
    w = HybridWeights.make(cfg, seed=seed, device=DEV)
    g = torch.Generator(device=DEV)
    g.manual_seed(seed + 1)
    lens = list(prompt_lens)
    prompts = torch.randint(0, cfg.vocab, (sum(lens),), device=DEV, generator=g)
    return cfg, w, prompts, lens, TrainerModel, RolloutEngine, HybridWeights


def trainer_log(cfg, w, prompts, lens, TrainerModel, **kw):
    trainer = TrainerModel(cfg, w)
    trainer.blocks.region_log = RegionLog("trainer", **kw)
    trainer.hidden_states(prompts, lens)
    return trainer.blocks.region_log


def engine_log(cfg, w, prompts, lens, RolloutEngine, **kw):
    engine = RolloutEngine(cfg, w, max_num_seqs=len(lens) + 2, max_len=max(lens) + 8)
    engine.blocks.region_log = RegionLog("engine", **kw)
    engine.prefill([11 + 3 * i for i in range(len(lens))], prompts, lens)
    return engine, engine.blocks.region_log


def test_trainer_pass_and_engine_prefill_agree_region_by_region():
    cfg, w, prompts, lens, TrainerModel, RolloutEngine, _ = setup()
    a = trainer_log(cfg, w, prompts, lens, TrainerModel, ladder=True, segment_rows=16)
    _, b = engine_log(cfg, w, prompts, lens, RolloutEngine, ladder=True, segment_rows=16)
    report = compare(a, b)
    # per layer: the mixer's output, the FFN's output, the normed stream and the residual
    assert report["matched"] == cfg.layers * 4 and report["mismatches"] == [] and report["unpaired"] == []
    regions = [r["region"] for r in a.records if r["out"] == "0" and r["layer"] == 0]
    assert regions == ["gdn.core", "moe.combine", "norms.rms"]
    assert {r["region"] for r in a.records if r["layer"] == 1} == {"attention.varlen", "moe.combine", "norms.rms"}
    assert all(set(r["ladder"]) == {"k6", "k4", "k2", "k0"} and len(r["segments"]) == -(-sum(lens) // 16) for r in a.records)
    assert "no divergence" in render(report)


def test_a_changed_weight_is_found_at_the_first_region_it_reaches():
    cfg, w, prompts, lens, TrainerModel, RolloutEngine, HybridWeights = setup()
    other = HybridWeights.make(cfg, seed=0, device=DEV)
    other.layers[2]["w2"].view(torch.int16)[:, 0, :] ^= 0x40       # top mantissa bit of one output row of every expert
    a = trainer_log(cfg, w, prompts, lens, TrainerModel, ladder=True, segment_rows=16)
    _, b = engine_log(cfg, other, prompts, lens, RolloutEngine, ladder=True, segment_rows=16)
    report = compare(a, b)
    first = report["first"]
    assert (first["region"], first["layer"], first["kind"]) == ("moe.combine", 2, "value")
    assert report["matched"] == 2 * 4 + 1                            # layers 0 and 1 whole, and layer 2's mixer
    assert all(m["layer"] >= 2 for m in report["mismatches"])
    assert isinstance(first["magnitude"], str) and "1 of" not in (first["segments"] or "")   # one column, every row
    assert "first divergence: moe.combine @ layer 2" in render(report)


def test_a_changed_token_is_found_with_its_rows():
    cfg, w, prompts, lens, TrainerModel, RolloutEngine, _ = setup()
    changed = prompts.clone()
    position = lens[0] + lens[1] + 40                                 # inside the third sequence (rows 42..105)
    changed[position] = (changed[position] + 1) % cfg.vocab
    a = trainer_log(cfg, w, prompts, lens, TrainerModel, segment_rows=8)
    _, b = engine_log(cfg, w, changed, lens, RolloutEngine, segment_rows=8)
    report = compare(a, b)
    first = report["first"]
    assert (first["region"], first["layer"]) == ("gdn.core", 0)
    # causal and per sequence: rows from the changed token to the end of ITS sequence, nothing before, nothing after
    end = lens[0] + lens[1] + lens[2]
    sa, sb = a.records[0]["segments"], b.records[0]["segments"]
    differing = [i for i, (x, y) in enumerate(zip(sa, sb)) if x != y]
    assert differing[0] == position // 8 and differing[-1] <= (end - 1) // 8
    assert f"first: segment {position // 8}, rows {position // 8 * 8}.." in first["segments"]


def test_nothing_is_read_back_under_graph_capture():
    cfg, w, prompts, lens, TrainerModel, RolloutEngine, _ = setup(prompt_lens=(9, 4))
    engine, log = engine_log(cfg, w, prompts, lens, RolloutEngine)
    before = len(log.records)
    slots = [11, 14]
    tokens = torch.tensor([3, 5], device=DEV)
    engine.decode(slots, tokens)                                       # eager: recorded
    eager = len(log.records) - before
    assert eager == cfg.layers * 4
    graph = engine.capture_decode(slots)
    assert log.capture_skipped > 0
    count = len(log.records)
    graph.step(tokens)
    assert len(log.records) == count                                   # a replay runs no host code: nothing is recorded


def test_wrap_region_records_the_return_value():
    log = RegionLog("trainer")
    double = wrap_region(log, "mm", lambda x: (x * 2, {"aux": x + 1}), layer=3)
    x = torch.arange(6, dtype=torch.float32, device=DEV).reshape(2, 3)
    out = double(x)
    assert torch.equal(out[0], x * 2)
    assert [(r["out"], r["layer"], r["shape"]) for r in log.records] == [("0", 3, [2, 3]), ("1.aux", 3, [2, 3])]
    from isoexec_amd.debug import thash

    assert log.records[0]["digest"] == f"{thash.tensor_digest(x * 2):016x}"


def test_file_traces_of_both_runtimes_compare_offline(tmp_path):
    """The same comparison through files: each runtime writes its trace directory, the offline tool reads both."""
    from isoexec_amd.debug import compare as offline
    from isoexec_amd.debug.trace import Tracer

    cfg, w, prompts, lens, TrainerModel, RolloutEngine, HybridWeights = setup()
    other = HybridWeights.make(cfg, seed=0, device=DEV)
    other.layers[2]["w2"].view(torch.int16)[:, 0, :] ^= 0x40

    def trace_trainer(name):
        tracer = Tracer(str(tmp_path / name), side="trainer", ladder=True, segment_rows=16, ring=7)
        trainer = TrainerModel(cfg, w)
        trainer.blocks.region_log = tracer
        tracer.set_step(0)
        trainer.hidden_states(prompts, lens)
        tracer.flush()
        return tracer

    def trace_engine(name, weights):
        tracer = Tracer(str(tmp_path / name), side="engine", ladder=True, segment_rows=16)
        engine = RolloutEngine(cfg, weights, max_num_seqs=len(lens) + 2, max_len=max(lens) + 8)
        engine.blocks.region_log = tracer
        tracer.set_step(0)
        engine.prefill([11 + 3 * i for i in range(len(lens))], prompts, lens)
        tracer.flush()
        return tracer

    a, b, c = trace_trainer("trainer"), trace_engine("engine", w), trace_engine("engine_changed", other)
    assert a.written == cfg.layers * 4 and a.manifest()["digest_backend"]
    assert offline.main([a.dir, b.dir]) == 0
    report = offline.compare_dirs(a.dir, c.dir)
    first = report["first_divergence"]
    assert report["status"] == "divergent" and (first["region"], first["layer"], first["kind"]) == ("moe.combine", 2, "value")
    assert report["regions"]["gdn.core"]["aligned_on"] == ["step"] and not first["inherited"]
    assert all(d["layer"] >= 2 for d in report["divergences"]) and offline.main([a.dir, c.dir]) == 2


def test_the_environment_switch_reaches_the_runtime(tmp_path, monkeypatch):
    from isoexec_amd.debug import trace

    cfg, w, prompts, lens, TrainerModel, _, _ = setup(prompt_lens=(9, 4))
    trace._forget_for_tests()
    monkeypatch.delenv(trace.ENV_TRACE, raising=False)
    assert TrainerModel(cfg, w).blocks.region_log is None
    trace._forget_for_tests()
    monkeypatch.setenv(trace.ENV_TRACE, str(tmp_path / "t"))
    monkeypatch.setenv(trace.ENV_SIDE, "trainer")
    monkeypatch.setenv(trace.ENV_REGIONS, "gdn.core,attention.varlen")
    try:
        trainer = TrainerModel(cfg, w)
        assert trainer.blocks.region_log is trace.get_tracer()
        trainer.hidden_states(prompts, lens)
        trace.flush()
        from isoexec_amd.debug.compare import load_dir

        records = load_dir(str(tmp_path / "t"))
        assert len(records) == cfg.layers and {r["region"] for r in records} == {"gdn.core", "attention.varlen"}
        assert all(r["side"] == "trainer" and r["layer_src"] == "caller" for r in records)
    finally:
        trace._forget_for_tests()


def test_installed_doors_record_what_the_runtime_calls_and_change_nothing(tmp_path, monkeypatch):
    from isoexec_amd.debug import install, trace
    from isoexec_amd.debug.compare import load_dir

    cfg, w, prompts, lens, TrainerModel, _, _ = setup(prompt_lens=(33, 7))
    trace._forget_for_tests()
    monkeypatch.delenv(trace.ENV_TRACE, raising=False)
    plain = TrainerModel(cfg, w).hidden_states(prompts, lens)
    trace._forget_for_tests()
    monkeypatch.setenv(trace.ENV_TRACE, str(tmp_path / "doors"))
    monkeypatch.setenv(trace.ENV_SIDE, "trainer")
    try:
        assert install.install_debug_hooks() > 0
        traced = TrainerModel(cfg, w).hidden_states(prompts, lens)
        trace.flush()
        assert torch.equal(traced, plain)
        records = load_dir(str(tmp_path / "doors"))
        by_region = {}
        for r in records:
            by_region.setdefault(r["region"], []).append(r)
        # the doors the pass goes through, once per layer of their kind (no layer: the door does not know it) ...
        gdn_layers = sum(not cfg.is_attention(i) for i in range(cfg.layers))
        assert len([r for r in by_region["gdn.conv"] if r["layer"] is None]) == gdn_layers
        assert len([r for r in by_region["attention.varlen"] if r["layer"] is None]) == cfg.layers - gdn_layers
        assert len([r for r in by_region["moe.router"] if r["out"] == "0"]) == cfg.layers
        assert {"gdn.core", "gdn.l2norm", "gdn.gating", "norms.gated_out", "norms.rms", "rope.rope", "moe.experts"} <= set(by_region)
        assert "mm" not in by_region
        # ... beside the runtime's own per-layer records
        assert len([r for r in by_region["gdn.core"] if r["layer"] is not None]) == gdn_layers
    finally:
        install.uninstall_debug_hooks()
        trace._forget_for_tests()
