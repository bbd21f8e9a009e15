"""End to end: the trainer's full-sequence logprobs equal the rollout's incremental logprobs bit for
bit (importance ratio exactly 1.0), and the two runtimes hold the same contract hash.

The reduced model exercises every layer kind quickly with ragged prompts, a padded pool and a
different batch composition on each side; the last test is the benchmark's configuration at full size.
"""

import numpy as np
import pytest
import torch

from _util import same_bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def small_config():
    from isoexec_amd.runtimes.hybrid import HybridConfig

    return HybridConfig(hidden=256, vocab=8192, layers=4, attention_every=2, gdn_k_heads=2, gdn_v_heads=4, gdn_head_dim=64,
                        q_heads=8, kv_heads=2, head_dim=128, max_positions=512, experts=8, topk=2, expert_inter=64)


def rollout_then_score(cfg, prompt_lens, steps, seed, slots=None):
    from isoexec_amd.runtimes.hybrid import HybridWeights, RolloutEngine, TrainerModel

    w = HybridWeights.make(cfg, seed=seed, device=DEV)
    n = len(prompt_lens)
    g = torch.Generator(device=DEV)
    g.manual_seed(seed + 1)
    prompts = torch.randint(0, cfg.vocab, (sum(prompt_lens),), device=DEV, generator=g)
    slots = slots or [11 + 3 * i for i in range(n)]
    engine = RolloutEngine(cfg, w, max_num_seqs=n + 2, max_len=max(prompt_lens) + steps)
    toks, lps = engine.generate(slots, prompts, prompt_lens, steps, seed=seed)
    # the sequences the trainer sees: prompt + sampled response, packed
    parts, lens, start = [], [], 0
    for i, p in enumerate(prompt_lens):
        parts += [prompts[start : start + p], toks[i]]
        lens.append(p + steps)
        start += p
    packed = torch.cat(parts)
    trainer = TrainerModel(cfg, w)
    return w, engine, trainer, packed, lens, toks, lps


def test_reduced_model_ratio_is_exactly_one():
    cfg = small_config()
    prompt_lens, steps = [37, 5, 64, 1, 90], 40
    w, engine, trainer, packed, lens, toks, lps = rollout_then_score(cfg, prompt_lens, steps, seed=0)
    scored = trainer.response_logprobs(packed, lens, prompt_lens)
    for i in range(len(lens)):
        assert same_bits(scored[i], lps[i]), f"sequence {i}"
        ratio = torch.exp(scored[i] - lps[i])
        assert bool((ratio == 1.0).all())
    assert bool(torch.isfinite(lps).all()) and float(lps.max()) <= 0.0
    # The sampled tokens are not degenerate (the sampler explores) and the model is not uniform.
    assert toks.unique().numel() > steps and float(lps.std()) > 0.1

    # The trainer scoring the sequences one by one, or in another order, gives the same bits.
    alone = trainer.response_logprobs(packed[: lens[0]], lens[:1], prompt_lens[:1])
    assert same_bits(alone[0], scored[0])
    order = [3, 0, 4]
    offs = np.concatenate([[0], np.cumsum(lens)])
    shuffled = torch.cat([packed[offs[i] : offs[i + 1]] for i in order])
    again = trainer.response_logprobs(shuffled, [lens[i] for i in order], [prompt_lens[i] for i in order])
    for j, i in enumerate(order):
        assert same_bits(again[j], scored[i])


def test_boundary_kernel_ratio_is_exactly_one_too():
    """The cpr composition (fp32 chain at chunk boundaries, bf16 snapshot as the running state): the engine's
    prefill + decode out of CprGDN state and the trainer's boundary-form forward are the same function, so the
    ratio is exactly one -- and it is a different function from the recurrent composition."""
    import dataclasses

    base = small_config()
    cfg = dataclasses.replace(base, gdn_kernel="cpr", gdn_chunk=16)
    prompt_lens, steps = [37, 5, 64, 1, 16], 40   # prompts ending inside, before and exactly on chunk boundaries
    w, engine, trainer, packed, lens, toks, lps = rollout_then_score(cfg, prompt_lens, steps, seed=0)
    scored = trainer.response_logprobs(packed, lens, prompt_lens)
    for i in range(len(lens)):
        assert same_bits(scored[i], lps[i]), f"sequence {i}"
    # the graph-replayed decode gives the same tokens and logprobs
    engine2 = type(engine)(cfg, w, max_num_seqs=len(lens) + 2, max_len=max(prompt_lens) + steps)
    g = torch.Generator(device=DEV)
    g.manual_seed(1)
    prompts = torch.randint(0, cfg.vocab, (sum(prompt_lens),), device=DEV, generator=g)
    toks2, lps2 = engine2.generate([11 + 3 * i for i in range(len(lens))], prompts, prompt_lens, steps, seed=0, use_graph=True)
    assert torch.equal(toks2, toks) and same_bits(lps2, lps)
    # not the recurrent function: scoring the same sequences with the recurrent kernel moves some bits
    from isoexec_amd.runtimes.hybrid import TrainerModel

    other = TrainerModel(base, w).response_logprobs(packed, lens, prompt_lens)
    assert any(not same_bits(a, b) for a, b in zip(other, scored))
    assert max(float((a - b).abs().max()) for a, b in zip(other, scored)) < 0.25


def test_rollout_bits_do_not_depend_on_batch_or_chunked_prefill(monkeypatch):
    """The same request decoded alone, inside a batch, and after a prefill cut into chunks."""
    from isoexec_amd.runtimes.hybrid import HybridWeights, RolloutEngine

    cfg = small_config()
    w = HybridWeights.make(cfg, seed=3, device=DEV)
    g = torch.Generator(device=DEV)
    g.manual_seed(4)
    lens = [50, 23, 77]
    prompts = torch.randint(0, cfg.vocab, (sum(lens),), device=DEV, generator=g)
    follow = torch.randint(0, cfg.vocab, (3, 12), device=DEV, generator=g)

    def run(engine, slots, idx):
        offs = np.concatenate([[0], np.cumsum(lens)])
        packed = torch.cat([prompts[offs[i] : offs[i + 1]] for i in idx])
        xs = [engine.prefill(slots, packed, [lens[i] for i in idx])]
        for s in range(12):
            xs.append(engine.decode(slots, follow[idx, s]))
        return torch.stack(xs, dim=1)  # [n, 13, H]

    batch = run(RolloutEngine(cfg, w, 4, 128), [5, 6, 7], [0, 1, 2])
    alone = run(RolloutEngine(cfg, w, 4, 128), [9], [1])
    assert same_bits(alone[0], batch[1])

    # chunked prefill of request 2: 77 tokens as 30 + 1 + 46, other requests decoding in between
    monkeypatch.setenv("SKYRL_ISOEXEC_GDN_CHUNKED_PREFILL", "1")
    eng = RolloutEngine(cfg, w, 4, 128)
    p2 = prompts[lens[0] + lens[1] :]
    # A chunk continues a sequence: its positions and key/value rows follow the context so far.
    x = None
    done = 0
    for n in (30, 1, 46):
        x = chunk_prefill(eng, 21, p2[done : done + n], done)
        done += n
    xs = [x]
    for s in range(12):
        xs.append(eng.decode([21], follow[2:3, s]))
    assert same_bits(torch.stack(xs, dim=1)[0], batch[2])


def test_graph_replayed_decode_equals_eager_decode():
    """The decode step recorded as a HIP graph and replayed 38 times, with the sampler's eager work
    between replays, against the same rollout run eagerly: same tokens, same logprobs, same state."""
    from isoexec_amd.runtimes.hybrid import HybridWeights, RolloutEngine

    cfg = small_config()
    w = HybridWeights.make(cfg, seed=5, device=DEV)
    g = torch.Generator(device=DEV)
    g.manual_seed(6)
    lens = [33, 8, 70, 21]
    prompts = torch.randint(0, cfg.vocab, (sum(lens),), device=DEV, generator=g)
    slots = [4, 9, 2, 30]
    runs = []
    for use_graph in (False, True):
        eng = RolloutEngine(cfg, w, max_num_seqs=6, max_len=128)
        toks, lps = eng.generate(slots, prompts, lens, 40, seed=11, use_graph=use_graph)
        states = [torch.stack([layer.ssm_state[layer.require_row(s)] for s in slots]) for layer in eng.gdn.values()]
        caches = [kv.k[[eng.kv_rows[s] for s in slots]].clone() for kv in eng.kv.values()]
        runs.append((toks, lps, states, caches, dict(eng.context)))
    (t0, l0, s0, c0, x0), (t1, l1, s1, c1, x1) = runs
    assert torch.equal(t0, t1) and same_bits(l0, l1) and x0 == x1
    assert all(same_bits(a, b) for a, b in zip(s0, s1)) and all(same_bits(a, b) for a, b in zip(c0, c1))


def chunk_prefill(engine, slot, tokens, context):
    """One chunk of a chunked prefill through the engine's own blocks (the engine's ``prefill`` starts
    a request; a continuation chunk differs only in its positions and where its keys land)."""
    from isoexec_amd.ops.attention.varlen_attn import varlen_attention

    b, c = engine.blocks, engine.cfg
    n = tokens.numel()
    dev = tokens.device
    row = engine._kv_row(slot)
    positions = torch.arange(context, context + n, dtype=torch.int32, device=dev)
    cu = torch.tensor([0, n], dtype=torch.int32, device=dev)
    kv_start = torch.tensor([row * engine.max_len], dtype=torch.int64, device=dev)
    pos0 = torch.tensor([context], dtype=torch.int32, device=dev)
    slots_t = torch.tensor([slot], device=dev)

    def mixer(i, x):
        if c.is_attention(i):
            q, k, v = b.attn_qkv(i, x, positions)
            engine.kv[i].write(positions.long() + row * engine.max_len, k, v)
            kf, vf = engine.kv[i].flat()
            return b.attn_out(i, varlen_attention(q, kf, vf, cu, n, kv_start=kv_start, q_pos0=pos0))
        qkv, z, bb, a = b.gdn_in(i, x)
        o = engine.gdn[i].prefill(slots_t, [slot], qkv, a, bb, [0, n], has_initial_state=[context > 0])
        return b.gdn_out(i, o, z)

    x = b.run_layers(b.embed(tokens), mixer)
    engine.context[slot] = context + n
    return x[-1:]


def test_both_runtimes_hold_the_same_contract(monkeypatch):
    """Each runtime builds its contract from the model declaration; the hashes must agree, a
    one-sided change must refuse, and what each runtime installs must match what the contract names."""
    from isoexec_amd.core import enforce, fingerprint, process_contract
    from isoexec_amd.core.arch import detect_arch

    assert detect_arch() == "gfx950"

    def build_side():
        process_contract._reset_for_tests()
        c = process_contract.get_process_contract("Qwen/Qwen3.5-35B-A3B")
        return c, process_contract.contract_hash(), process_contract.cached_contract_view()

    trainer_c, trainer_hash, _ = build_side()
    engine_c, engine_hash, view = build_side()
    assert trainer_hash == engine_hash and len(trainer_hash) == 64
    assert all(e.impl.arch == "gfx950" for e in engine_c.composition)
    assert process_contract.assert_contract_agreement(trainer_hash, other_side="trainer") is True
    monkeypatch.setenv("SKYRL_ISOEXEC_PIK_LEAVES", "8")
    with pytest.raises(RuntimeError, match="MISMATCH"):
        process_contract.assert_contract_agreement("0" * 64, other_side="trainer")
    # the library's ABI version folds into the handshake as an extension on both sides
    from isoexec_amd import _lib

    process_contract.register_contract_extension("libisoexec_hip.abi", lambda: _lib.lib().ix_abi_version())
    assert process_contract.contract_hash() != trainer_hash
    # install fingerprint: record what the hybrid runtimes bind and compare with the contract's view
    fingerprint._reset_for_tests()
    enforce._reset_for_tests()
    from isoexec_amd.ops.attention import varlen_attn
    from isoexec_amd.ops.logprobs import rowinv
    from isoexec_amd.ops.mm import mm_hip

    fingerprint.record_installs("mm", fingerprint.ALL_SITES, "hip_mfma_batch_invariant", mm_hip.linear_nt)
    fingerprint.record_installs("attention.varlen", fingerprint.ALL_SITES, "hip_varlen_ns1", varlen_attn.varlen_attention,
                                pinned={"num_splits": 1})
    fingerprint.record_installs("logprobs.log_softmax", fingerprint.ALL_SITES, "hip_rowinv_leaftree", rowinv.sampled_forward,
                                pinned={"leaves": rowinv.leaves(), "block": rowinv.BLOCK, "accum": "kahan_fp32"})
    assert fingerprint.log_fingerprint(view) == []
    monkeypatch.setenv("SKYRL_ISOEXEC_PIK_LEAVES", "4")  # a one-sided flag flip shows up as a pin mismatch
    fingerprint.record_installs("logprobs.log_softmax", fingerprint.ENGINE_SITES, "hip_rowinv_leaftree", rowinv.sampled_forward,
                                pinned={"leaves": rowinv.leaves(), "block": rowinv.BLOCK, "accum": "kahan_fp32"})
    assert len(fingerprint.log_fingerprint(view)) == 2
    process_contract._reset_for_tests()


def test_config4_full_size_ratio_is_exactly_one():
    """8 layers (3 GatedDeltaNet : 1 attention), hidden 2048, 128 experts top-8, vocabulary 151936;
    64 sequences of a 2048-token prompt and 512 sampled response tokens."""
    from isoexec_amd.runtimes.hybrid import HybridConfig

    cfg = HybridConfig()
    n, prompt, steps = 64, 2048, 512
    w, engine, trainer, packed, lens, toks, lps = rollout_then_score(cfg, [prompt] * n, steps, seed=7)
    assert toks.shape == (n, steps) and bool(torch.isfinite(lps).all())
    scored = torch.stack(trainer.response_logprobs(packed, lens, [prompt] * n))
    mismatched = int((scored.view(torch.int32) != lps.view(torch.int32)).sum())
    assert mismatched == 0, f"{mismatched} of {n * steps} response tokens differ"
    assert bool((torch.exp(scored - lps) == 1.0).all())
