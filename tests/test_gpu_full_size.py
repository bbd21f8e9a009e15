"""The benchmark configurations at their full sizes, checked through size-independent properties.

No oracle runs here (it would take hours at these sizes): a row's bits must not depend on how many
rows share the call, how the sequence was cut into calls, or how loaded the experts are. Bit-exact
agreement with the oracle at small sizes is covered by the other GPU tests.
"""

import pytest
import torch

from _util import same_bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def dev_gen(seed):
    g = torch.Generator(device=DEV)
    g.manual_seed(seed)
    return g


def test_config1_dense_head_rows_do_not_depend_on_token_count():
    """Hidden 4096, vocabulary 151936, M in {1, 7, 64, 513, 4096}: norm -> LM head -> logprob."""
    from isoexec_amd.ops.logprobs.rowinv import dense_head_logprobs

    g = dev_gen(1)
    M, Hd, V = 4096, 4096, 151936
    hidden = torch.randn(M, Hd, device=DEV, generator=g).to(torch.bfloat16)
    gamma = (0.02 * torch.randn(Hd, device=DEV, generator=g)).to(torch.bfloat16)  # zero-centred: 1 + w
    head = (0.02 * torch.randn(V, Hd, device=DEV, generator=g)).to(torch.bfloat16)
    target = torch.randint(0, V, (M,), device=DEV, generator=g)
    lp, logits = dense_head_logprobs(hidden, gamma, head, target)
    assert bool(torch.isfinite(lp).all()) and float(lp.max()) < 0
    for m in (1, 7, 64, 513):
        lp_m, logits_m = dense_head_logprobs(hidden[:m], gamma, head, target[:m])
        assert same_bits(lp_m, lp[:m]) and same_bits(logits_m, logits[:m]), m
    # A row in the middle, alone and as the last row of a ragged batch.
    lp_1, _ = dense_head_logprobs(hidden[2000:2001], gamma, head, target[2000:2001])
    lp_r, _ = dense_head_logprobs(hidden[1488:2001], gamma, head, target[1488:2001])
    assert same_bits(lp_1, lp[2000:2001]) and same_bits(lp_r, lp[1488:2001])
    # Truth for a few rows in float64.
    rows = torch.tensor([0, 513, 4095], device=DEV)
    x = hidden[rows].double()
    xn = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-6) * (1 + gamma.double())
    ref = torch.log_softmax(xn @ head.double().T, -1).gather(1, target[rows].unsqueeze(1)).squeeze(1)
    assert float((lp[rows].double() - ref).abs().max()) < 0.05  # bf16 logits: ~3 significant digits


@pytest.mark.parametrize("B", [1, 16, 64, 256])
def test_config2_decode_equals_the_full_sequence_pass(B):
    """16 key heads, 32 value heads, d=128, conv width 4; T=8192 prefill then 512 decode steps.
    The decode outputs and the final states equal those of one pass over all 8704 tokens, and
    sequence 0 gives the same bits at every batch size."""
    from isoexec_amd.ops.gdn.gdn_recurrent_state import RecurrentGDN

    H, K, HV, V, W, T, S = 16, 128, 32, 128, 4, 8192, 512
    D = 2 * H * K + HV * V
    g = dev_gen(2)
    bf = torch.bfloat16
    params = dict(
        conv_weight=(0.4 * torch.randn(D, W, device=DEV, generator=g)).to(bf),
        conv_bias=(0.1 * torch.randn(D, device=DEV, generator=g)).to(bf),
        A_log=0.3 * torch.randn(HV, device=DEV, generator=g), dt_bias=0.3 * torch.randn(HV, device=DEV, generator=g),
        num_k_heads=H, head_k_dim=K, num_v_heads=HV, head_v_dim=V, device=DEV)
    L = T + S
    # Sequence b draws from its own seed, so sequence 0 is the same tokens at every B.
    x = torch.empty(B, L, D, dtype=bf, device=DEV)
    a = torch.empty(B, L, HV, dtype=bf, device=DEV)
    b = torch.empty(B, L, HV, dtype=bf, device=DEV)
    for i in range(B):
        gi = dev_gen(1000 + i)
        x[i] = torch.randn(L, D, device=DEV, generator=gi).to(bf)
        a[i] = torch.randn(L, HV, device=DEV, generator=gi).to(bf)
        b[i] = torch.randn(L, HV, device=DEV, generator=gi).to(bf)
    slots_cpu = [7 * i + 3 for i in range(B)]
    slots = torch.tensor(slots_cpu, device=DEV)

    whole = RecurrentGDN(capacity=B, **params)
    o_full = whole.prefill(slots, slots_cpu, x.view(B * L, D), a.view(B * L, HV), b.view(B * L, HV),
                           [i * L for i in range(B + 1)]).view(B, L, HV, V)
    assert bool(torch.isfinite(o_full.float()).all())

    split = RecurrentGDN(capacity=B, **params)
    o_pre = split.prefill(slots, slots_cpu, x[:, :T].reshape(B * T, D), a[:, :T].reshape(B * T, HV),
                          b[:, :T].reshape(B * T, HV), [i * T for i in range(B + 1)]).view(B, T, HV, V)
    assert same_bits(o_pre, o_full[:, :T].contiguous())
    del o_pre
    mism = 0
    for s in range(S):
        od = split.decode(slots, x[:, T + s].contiguous(), a[:, T + s].contiguous(), b[:, T + s].contiguous())
        mism += int(not same_bits(od, o_full[:, T + s].contiguous()))
    assert mism == 0
    rows_w = [whole.require_row(s) for s in slots_cpu]
    rows_s = [split.require_row(s) for s in slots_cpu]
    assert same_bits(whole.ssm_state[rows_w], split.ssm_state[rows_s])
    assert same_bits(whole.conv_state[rows_w], split.conv_state[rows_s])

    # Sequence 0 alone (B = 1) is the reference every batch size must reproduce.
    key = "_seq0"
    keep = (o_full[0, T:].clone(), whole.ssm_state[rows_w[0]].clone())
    store = test_config2_decode_equals_the_full_sequence_pass.__dict__.setdefault(key, {})
    if store:
        first = next(iter(store.values()))
        assert same_bits(keep[0], first[0]) and same_bits(keep[1], first[1])
    store[B] = keep


def test_config3_token_outputs_do_not_depend_on_cobatch_or_expert_load():
    """Hidden 2048, 128 experts, top-8, softmax-then-topk renormalised, intermediate 768; token counts
    {1, 33, 512, 4096, 16384}; +3.0 on the logits of 4 experts skews everyone else's routing."""
    from isoexec_amd.ops.moe.moe_hip import moe_ffn_forward

    T, Hd, E, F, k = 16384, 2048, 128, 768, 8
    g = dev_gen(3)
    bf = torch.bfloat16
    x = torch.randn(T, Hd, device=DEV, generator=g).to(bf)
    wr = (0.02 * torch.randn(E, Hd, device=DEV, generator=g)).to(bf)
    w1 = (0.02 * torch.randn(E, 2 * F, Hd, device=DEV, generator=g)).to(bf)
    w2 = (0.02 * torch.randn(E, Hd, F, device=DEV, generator=g)).to(bf)
    run = lambda xs, **kw: moe_ffn_forward(xs, wr, w1, w2, k, pre_softmax=True, **kw)
    ref = run(x)
    assert bool(torch.isfinite(ref.float()).all()) and float(ref.float().abs().max()) > 0
    for t in (1, 33, 512, 4096):
        assert same_bits(run(x[:t]), ref[:t]), t
    assert same_bits(run(x[9000:9001]), ref[9000:9001])
    assert same_bits(run(x[4063:4096]), ref[4063:4096])
    # Skew: every token but the probes gets +3.0 on experts 0..3, which piles most of the batch onto
    # four experts. The probes keep their own logits and must keep their bits.
    probes = torch.arange(0, T, 997, device=DEV)
    bias = torch.zeros(T, E, device=DEV)
    bias[:, :4] = 3.0
    bias[probes] = 0.0
    skew = run(x, logit_bias=bias)
    assert same_bits(skew[probes], ref[probes])
    changed = (skew != ref).any(dim=1).float().mean()
    assert float(changed) > 0.5  # the skew did move the others
    for bm in (32, 128, 256):
        assert same_bits(run(x, logit_bias=bias, BM=bm), skew), bm
