"""GPU parity: MoE router, permutation, grouped experts and combine (config 3, reduced where stated)."""

import numpy as np
import pytest
import torch

from _util import DevicePrims, bf16_to_np, cpu_gen, np_bits, np_to_bf16, same_bits
from oracle import moe as o_moe

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def dprims():
    return DevicePrims(DEV)


def make_moe(T, H, E, F, seed):
    g = cpu_gen(seed)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    wr = (0.02 * torch.randn(E, H, generator=g)).to(torch.bfloat16)
    w1 = (0.02 * torch.randn(E, 2 * F, H, generator=g)).to(torch.bfloat16)
    w2 = (0.02 * torch.randn(E, H, F, generator=g)).to(torch.bfloat16)
    return x, wr, w1, w2


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("E,k", [(128, 8), (16, 4), (60, 2), (200, 1)])
def test_router_bit_exact_ties_and_nan(mode, E, k, dprims):
    from isoexec_amd.ops.moe.moe_hip import router_topk

    g = cpu_gen(E + k)
    logits = 2 * torch.randn(64, E, generator=g)
    logits[1, :] = 0.5  # all tied: lowest indices win
    logits[2, 3] = float("nan")  # NaN counts as -inf
    logits[3, 5] = logits[3, 9] = 7.0  # a tied pair at the top
    logits[4, :] = -1e4
    logits[4, 7] = 80.0  # outlier: the other exp terms underflow
    idx, prob, dprob, dmap = router_topk(logits.to(DEV), k, pre_softmax=bool(mode), dense=True)
    widx, wprob = o_moe.router_topk(logits.numpy(), k, mode, prims=dprims)
    assert np.array_equal(idx.cpu().numpy(), widx)
    assert np.array_equal(np_bits(prob.cpu().numpy()), np_bits(wprob))
    assert idx[1].tolist() == list(range(k))
    if E > 3 and k < E:
        assert 3 not in idx[2].tolist() or k >= E
    wd, wm = o_moe.dense_from_topk(widx, wprob, E)
    assert np.array_equal(np_bits(dprob.cpu().numpy()), np_bits(wd)) and np.array_equal(dmap.cpu().numpy(), wm)
    # library check: torch.topk membership and softmax values (libm exp) within 1e-6
    lt = torch.nan_to_num(logits, nan=float("-inf"))
    if mode == 0:
        tv, _ = torch.topk(lt, k, dim=1)
        ref = torch.softmax(tv, dim=-1)
    else:
        tv, _ = torch.topk(torch.softmax(lt, dim=-1), k, dim=1)
        ref = tv / tv.sum(-1, keepdim=True)
    assert (prob.cpu() - ref).abs().max().item() <= 2e-6
    # row invariance
    i1, p1, _, _ = router_topk(logits[5:6].to(DEV), k, pre_softmax=bool(mode))
    assert torch.equal(i1, idx[5:6]) and same_bits(p1, prob[5:6])


@pytest.mark.parametrize("T,E,k", [(1, 128, 8), (33, 128, 8), (256, 128, 8), (200, 37, 2), (64, 512, 16), (257, 37, 2), (700, 16, 4), (513, 128, 8)])
def test_permutation_exact(T, E, k):
    from isoexec_amd.ops.moe.moe_hip import permute, router_topk

    g = cpu_gen(T)
    logits = torch.randn(T, E, generator=g)
    logits[:, :4] += 3.0  # skewed load
    idx, prob, _, _ = router_topk(logits.to(DEV), k)
    for BM in (32, 128, 256):
        p = permute(idx, prob, E, BM=BM)
        counts, st, pp, cr = o_moe.permute(idx.cpu().numpy(), prob.cpu().numpy(), E)
        assert np.array_equal(p.counts.cpu().numpy(), counts)
        assert np.array_equal(p.sorted_token.cpu().numpy(), st)
        assert np.array_equal(np_bits(p.permuted_prob.cpu().numpy()), np_bits(pp))
        assert np.array_equal(p.combine_rows.cpu().numpy(), cr)
        assert np.array_equal(p.offsets.cpu().numpy(), np.concatenate([[0], np.cumsum(counts)]))
        meta = p.tile_meta.cpu().numpy()
        nt = int(meta[0])
        te, r0, nr = (meta[1 + i * p.max_tiles: 1 + i * p.max_tiles + nt] for i in range(3))
        assert nt == int(sum(-(-c // BM) for c in counts)) and nr.sum() == T * k
        off = np.concatenate([[0], np.cumsum(counts)])
        for e_, r_, n_ in zip(te, r0, nr):
            assert off[e_] <= r_ and r_ + n_ <= off[e_ + 1] and 0 < n_ <= BM


def test_moe_ffn_parity_and_batch_invariance(dprims):
    """Reduced config 3 (hidden 256, 16 experts, top-4, inter 128): the full chain against the
    oracle (device router logits fed to the oracle so the discrete choice is compared like for
    like), then every token alone == co-batched == co-batched under skewed routing, for every BM."""
    from isoexec_amd.ops.mm.mm_hip import router_gemm
    from isoexec_amd.ops.moe.moe_hip import combine, experts_forward, moe_ffn_forward, permute, router_topk

    T, H, E, F, k = 300, 256, 16, 128, 4
    x, wr, w1, w2 = make_moe(T, H, E, F, seed=1)
    xd, wrd, w1d, w2d = (t.to(DEV) for t in (x, wr, w1, w2))
    for mode in (0, 1):
        logits = router_gemm(xd, wrd)
        idx, prob, _, _ = router_topk(logits, k, pre_softmax=bool(mode))
        p = permute(idx, prob, E)
        eo = experts_forward(xd, w1d, w2d, p)
        out = combine(eo, p)
        # oracle with float64 matmuls: each bf16 round may differ by an ulp where the fp32 sum
        # lands near a rounding boundary, so compare with a tolerance in bf16 ulps of the scale
        mm64 = lambda a, w: (a.astype(np.float64) @ w.astype(np.float64).T).astype(np.float32)
        counts, st, pp, cr = o_moe.permute(idx.cpu().numpy(), prob.cpu().numpy(), E)
        weo, _ = o_moe.expert_chain(bf16_to_np(x), bf16_to_np(w1), bf16_to_np(w2), st, pp, counts, prims=dprims,
                                    matmul=mm64)
        got = bf16_to_np(eo)
        scale = np.abs(weo).max()
        assert np.abs(got - weo).max() <= 2.0 ** -7 * scale, (np.abs(got - weo).max(), scale)
        assert (got != weo).mean() < 0.05
        # combine is exact given the expert rows
        assert same_bits(out.cpu(), np_to_bf16(o_moe.combine(got, cr)))
        assert same_bits(combine(eo, p, fp32_acc=True).cpu(), np_to_bf16(o_moe.combine(got, cr, fp32_acc=True)))
        assert same_bits(moe_ffn_forward(xd, wrd, w1d, w2d, k, pre_softmax=bool(mode)), out)
    # invariance: alone vs co-batched vs skewed co-batch, all BM
    ref = moe_ffn_forward(xd, wrd, w1d, w2d, k, BM=256)
    for BM in (32, 128):
        assert same_bits(moe_ffn_forward(xd, wrd, w1d, w2d, k, BM=BM), ref)
    # the square 128 x 128 tile (two workgroups per CU) through ix_moe_experts_tile: same rows, same bits
    idx, prob, _, _ = router_topk(router_gemm(xd, wrd), k)
    rows = experts_forward(xd, w1d, w2d, permute(idx, prob, E, BM=128))
    assert same_bits(experts_forward(xd, w1d, w2d, permute(idx, prob, E, BM=128, BN=128)), rows)
    with pytest.raises(RuntimeError):
        experts_forward(xd, w1d, w2d, permute(idx, prob, E, BM=256, BN=128))   # only the square pairing exists
    for t in (0, 17, 299):
        assert same_bits(moe_ffn_forward(xd[t:t + 1], wrd, w1d, w2d, k), ref[t:t + 1])
    assert same_bits(moe_ffn_forward(xd[:33], wrd, w1d, w2d, k), ref[:33])
    # skew the OTHER tokens' routing (+3.0 on 4 experts): token 5 keeps its own logits
    bias = torch.zeros(T, E, device=DEV)
    bias[:, :4] = 3.0
    bias[5] = 0.0
    skew = moe_ffn_forward(xd, wrd, w1d, w2d, k, logit_bias=bias)
    assert same_bits(skew[5:6], ref[5:6])


def test_config3_shapes_small_T():
    """Config 3 dimensions (hidden 2048, 128 experts, top-8, inter 768, softmax-then-topk with
    renormalisation, +3.0 skew on 4 experts) at T in {1, 33, 512}: alone == co-batched bits."""
    from isoexec_amd.ops.moe.moe_hip import moe_ffn_forward

    T, H, E, F, k = 512, 2048, 128, 768, 8
    x, wr, w1, w2 = make_moe(T, H, E, F, seed=3)
    xd, wrd, w1d, w2d = (t.to(DEV) for t in (x, wr, w1, w2))
    ref = moe_ffn_forward(xd, wrd, w1d, w2d, k, pre_softmax=True)
    assert bool(torch.isfinite(ref.float()).all())
    assert same_bits(moe_ffn_forward(xd[:1], wrd, w1d, w2d, k, pre_softmax=True), ref[:1])
    assert same_bits(moe_ffn_forward(xd[:33], wrd, w1d, w2d, k, pre_softmax=True), ref[:33])
    bias = torch.zeros(T, E, device=DEV)
    bias[1:, :4] = 3.0
    skew = moe_ffn_forward(xd, wrd, w1d, w2d, k, pre_softmax=True, logit_bias=bias)
    assert same_bits(skew[:1], ref[:1])
    # dense fp64 reference for token 0 (top-8 of softmax, renormalised)
    lg = (x[:1].double() @ wr.double().T)
    pr = torch.softmax(lg, -1)
    tv, ti = torch.topk(pr, k)
    tv = tv / tv.sum()
    acc = torch.zeros(H, dtype=torch.float64)
    for pj, ej in zip(tv[0], ti[0]):
        h = x[0].double() @ w1[ej].double().T
        a = torch.nn.functional.silu(h[:F]) * h[F:] * pj
        acc += a @ w2[ej].double().T
    err = (ref[0].double().cpu() - acc).abs().max().item()
    assert err <= 0.03 * acc.abs().max().item() + 1e-3, err


@pytest.mark.parametrize("T,E,k,mode", [(1, 128, 8, 1), (16, 128, 8, 1), (64, 128, 8, 1), (64, 128, 8, 0), (255, 128, 8, 1),
                                         (256, 128, 8, 0), (33, 64, 4, 1), (100, 16, 2, 0), (70, 60, 4, 1)])
def test_one_launch_route_and_permute_equals_the_two_calls(T, E, k, mode):
    """``ix_moe_route_one_tile`` (router + permutation of a decode-size batch in one launch) against ``router_topk`` +
    ``permute``, both pinned against the oracle in this file: every integer and every weight, on poisoned outputs, with
    ties and a NaN in the logits and a skewed routing."""
    from isoexec_amd.ops.moe.moe_hip import permute, route_and_permute, router_topk

    g = cpu_gen(1000 * T + E)
    logits = torch.randn(T, E, generator=g)
    logits[:, :4] += 3.0
    logits[0, : min(E, 12)] = 0.25          # ties: lowest index wins
    if T > 2:
        logits[2, 5] = float("nan")
    lg = logits.to(DEV)
    pre = bool(mode)
    for scaling in (None, 2.5):
        idx, prob, _, _ = router_topk(lg, k, pre_softmax=pre, scaling_factor=scaling)
        want = permute(idx, prob, E)
        gi, gp, got = route_and_permute(lg, k, pre_softmax=pre, scaling_factor=scaling)
        assert torch.equal(gi, idx) and same_bits(gp, prob)
        assert (got.BM, got.max_tiles) == (want.BM, want.max_tiles)
        n = int(want.tile_meta[0])
        assert int(got.tile_meta[0]) == n
        for name in ("counts", "offsets", "sorted_token", "combine_rows"):
            assert torch.equal(getattr(got, name), getattr(want, name)), name
        assert same_bits(got.permuted_prob, want.permuted_prob)
        mt = want.max_tiles
        for part in range(3):
            assert torch.equal(got.tile_meta[1 + part * mt: 1 + part * mt + n], want.tile_meta[1 + part * mt: 1 + part * mt + n])
    # a strided logits view (the gating product's output inside a wider buffer)
    wide = torch.zeros(T, E + 8, device=DEV)
    wide[:, :E] = lg
    gi2, gp2, got2 = route_and_permute(wide[:, :E], k, pre_softmax=pre, scaling_factor=2.5)
    assert torch.equal(gi2, gi) and same_bits(gp2, gp) and torch.equal(got2.sorted_token, got.sorted_token)


@pytest.mark.parametrize("T,H,k", [(1, 2048, 8), (67, 2048, 8), (300, 1024, 4), (9, 4096, 8), (130, 512, 4), (5, 2048, 2)])
def test_combine_add_norm_in_one_launch_equals_the_two_calls(T, H, k):
    """``combine_add_rms_norm`` against ``combine`` + ``fused_add_rms_norm_gamma`` (both pinned against the oracle):
    the normed rows and the new residual stream, both combine arithmetics, bit for bit."""
    from isoexec_amd.ops.moe.moe_hip import combine, combine_add_rms_norm, permute, router_topk
    from isoexec_amd.ops.norms.fused_outnorm import fused_add_rms_norm_gamma

    g = cpu_gen(77 * T + H)
    E = 16
    idx, prob, _, _ = router_topk(torch.randn(T, E, generator=g).to(DEV), k)
    p = permute(idx, prob, E)
    eo = torch.randn(T * k, H, generator=g).to(torch.bfloat16).to(DEV)
    res = torch.randn(T, H, generator=g).to(torch.bfloat16).to(DEV)
    w = (0.1 * torch.randn(H, generator=g)).to(torch.bfloat16).to(DEV)
    for fp32_acc in (False, True):
        want_y, want_h = fused_add_rms_norm_gamma(combine(eo, p, fp32_acc=fp32_acc), res, w, 1e-6)
        got = combine_add_rms_norm(eo, p, res, w, 1e-6, fp32_acc=fp32_acc)
        assert got is not None
        assert same_bits(got[0], want_y) and same_bits(got[1], want_h), fp32_acc
    # NaNs and infinities (with payloads and signs of their own) in expert rows, residual and weight: the one launch
    # rounds inside its chain with the hardware convert and must still store what the two calls store
    eo2, res2, w2 = eo.clone(), res.clone(), w.clone()
    bits = eo2.view(torch.int16)
    bits[0, 3] = 0x7fa5                                      # a NaN with a payload
    bits[(T * k) // 2, 9] = -1                               # 0xffff: negative NaN, full payload
    eo2[T * k - 1, 17] = float("inf")
    eo2[0, 40] = float("-inf")
    res2[T - 1, 5] = float("nan")
    res2[0, 41] = float("inf")
    res2.view(torch.int16)[T // 2, 100] = 0x7f81             # signalling-pattern NaN
    w2[7] = float("inf")
    w2[200] = float("nan")
    eo2[:, 300] = 3.0e38                                     # sums overflow to infinity on the way
    for fp32_acc in (False, True):
        want_y, want_h = fused_add_rms_norm_gamma(combine(eo2, p, fp32_acc=fp32_acc), res2, w2, 1e-6)
        got = combine_add_rms_norm(eo2, p, res2, w2, 1e-6, fp32_acc=fp32_acc)
        assert not torch.isfinite(want_y.float()).all() and not torch.isfinite(want_h.float()).all()
        assert same_bits(got[0], want_y) and same_bits(got[1], want_h), fp32_acc
    assert combine_add_rms_norm(eo[:, :384].contiguous(), p, res[:, :384].contiguous(), w[:384].contiguous(), 1e-6) is None
