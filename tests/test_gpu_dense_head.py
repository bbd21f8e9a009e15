"""GPU parity: primitives, RMSNorm family, batch-invariant GEMMs, log-softmax/gather (configs 1)."""

import numpy as np
import pytest
import torch

from _util import DevicePrims, bf16_to_np, bits, cpu_gen, np_bits, np_to_bf16, same_bits
from oracle import logprobs as o_lp
from oracle import mm as o_mm
from oracle import norms as o_norms
from oracle import prims as o_prims

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def dprims():
    return DevicePrims(DEV)


# ---- primitives ---------------------------------------------------------------------------------
def test_prim_round_bf16_and_rsqrt_bit_exact(dprims):
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(4096).astype(np.float32) * 7,
                        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.4e38, 1e-40, np.inf, -np.inf], np.float32)])
    got = dprims._run("round_bf16", x)
    assert np.array_equal(np_bits(got), np_bits(o_prims.round_bf16(x)))
    pos = np.abs(x[np.isfinite(x)]) + np.float32(1e-6)
    assert np.array_equal(np_bits(dprims._run("rsqrt_ieee", pos)), np_bits(o_prims.Prims.rsqrt_ieee(pos)))


def test_prim_transcendentals_close_to_libm(dprims):
    rng = np.random.default_rng(2)
    x = (rng.standard_normal(8192) * 8).astype(np.float32)
    host = o_prims.DEFAULT
    for name, arg in (("exp", x), ("sigmoid", x), ("silu_div", x), ("softplus", x), ("log", np.abs(x) + 1e-3),
                      ("exp_fast", -np.abs(x) * 4), ("exp2", np.clip(-np.abs(x) * 4, -120.0, 0.0))):
        got = dprims._run(name, arg)
        ref = getattr(host, name)(arg.astype(np.float32))
        rel = np.abs(got - ref) / np.maximum(np.abs(ref), 1e-30)
        # exp_fast, and the sigmoid built on the hardware 2^x, round their argument product once:
        # relative error <= |x| * 2^-24 * ln2 + a few ulp
        tol = 6e-6 if name in ("exp_fast", "sigmoid", "silu_div") else 4e-7
        assert rel.max() <= tol, (name, rel.max())


# ---- RMSNorm family --------------------------------------------------------------------------------
@pytest.mark.parametrize("N", [128, 1024, 2048, 4096, 8192, 100, 24])
@pytest.mark.parametrize("zc", [True, False])
def test_rmsnorm_bit_exact_and_row_invariant(N, zc):
    from isoexec_amd.ops.norms.fused_outnorm import fused_rms_norm_gamma

    g = cpu_gen(10 + N)
    x = torch.randn(300, N, generator=g).to(torch.bfloat16)
    w = (0.02 * torch.randn(N, generator=g) + (0.0 if zc else 1.0)).to(torch.bfloat16)
    want = o_norms.rms_norm_gamma(bf16_to_np(x), bf16_to_np(w), 1e-6, zero_centered=zc)
    full = fused_rms_norm_gamma(x.to(DEV), w.to(DEV), 1e-6, zero_centered=zc)
    assert same_bits(full.cpu(), np_to_bf16(want))
    for M in (1, 5, 64):
        part = fused_rms_norm_gamma(x[:M].to(DEV), w.to(DEV), 1e-6, zero_centered=zc)
        assert same_bits(part, full[:M])


def test_gated_out_norm_bit_exact(dprims):
    from isoexec_amd.ops.norms.fused_outnorm import fused_gated_out_norm

    g = cpu_gen(3)
    T, HV, N = 37, 4, 128
    x = torch.randn(T, HV, N, generator=g).to(torch.bfloat16)
    proj = (3 * torch.randn(T, 2 * HV * N + 16, generator=g)).to(torch.bfloat16)
    gate = proj[:, 16:16 + HV * N].view(T, HV, N)  # a strided slice of a wider projection
    w = (0.02 * torch.randn(N, generator=g)).to(torch.bfloat16)
    want = o_norms.gated_out_norm(bf16_to_np(x), bf16_to_np(gate), bf16_to_np(w), 1e-6, prims=dprims)
    pd = proj.to(DEV)
    got = fused_gated_out_norm(x.to(DEV), pd[:, 16:16 + HV * N].view(T, HV, N), w.to(DEV), 1e-6)
    assert same_bits(got.cpu(), np_to_bf16(want))
    host = o_norms.gated_out_norm(bf16_to_np(x), bf16_to_np(gate), bf16_to_np(w), 1e-6)
    assert np.abs(bf16_to_np(got) - host).max() <= 2 ** -6  # <= 1 bf16 ulp at |y| < 4 with libm's exp


def test_add_rmsnorm_bit_exact():
    from isoexec_amd.ops.norms.fused_outnorm import fused_add_rms_norm_gamma

    g = cpu_gen(4)
    x = torch.randn(65, 2048, generator=g).to(torch.bfloat16)
    r = torch.randn(65, 2048, generator=g).to(torch.bfloat16)
    w = (0.02 * torch.randn(2048, generator=g)).to(torch.bfloat16)
    want_y, want_h = o_norms.add_rms_norm_gamma(bf16_to_np(x), bf16_to_np(r), bf16_to_np(w), 1e-6)
    y, h = fused_add_rms_norm_gamma(x.to(DEV), r.to(DEV), w.to(DEV), 1e-6)
    assert same_bits(h.cpu(), np_to_bf16(want_h)) and same_bits(y.cpu(), np_to_bf16(want_y))


# ---- dense GEMM ----------------------------------------------------------------------------------
@pytest.mark.parametrize("tile", [1, 2, 3, 4, 5, 6])
def test_gemm_small_integer_known_answer(tile):
    """Small-integer operands: every partial sum is exact in fp32, so any correct kernel returns
    exactly the integer matmul. Catches a wrong fragment layout, a dropped k-slice, a bad tail."""
    from isoexec_amd.ops.mm.mm_hip import linear_nt

    rng = np.random.default_rng(tile)
    for (M, N, K) in ((1, 40, 64), (7, 1000, 200), (513, 333, 4096), (300, 256, 72)):
        a, w = o_mm.small_int_operands(rng, M, N, K)
        want = o_mm.gemm_nt_fp64(a, w)
        got = linear_nt(np_to_bf16(a, DEV), np_to_bf16(w, DEV), tile=tile)
        assert np.array_equal(bf16_to_np(got).astype(np.float64), o_prims.round_bf16(want.astype(np.float32)))


def test_gemm_tolerance_and_bias():
    from isoexec_amd.ops.mm.mm_hip import linear_nt

    g = cpu_gen(5)
    M, N, K = 129, 777, 1024
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (0.02 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
    b = torch.randn(N, generator=g).to(torch.bfloat16)
    an, wn, bn = bf16_to_np(a), bf16_to_np(w), bf16_to_np(b)
    for bias, bnp in ((None, None), (b, bn)):
        got = bf16_to_np(linear_nt(a.to(DEV), w.to(DEV), None if bias is None else bias.to(DEV)))
        truth = o_mm.gemm_nt_fp64(an, wn, bnp)
        tol = o_mm.gemm_tolerance(an, wn) + (0 if bnp is None else 2.0 ** -8 * np.abs(truth))
        assert (np.abs(got - truth) <= tol).all()
        # and against the fp32-accumulated library matmul: equal up to one bf16 ulp, mostly equal
        lib = o_mm.gemm_nt_bf16(an, wn, bnp)
        assert (got != lib).mean() < 0.02


def test_gemm_row_bits_independent_of_M_and_tile():
    """Config 1's invariance at a reduced vocabulary: row m's logits are bitwise the same at
    M in {1, 7, 64, 513} and under every tile shape."""
    from isoexec_amd.ops.mm.mm_hip import linear_nt

    g = cpu_gen(6)
    K, N = 4096, 2000
    a = torch.randn(513, K, generator=g).to(torch.bfloat16).to(DEV)
    w = (0.02 * torch.randn(N, K, generator=g)).to(torch.bfloat16).to(DEV)
    ref = linear_nt(a, w, tile=3)
    for tile in (1, 2, 4, 5, 6):
        assert same_bits(linear_nt(a, w, tile=tile), ref)
    for M in (1, 7, 64):
        assert same_bits(linear_nt(a[:M].contiguous(), w), ref[:M])
        assert same_bits(linear_nt(a[200:200 + M].contiguous(), w), ref[200:200 + M])


def test_gemm_fp32_out_row_max_and_fused_head(dprims):
    """fp32 store == the accumulator whose bf16 round is the bf16 store; the epilogue row max is
    the exact max of the stored row; the fused dense-head pipeline == the three ops run apart."""
    from isoexec_amd.ops.logprobs.rowinv import dense_head_logprobs, sampled_forward
    from isoexec_amd.ops.mm.mm_hip import linear_nt
    from isoexec_amd.ops.norms.fused_outnorm import fused_rms_norm_gamma

    g = cpu_gen(12)
    M, K, V = 300, 512, 8192
    h = torch.randn(M, K, generator=g).to(torch.bfloat16).to(DEV)
    wn = (0.02 * torch.randn(K, generator=g)).to(torch.bfloat16).to(DEV)
    wl = (0.05 * torch.randn(V, K, generator=g)).to(torch.bfloat16).to(DEV)
    t = torch.randint(0, V, (M,), generator=g).to(DEV)
    x = fused_rms_norm_gamma(h, wn, 1e-6)
    for tile in (1, 2, 3, 4, 5, 6):
        c16, rm = linear_nt(x, wl, tile=tile, want_row_max=True)
        c32, rm32 = linear_nt(x, wl, tile=tile, out_dtype=torch.float32, want_row_max=True)
        assert same_bits(c32.to(torch.bfloat16), c16)
        assert same_bits(rm, c16.float().amax(dim=1)) and same_bits(rm32, c32.amax(dim=1))
    lp_sep, _ = sampled_forward(c16, t, 8)
    lp_rm, _ = sampled_forward(c16, t, 8, row_max=rm)
    lp_fused, logits = dense_head_logprobs(h, wn, wl, t, g=8)
    assert same_bits(lp_rm, lp_sep) and same_bits(lp_fused, lp_sep) and same_bits(logits, c16)
    for Ms in (1, 7, 64):
        lp_s, _ = dense_head_logprobs(h[:Ms], wn, wl, t[:Ms], g=8)
        assert same_bits(lp_s, lp_sep[:Ms])


def test_gemm_f32_router_shape():
    from isoexec_amd.ops.mm.mm_hip import linear_f32_nt

    g = cpu_gen(7)
    x = torch.randn(300, 2048, generator=g).to(torch.bfloat16)
    w = (0.02 * torch.randn(128, 2048, generator=g)).float()
    got = linear_f32_nt(x.to(DEV), w.to(DEV))
    truth = bf16_to_np(x).astype(np.float64) @ w.numpy().astype(np.float64).T
    mag = np.abs(bf16_to_np(x).astype(np.float64)) @ np.abs(w.numpy().astype(np.float64)).T
    assert (np.abs(got.cpu().numpy() - truth) <= 2048 * 2.0 ** -24 * mag + 1e-30).all()
    for M in (1, 33, 64, 65):
        assert same_bits(linear_f32_nt(x[:M].to(DEV), w.to(DEV)), got[:M])
    xf = x.float()
    assert same_bits(linear_f32_nt(xf.to(DEV), w.to(DEV)), got)  # bf16 widening is exact
    # bf16-representable router weight: the bf16 MFMA core with an fp32 store is the same product
    from isoexec_amd.ops.mm.mm_hip import router_gemm

    wb = w.to(torch.bfloat16)
    fast = router_gemm(x.to(DEV), wb.to(DEV))
    truth = bf16_to_np(x).astype(np.float64) @ bf16_to_np(wb).astype(np.float64).T
    mag = np.abs(bf16_to_np(x).astype(np.float64)) @ np.abs(bf16_to_np(wb).astype(np.float64)).T
    assert fast.dtype is torch.float32 and (np.abs(fast.cpu().numpy() - truth) <= 2048 * 2.0 ** -24 * mag + 1e-30).all()
    assert same_bits(router_gemm(x[:1].to(DEV), wb.to(DEV)), fast[:1])


# ---- log-softmax + gather ------------------------------------------------------------------------
def _lp_case(rows, V, seed, scale=4.0):
    g = cpu_gen(seed)
    x = (scale * torch.randn(rows, V, generator=g)).to(torch.bfloat16)
    t = torch.randint(0, V, (rows,), generator=g)
    return x, t


@pytest.mark.parametrize("rows,V,G", [(5, 8192, 8), (3, 151936, 8), (4, 4004, 4), (2, 40960, 1), (6, 131072, 16)])
def test_logprob_bit_exact_vs_oracle_both_shapes(rows, V, G, dprims):
    from isoexec_amd.ops.logprobs.rowinv import sampled_forward

    x, t = _lp_case(rows, V, 100 + rows)
    L = V // G
    t[0] = 0
    t[-1] = V - 1
    if rows > 2:
        t[1] = L  # first column of leaf 1 (rowinv_gpu.py:76-79 adversarial targets)
        t[2] = L - 1
    want_lp, want_lse = o_lp.rowinv_sampled(bf16_to_np(x), t.numpy(), G, prims=dprims)
    for shape in (1, 2):
        lp, lse = sampled_forward(x.to(DEV), t.to(DEV), G, force_shape=shape)
        assert np.array_equal(np_bits(lp.cpu().numpy()), np_bits(want_lp)), (shape,)
        assert np.array_equal(np_bits(lse.cpu().numpy()), np_bits(want_lse)), (shape,)
    truth = o_lp.truth_fp64(bf16_to_np(x), t.numpy())
    assert np.abs(lp.cpu().numpy() - truth).max() <= 1e-5  # reference gate: 1e-4 (rowinv.py:21-22)


def test_logprob_fp32_input_and_out_of_range_targets(dprims):
    from isoexec_amd.ops.logprobs.rowinv import sampled_forward

    g = cpu_gen(8)
    x = 5 * torch.randn(4, 8192, generator=g)
    t = torch.tensor([3, -1, 8192, 8191])
    want, _ = o_lp.rowinv_sampled(x.numpy(), t.numpy(), 8, prims=dprims)
    lp, _ = sampled_forward(x.to(DEV), t.to(DEV), 8)
    assert np.array_equal(np_bits(lp.cpu().numpy()), np_bits(want))
    assert lp[1].item() == 0.0 and lp[2].item() == 0.0
    # a bf16 row widened to fp32 is the same function
    xb = x.to(torch.bfloat16)
    a, _ = sampled_forward(xb.to(DEV), t.to(DEV), 8)
    b, _ = sampled_forward(xb.float().to(DEV), t.to(DEV), 8)
    assert same_bits(a, b)


def test_logprob_constant_row_closed_form():
    from isoexec_amd.ops.logprobs.rowinv import sampled_forward

    V = 151936
    x = torch.full((2, V), 1.5, dtype=torch.bfloat16)
    t = torch.tensor([7, V - 1])
    lp, lse = sampled_forward(x.to(DEV), t.to(DEV), 8)
    # every term is exp(0) = 1 exactly, all partial sums are integers below 2^24: S == V exactly
    assert abs(lp[0].item() + float(np.log(np.float32(V)))) <= 1e-6 and lp[0].item() == lp[1].item()


def test_logprob_row_bits_independent_of_row_count():
    """Each row's logprob is bitwise identical at M in {1, 7, 64, 513} (both launch shapes occur)."""
    from isoexec_amd.ops.logprobs.rowinv import full_forward, sampled_forward

    V = 151936
    x, t = _lp_case(513, V, 9)
    xd, td = x.to(DEV), t.to(DEV)
    ref, ref_lse = sampled_forward(xd, td, 8)
    for M in (1, 7, 64):
        lp, lse = sampled_forward(xd[:M], td[:M], 8)
        assert same_bits(lp, ref[:M]) and same_bits(lse, ref_lse[:M])
        lp, _ = sampled_forward(xd[300:300 + M], td[300:300 + M], 8)
        assert same_bits(lp, ref[300:300 + M])
    full = full_forward(xd[:3], 8)
    assert same_bits(full.gather(1, td[:3, None])[:, 0], ref[:3])
    assert same_bits(full_forward(xd[:3], 8, force_shape=1), full_forward(xd[:3], 8, force_shape=2))


def test_rowinv_entry_points_protocol(monkeypatch):
    from isoexec_amd.ops.logprobs import rowinv

    rowinv._reset_for_test()
    x, t = _lp_case(4, 8192, 11)
    xd, td = x.to(DEV), t.to(DEV)
    kw = dict(vocab_start_index=0, vocab_end_index=8192, group=None, src_dtype=torch.bfloat16)
    monkeypatch.delenv("SKYRL_ISOEXEC", raising=False)
    assert rowinv.rowinv_sampled_logprobs(xd, td, reference=None, **kw) is None  # inert unless enabled
    monkeypatch.setenv("SKYRL_ISOEXEC", "1")
    ref = lambda: torch.log_softmax(xd.float(), -1).gather(1, td[:, None])[:, 0]
    out = rowinv.rowinv_sampled_logprobs(xd, td, reference=ref, **kw)
    assert out is not None and out.shape == t.shape and rowinv.stats()["agreed"] is True
    assert (out - ref()).abs().max().item() <= 1e-5
    # 3-D logits [B, S, V] and chunked == unchunked bits
    x3 = xd.view(2, 2, 8192)
    out3 = rowinv.rowinv_sampled_logprobs(x3, td.view(2, 2), reference=None, **kw)
    assert same_bits(out3.reshape(-1), out)
    monkeypatch.setenv("SKYRL_ISOEXEC_PIK_LEAVES", "3")
    assert rowinv.rowinv_sampled_logprobs(xd, td, reference=None, **kw) is None  # not a power of two
    monkeypatch.setenv("SKYRL_ISOEXEC_PIK_LEAVES", "8")
    assert rowinv.rowinv_sampled_logprobs(xd[:, :8190].contiguous(), td.clamp(max=8189), reference=None,
                                          vocab_start_index=0, vocab_end_index=8190, group=None,
                                          src_dtype=torch.bfloat16) is None  # V % G != 0
    full = rowinv.rowinv_full_logprobs(xd, src_dtype=torch.bfloat16, reference=None)
    assert same_bits(full.gather(1, td[:, None])[:, 0], out)
