"""CPU: pins for the oracle's primitives, norms, matmul reference and log-softmax tree."""

import numpy as np
import torch

from oracle import logprobs as o_lp
from oracle import mm as o_mm
from oracle import norms as o_norms
from oracle import prims as o_prims


def test_round_bf16_matches_torch_cast():
    rng = np.random.default_rng(0)
    x = np.concatenate([(rng.standard_normal(20000) * 10 ** rng.uniform(-30, 30, 20000)).astype(np.float32),
                        np.array([0.0, -0.0, np.inf, -np.inf, 1.00390625, 1.01171875, 3.3e38, 1e-45], np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
    got = o_prims.round_bf16(x)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.isnan(o_prims.round_bf16(np.array([np.nan], np.float32))[0])


def test_pairwise_tree_is_the_adjacent_tree():
    a = np.array([1e8, 1.0, -1e8, 1.0, 3.0, 4.0, 5.0, 6.0], np.float32)
    want = np.float32(np.float32(np.float32(a[0] + a[1]) + np.float32(a[2] + a[3]))
                      + np.float32(np.float32(a[4] + a[5]) + np.float32(a[6] + a[7])))
    assert o_prims.pairwise_tree(a) == want
    assert o_prims.pairwise_tree(a) != np.float32(np.sum(a.astype(np.float64)))  # order is visible


def test_combine_order_matches_reference_schedule():
    # the G=8 schedule the reference documents (pik/plan.py:104-119)
    assert o_lp.combine_order(8) == [(0, 0, 1), (2, 2, 3), (4, 4, 5), (6, 6, 7), (0, 0, 2), (4, 4, 6), (0, 0, 4)]
    assert o_lp.combine_order(1) == [] and o_lp.combine_order(2) == [(0, 0, 1)]


def test_logprob_against_fp64_truth_and_adversarial_rows():
    rng = np.random.default_rng(1)
    V = 151936
    x = o_prims.round_bf16((4 * rng.standard_normal((6, V))).astype(np.float32))
    x[1, :] = -30.0
    x[1, 77] = 40.0  # one dominant column: every other term is tiny
    x[2, :] = 0.25  # constant row
    L = V // 8
    t = np.array([0, 77, 5, L, L - 1, V - 1])
    lp, lse = o_lp.rowinv_sampled(x, t, 8)
    truth = o_lp.truth_fp64(x, t)
    assert np.abs(lp - truth).max() <= 2e-6
    assert abs(lp[2] + np.log(V)) <= 1e-6  # closed form: S == V exactly
    full = o_lp.rowinv_full(x[:2], 8)
    assert np.array_equal(full[np.arange(2), t[:2]].view(np.uint32), lp[:2].view(np.uint32))
    bad, _ = o_lp.rowinv_sampled(x[:2], np.array([-1, V]), 8)
    assert (bad == 0).all()


def test_logprob_tree_brute_force_tiny():
    """Scalar evaluation of the documented tree on V = 32, G = 4 (one masked block per leaf)."""
    rng = np.random.default_rng(2)
    x = rng.standard_normal((1, 32)).astype(np.float32)
    f = np.float32
    m = x.max()
    leaves = []
    for g in range(4):
        terms = [f(np.exp2(f(f(x[0, g * 8 + i] - m) * o_prims.LOG2E))) for i in range(8)]
        # 8 live columns sit in chunk 0 at positions 0..7: the tree over 512 columns reduces to
        # the adjacent tree over those 8 (all other columns are +0)
        s = f(f(f(terms[0] + terms[1]) + f(terms[2] + terms[3])) + f(f(terms[4] + terms[5]) + f(terms[6] + terms[7])))
        leaves.append(s)
    S = f(f(leaves[0] + leaves[1]) + f(leaves[2] + leaves[3]))
    want = f(f(x[0, 3] - m) - f(np.log(S)))
    got, _ = o_lp.rowinv_sampled(x, np.array([3]), 4)
    assert got[0] == want


def test_logprob_row_invariance_and_kahan_blocks():
    rng = np.random.default_rng(3)
    x = o_prims.round_bf16((3 * rng.standard_normal((9, 40960))).astype(np.float32))
    t = rng.integers(0, 40960, 9)
    all_rows, _ = o_lp.rowinv_sampled(x, t, 8)
    for i in (0, 4, 8):
        one, _ = o_lp.rowinv_sampled(x[i:i + 1], t[i:i + 1], 8)
        assert one[0] == all_rows[i]


def test_rmsnorm_against_library_and_fp64():
    g = torch.Generator().manual_seed(4)
    for N in (128, 2048, 4096, 100):
        x = torch.randn(33, N, generator=g).to(torch.bfloat16)
        w = (0.02 * torch.randn(N, generator=g)).to(torch.bfloat16)
        got = o_norms.rms_norm_gamma(x.float().numpy(), w.float().numpy(), 1e-6)
        lib = (torch.nn.functional.rms_norm(x, (N,), None, 1e-6) * (1.0 + w)).float().numpy()
        ulp = 2.0 ** -7 * np.maximum(np.abs(lib), 2.0 ** -20)
        assert (np.abs(got - lib) <= ulp).all() and (got != lib).mean() < 0.01
        x64 = x.double().numpy()
        truth = x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + 1e-6) * (1.0 + w.double().numpy())
        assert (np.abs(got - truth) <= 2.0 ** -6 * np.abs(truth) + 1e-6).all()
        one = o_norms.rms_norm_gamma(x[5:6].float().numpy(), w.float().numpy(), 1e-6)
        assert np.array_equal(one[0], got[5])
    plain = o_norms.rms_norm_gamma(x.float().numpy(), w.float().numpy(), 1e-6, zero_centered=False)
    lib = (torch.nn.functional.rms_norm(x, (N,), None, 1e-6) * w).float().numpy()
    assert (np.abs(plain - lib) <= 2.0 ** -7 * np.maximum(np.abs(lib), 2.0 ** -20)).all()


def test_gated_and_add_norm_against_eager_expression():
    g = torch.Generator().manual_seed(5)
    x = torch.randn(7, 4, 128, generator=g).to(torch.bfloat16)
    gate = (3 * torch.randn(7, 4, 128, generator=g)).to(torch.bfloat16)
    w = (0.02 * torch.randn(128, generator=g)).to(torch.bfloat16)
    got = o_norms.gated_out_norm(x.float().numpy(), gate.float().numpy(), w.float().numpy(), 1e-6)
    # eager form (gdn_fla_shim.py:390-425): norm in bf16, SiLU(gate) in fp32, one round
    y = torch.nn.functional.rms_norm(x.reshape(-1, 128), (128,), None, 1e-6) * (1.0 + w)
    eager = (y.float() * torch.nn.functional.silu(gate.reshape(-1, 128).float())).to(torch.bfloat16).float().numpy()
    assert (np.abs(got - eager) <= 2.0 ** -6 * np.maximum(np.abs(eager), 2.0 ** -20)).all()
    r = torch.randn(7, 512, generator=g).to(torch.bfloat16)
    xx = torch.randn(7, 512, generator=g).to(torch.bfloat16)
    w2 = (0.02 * torch.randn(512, generator=g)).to(torch.bfloat16)
    yy, h = o_norms.add_rms_norm_gamma(xx.float().numpy(), r.float().numpy(), w2.float().numpy(), 1e-6)
    assert np.array_equal(h, (xx + r).float().numpy())


def test_gemm_reference_and_exact_integer_case():
    rng = np.random.default_rng(6)
    a, w = o_mm.small_int_operands(rng, 5, 9, 300)
    exact = o_mm.gemm_nt_fp64(a, w)
    assert np.array_equal(o_mm.gemm_nt_bf16(a, w), o_prims.round_bf16(exact.astype(np.float32)))
    a = o_prims.round_bf16(rng.standard_normal((8, 512)).astype(np.float32))
    w = o_prims.round_bf16((0.02 * rng.standard_normal((40, 512))).astype(np.float32))
    assert (np.abs(o_mm.gemm_nt_bf16(a, w) - o_mm.gemm_nt_fp64(a, w)) <= o_mm.gemm_tolerance(a, w)).all()
    b = o_prims.round_bf16(rng.standard_normal(40).astype(np.float32))
    ref = (torch.from_numpy(a).bfloat16() @ torch.from_numpy(w).bfloat16().T + torch.from_numpy(b).bfloat16())
    got = o_mm.gemm_nt_bf16(a, w, b)
    assert (np.abs(got - ref.float().numpy()) <= 2.0 ** -6 * np.abs(got) + 1e-3).all()
