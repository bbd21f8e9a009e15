"""GPU parity of the chunk-boundary GatedDeltaNet forward (``ops/gdn/gdn_cpr.py``; reference gdn_cpr.py:104-319).

The checker is ``oracle.gdn.cpr_forward``: an unrounded fp32 state chain gives the state entering every chunk, that
state is snapshotted in the wire dtype, and every chunk is then scanned as its own sequence from its snapshot. Its
structure is pinned on the CPU against a float64 chunk-state pass (tests/test_oracle_gdn_moe.py). The reference's own
boundary arithmetic (third-party chunk kernels, absent here) cannot be reproduced bit for bit: that one parity is
unpinned. Also checked here: the special cases the structure fixes (one chunk per sequence = the recurrent forward;
fp32 wire = no rounding at the boundaries = the recurrent forward for every chunk size)."""

import numpy as np
import pytest
import torch

from _util import DevicePrims, bf16_to_np, cpu_gen, np_to_bf16, same_bits
from oracle import gdn as o_gdn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
H, K, HV, V = 2, 64, 4, 64


@pytest.fixture(scope="module")
def dprims():
    return DevicePrims(DEV)


def make_inputs(lens, seed):
    g = cpu_gen(seed)
    T = sum(lens)
    q = torch.nn.functional.normalize(torch.randn(1, T, H, K, generator=g), dim=-1)
    k = torch.nn.functional.normalize(torch.randn(1, T, H, K, generator=g), dim=-1)
    v = torch.randn(1, T, HV, V, generator=g)
    gate = -torch.nn.functional.softplus(torch.randn(1, T, HV, generator=g))
    beta = torch.sigmoid(torch.randn(1, T, HV, generator=g))
    return q, k, v, gate, beta


def oracle_cpr(q, k, v, gate, beta, lens, chunk, dprims, init=None):
    """``oracle.gdn.cpr_forward`` (pinned on the CPU against the float64 chunk-state pass, tests/test_oracle_gdn_moe.py)
    on the bf16 images of the inputs, with the device's transcendentals plugged in."""
    r = lambda t: bf16_to_np(t.to(torch.bfloat16))
    return o_gdn.cpr_forward(r(q[0]), r(k[0]), r(v[0]), gate[0].numpy().astype(np.float32), r(beta[0]), lens, chunk,
                             init=None if init is None else init.numpy(), prims=dprims)


@pytest.mark.parametrize("chunk", [16, 64])
def test_cpr_forward_bit_exact_against_the_composed_oracle(chunk, dprims):
    from isoexec_amd.ops.gdn.gdn_cpr import chunk_boundary_states, gdn_cpr_fwd

    lens = [5, 1, 64, 33, 130, 16]
    q, k, v, gate, beta = make_inputs(lens, 21)
    bf = lambda t: t.to(torch.bfloat16).to(DEV)
    cu = torch.tensor(np.cumsum([0] + lens), dtype=torch.int32, device=DEV)
    want_o, want_h, want_final = oracle_cpr(q, k, v, gate, beta, lens, chunk, dprims)
    o = gdn_cpr_fwd(bf(q), bf(k), bf(v), gate.to(DEV), bf(beta), cu_seqlens=cu, chunk_size=chunk)
    assert o.shape == (1, sum(lens), HV, V)
    assert same_bits(o[0].cpu(), np_to_bf16(want_o))
    h, final, ci = chunk_boundary_states(None, bf(k), bf(v), gate.to(DEV), bf(beta), cu, chunk, output_final_state=True)
    assert h.dtype is torch.bfloat16 and h.shape == (1, len(want_h), HV, V, K)
    assert same_bits(h[0].cpu(), np_to_bf16(np.stack(want_h)))
    assert final.dtype is torch.float32 and np.array_equal(final.cpu().numpy().view(np.uint32),
                                                           np.stack(want_final).view(np.uint32))
    assert ci.tolist() == [[s, c] for s, n in enumerate(lens) for c in range(-(-n // chunk))]


def test_cpr_with_entry_states_and_an_empty_sequence(dprims):
    from isoexec_amd.ops.gdn.gdn_cpr import chunk_boundary_states

    lens = [40, 0, 7]
    q, k, v, gate, beta = make_inputs(lens, 22)
    init = torch.randn(3, HV, V, K, generator=cpu_gen(5))
    bf = lambda t: t.to(torch.bfloat16).to(DEV)
    cu = torch.tensor(np.cumsum([0] + lens), dtype=torch.int32, device=DEV)
    _, want_h, want_final = oracle_cpr(q, k, v, gate, beta, lens, 16, dprims, init=init)
    h, final, _ = chunk_boundary_states(None, bf(k), bf(v), gate.to(DEV), bf(beta), cu, 16,
                                        initial_state=init.to(DEV), output_final_state=True)
    assert same_bits(h[0].cpu(), np_to_bf16(np.stack(want_h)))
    assert np.array_equal(final.cpu().numpy().view(np.uint32), np.stack(want_final).view(np.uint32))
    assert torch.equal(final[1].cpu(), init[1])          # no tokens: the entry state passes through


def test_one_chunk_per_sequence_is_the_recurrent_forward():
    from isoexec_amd.ops.gdn.gdn_cpr import gdn_cpr_fwd
    from isoexec_amd.ops.gdn.gdn_ops import gdn_recurrent

    lens = [5, 64, 33]
    q, k, v, gate, beta = make_inputs(lens, 23)
    bf = lambda t: t.to(torch.bfloat16).to(DEV)
    cu = torch.tensor(np.cumsum([0] + lens), dtype=torch.int32, device=DEV)
    ref, _ = gdn_recurrent(bf(q), bf(k), bf(v), gate.to(DEV), bf(beta), cu_seqlens=cu)
    one = gdn_cpr_fwd(bf(q), bf(k), bf(v), gate.to(DEV), bf(beta), cu_seqlens=cu, chunk_size=64)
    assert same_bits(one, ref)
    # an fp32 wire dtype snapshots without rounding: every chunk size gives the recurrent forward's bits
    f = lambda t: t.float().to(DEV)
    ref32, _ = gdn_recurrent(f(q), f(k), f(v), gate.to(DEV), f(beta), cu_seqlens=cu)
    for chunk in (16, 32):
        got = gdn_cpr_fwd(f(q), f(k), f(v), gate.to(DEV), f(beta), cu_seqlens=cu, chunk_size=chunk)
        assert same_bits(got, ref32), chunk
    # with bf16 snapshots a smaller chunk is a different (rounded-boundary) function, close to the recurrent one
    small = gdn_cpr_fwd(bf(q), bf(k), bf(v), gate.to(DEV), bf(beta), cu_seqlens=cu, chunk_size=16)
    assert not same_bits(small, ref)
    assert (small.float() - ref.float()).abs().max() <= 2 ** -5


def test_native_cpr_equals_cpr_on_prepared_inputs():
    from isoexec_amd.ops.gdn.gdn_cpr import gdn_cpr_fwd, gdn_native_cpr_fwd
    from isoexec_amd.ops.gdn.gdn_ops import gdn_gate_and_beta, gdn_l2norm

    lens = [20, 70]
    g = cpu_gen(24)
    T = sum(lens)
    bf = lambda t: t.to(torch.bfloat16).to(DEV)
    q, k = bf(torch.randn(1, T, H, K, generator=g)), bf(torch.randn(1, T, H, K, generator=g))
    v = bf(torch.randn(1, T, HV, V, generator=g))
    a, b = bf(torch.randn(T, HV, generator=g)), bf(torch.randn(T, HV, generator=g))
    A_log, dt_bias = (torch.randn(HV, generator=g) * 0.3).to(DEV), (torch.randn(HV, generator=g) * 0.3).to(DEV)
    cu = torch.tensor(np.cumsum([0] + lens), dtype=torch.int32, device=DEV)
    got = gdn_native_cpr_fwd(q, k, v, a, b, A_log, dt_bias, cu_seqlens=cu, chunk_size=32)
    gate, beta = gdn_gate_and_beta(a, b, A_log, dt_bias)
    want = gdn_cpr_fwd(gdn_l2norm(q), gdn_l2norm(k), v, gate.view(1, T, HV), beta.view(1, T, HV), cu_seqlens=cu,
                       chunk_size=32)
    assert same_bits(got, want)


def test_trainer_door_follows_the_kernel_selector(monkeypatch):
    from isoexec_amd.ops.gdn.gdn_cpr import gdn_cpr_fwd
    from isoexec_amd.ops.gdn.gdn_ops import gdn_core, gdn_recurrent

    lens = [100, 30]
    q, k, v, gate, beta = make_inputs(lens, 25)
    bf = lambda t: t.to(torch.bfloat16).to(DEV)
    cu = torch.tensor(np.cumsum([0] + lens), dtype=torch.int32, device=DEV)
    args = (bf(q), bf(k), bf(v), gate.to(DEV), bf(beta))
    monkeypatch.delenv("SKYRL_ISOEXEC_GDN_KERNEL", raising=False)
    assert same_bits(gdn_core(*args, cu_seqlens=cu)[0], gdn_recurrent(*args, cu_seqlens=cu)[0])
    monkeypatch.setenv("SKYRL_ISOEXEC_GDN_KERNEL", "cpr")
    assert same_bits(gdn_core(*args, cu_seqlens=cu)[0], gdn_cpr_fwd(*args, cu_seqlens=cu, chunk_size=64))
    # a padded batch is B packed sequences
    B, T = 2, 80
    qp, kp, vp, gp, bp = make_inputs([B * T], 26)
    pad = lambda t: t.reshape(B, T, *t.shape[2:])
    o_pad, _ = gdn_core(bf(pad(qp)), bf(pad(kp)), bf(pad(vp)), pad(gp).to(DEV), bf(pad(bp)))
    cu2 = torch.tensor([0, T, 2 * T], dtype=torch.int32, device=DEV)
    o_pk = gdn_cpr_fwd(bf(qp), bf(kp), bf(vp), gp.to(DEV), bf(bp), cu_seqlens=cu2, chunk_size=64)
    assert same_bits(o_pad.reshape(1, B * T, HV, V), o_pk)
    monkeypatch.setenv("SKYRL_ISOEXEC_GDN_KERNEL", "chunk")
    with pytest.raises(NotImplementedError, match="not served"):
        gdn_core(*args, cu_seqlens=cu)
