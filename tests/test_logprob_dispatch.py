"""The single dispatch point of the logprob path and what it owes when the kernel cannot serve.

The cases are the ones the reference pins for its dispatch (isoexec/ops/logprobs/tests/
test_rowinv_dispatch_cpu.py:99-260): a switched-off kernel is byte for byte the incumbent, both grad
modes consult the kernel, gradients flow through a served call, the chunk walk changes no bit, a
decline anywhere abandons the kernel for the whole call, and exactly one function calls the kernel.
A differentiable row-wise stand-in replaces the kernel, so everything here runs on the host.
"""

import ast
import inspect

import pytest
import torch

from isoexec_amd.runtimes import logprob_callers as M

B, S, V = 2, 13, 32


def data(requires_grad=False):
    g = torch.Generator().manual_seed(3)
    logits = torch.randn(B, S, V, generator=g).to(torch.bfloat16)
    logits.requires_grad_(requires_grad)
    return logits, torch.randint(0, V, (B, S), generator=g)


def bits(t):
    return t.contiguous().view(torch.int32 if t.dtype is torch.float32 else torch.int16)


def rowwise_standin(chunk, target):
    """Row-independent sampled logprob: elementwise ops and a fixed-order column loop."""
    x = chunk.float()
    m = x.max(dim=-1).values
    e = torch.exp(x - m.unsqueeze(-1))
    s = torch.zeros_like(m)
    for j in range(e.shape[-1]):
        s = s + e[..., j]
    return (x.gather(-1, target.unsqueeze(-1)).squeeze(-1) - m) - torch.log(s)


def fake_kernel(monkeypatch, fn, stats=None):
    monkeypatch.setattr(M, "_ix_rowinv_available", lambda: True)
    monkeypatch.setattr(M, "_ix_rowinv_sampled_logprobs", fn)
    monkeypatch.setattr(M, "_ix_rowinv_stats", lambda: stats or {})


def apply(logits, target, inference_only=False, chunk_size=None):
    return M._ix_logprobs_apply(logits, target, 0, V, None, inference_only, chunk_size)


@pytest.mark.parametrize("inference_only", [True, False])
@pytest.mark.parametrize("chunk_size", [None, 5])
def test_switched_off_kernel_is_byte_for_byte_the_incumbent(monkeypatch, inference_only, chunk_size):
    monkeypatch.setattr(M, "_ix_rowinv_available", lambda: False)

    def never(*a, **k):
        raise AssertionError("the kernel must not be consulted")

    monkeypatch.setattr(M, "_ix_rowinv_sampled_logprobs", never)
    logits, target = data()
    got = apply(logits, target, inference_only, chunk_size)
    want = M.incumbent_logprobs(logits, target, 0, V)
    assert torch.equal(bits(got), bits(want)) and got.dtype is torch.float32 and got.is_contiguous()
    torch.testing.assert_close(got, torch.log_softmax(logits.float(), -1).gather(-1, target[..., None])[..., 0], rtol=0, atol=2e-6)


def test_missing_library_raises_instead_of_declining(monkeypatch):
    from isoexec_amd import _lib

    def gone():
        raise _lib.IsoExecLibraryError("libisoexec_hip.so not found")

    monkeypatch.setattr(_lib, "lib", gone)
    with pytest.raises(_lib.IsoExecLibraryError):
        apply(*data())


def test_both_grad_modes_consult_the_kernel(monkeypatch):
    seen = []

    def kernel(chunk, target, **kw):
        seen.append((torch.is_grad_enabled(), kw["src_dtype"], kw["group"], kw["vocab_end_index"], callable(kw["reference"])))
        return rowwise_standin(chunk, target)

    fake_kernel(monkeypatch, kernel)
    logits, target = data(requires_grad=True)
    apply(logits, target, inference_only=False)
    apply(logits, target, inference_only=True)
    with torch.no_grad():
        apply(logits, target, inference_only=False)
    assert [s[0] for s in seen] == [True, False, False]
    assert all(s[1:] == (torch.bfloat16, None, V, True) for s in seen)


def test_grad_flows_through_a_served_call(monkeypatch):
    fake_kernel(monkeypatch, lambda c, t, **kw: rowwise_standin(c, t))
    logits, target = data(requires_grad=True)
    out = apply(logits, target, chunk_size=4)
    out.sum().backward()
    want = -torch.softmax(logits.detach().float(), -1)
    want.scatter_add_(-1, target.unsqueeze(-1), torch.ones(B, S, 1))
    torch.testing.assert_close(logits.grad.float(), want, rtol=0, atol=1e-2)
    served_no_grad = apply(logits, target, inference_only=True)
    assert not served_no_grad.requires_grad


@pytest.mark.parametrize("chunk_size", [1, 4, 5, 12, 13, 50])
def test_chunk_walk_changes_no_bit(monkeypatch, chunk_size):
    shapes = []

    def kernel(chunk, target, **kw):
        assert chunk.is_contiguous()
        shapes.append(chunk.shape[1])
        return rowwise_standin(chunk, target)

    fake_kernel(monkeypatch, kernel)
    logits, target = data()
    whole = apply(logits, target)
    shapes.clear()
    walked = apply(logits, target, chunk_size=chunk_size)
    assert torch.equal(bits(walked), bits(whole))
    expect = [S] if chunk_size >= S else [chunk_size] * (S // chunk_size) + ([S % chunk_size] if S % chunk_size else [])
    assert shapes == expect


def test_a_decline_mid_walk_abandons_the_kernel_for_the_whole_call(monkeypatch):
    calls = []

    def kernel(chunk, target, **kw):
        calls.append(1)
        return None if len(calls) == 2 else rowwise_standin(chunk, target) + 100.0

    fake_kernel(monkeypatch, kernel)
    logits, target = data()
    got = apply(logits, target, chunk_size=5)
    assert len(calls) == 2  # the walk stops at the decline
    assert torch.equal(bits(got), bits(M.incumbent_logprobs(logits, target, 0, V)))  # no +100 anywhere


def test_a_graph_free_chunk_under_grad_falls_back_whole(monkeypatch):
    fake_kernel(monkeypatch, lambda c, t, **kw: rowwise_standin(c, t).detach() + 100.0)
    logits, target = data(requires_grad=True)
    got = apply(logits, target, chunk_size=5)
    assert got.requires_grad and float(got.max()) < 50
    assert float(apply(logits, target, inference_only=True).min()) > 50  # without grad the same result is fine


def test_a_probe_latch_seen_after_the_walk_falls_back_whole(monkeypatch):
    fake_kernel(monkeypatch, lambda c, t, **kw: rowwise_standin(c, t) + 100.0, stats={"agreed": False})
    logits, target = data()
    assert float(apply(logits, target, chunk_size=5).max()) < 50


def test_the_reference_closure_is_the_incumbent_for_that_chunk(monkeypatch):
    got = []

    def kernel(chunk, target, **kw):
        got.append((kw["reference"](), M.incumbent_logprobs(chunk, target, 0, V)))
        return rowwise_standin(chunk, target)

    fake_kernel(monkeypatch, kernel)
    apply(*data(requires_grad=True), chunk_size=6)
    assert len(got) == 3 and all(torch.equal(bits(a), bits(b.detach())) and not a.requires_grad for a, b in got)


def test_next_token_wrapper_shifts_targets(monkeypatch):
    fake_kernel(monkeypatch, lambda c, t, **kw: rowwise_standin(c, t))
    logits, tokens = data()
    got = M.from_parallel_logits_to_logprobs(logits, tokens, inference_only=True, chunk_size=4)
    want = rowwise_standin(logits[:, :-1], tokens[:, 1:])
    assert got.shape == (B, S - 1) and torch.equal(bits(got), bits(want))


def test_exactly_one_function_calls_each_kernel_entry():
    tree = ast.parse(inspect.getsource(M))
    callers = {"_ix_rowinv_sampled_logprobs": set(), "_ix_try_rowinv_logprobs": set(), "_ix_rowinv_full_logprobs": set()}
    for fn in ast.walk(tree):
        if isinstance(fn, ast.FunctionDef):
            for node in ast.walk(fn):
                if isinstance(node, ast.Call) and isinstance(node.func, ast.Name) and node.func.id in callers and fn.name != node.func.id:
                    callers[node.func.id].add(fn.name)
    assert callers["_ix_rowinv_sampled_logprobs"] == {"_ix_try_rowinv_logprobs"}
    assert callers["_ix_try_rowinv_logprobs"] == {"_ix_logprobs_apply"}
    assert callers["_ix_rowinv_full_logprobs"] <= {"make_engine_compute_logprobs", "_isoexec_compute_logprobs"}


def test_engine_hook_serves_or_hands_back_whole(monkeypatch):
    logits = data()[0][0]
    monkeypatch.setattr(M, "_ix_rowinv_full_logprobs", lambda x, **kw: torch.full(x.shape, 7.0))
    before = M.engine_logprob_census()
    hook = M.make_engine_compute_logprobs(lambda x: torch.full(x.shape, 3.0))
    assert M.make_engine_compute_logprobs(hook) is hook
    assert float(hook(logits).mean()) == 7.0
    monkeypatch.setattr(M, "_ix_rowinv_full_logprobs", lambda x, **kw: None)
    assert float(hook(logits).mean()) == 3.0
    after = M.engine_logprob_census()
    assert (after["calls"] - before["calls"], after["rowinv_owned"] - before["rowinv_owned"], after["incumbent"] - before["incumbent"]) == (2, 1, 1)
    default = M.make_engine_compute_logprobs()
    torch.testing.assert_close(default(logits), torch.log_softmax(logits.float(), -1), rtol=0, atol=2e-6)
