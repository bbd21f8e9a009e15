"""GPU: the grouped expert kernels pinned bit for bit, and the MoE doors with the reference's call shapes.

The grouped GEMMs share the dense kernel's core (one instruction, one K order), so each expert's rows must equal, bit
for bit, what the dense entry point gives for the same rows: fc1 = ``linear_nt(x[rows_e], W1[e])`` followed by the
oracle's SwiGLU * prob epilogue (device transcendentals plugged in), fc2 = ``linear_nt(inter_e, W2[e])``
(reference chain: ops/moe/moe_batched_experts.py:496-503; its invariance gate :652-708)."""

from types import SimpleNamespace

import numpy as np
import pytest
import torch

from _util import DevicePrims, bf16_to_np, cpu_gen, np_to_bf16, same_bits
from oracle.prims import round_bf16

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F32 = np.float32


def make(T, H, E, F, seed):
    g = cpu_gen(seed)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(DEV)
    wr = (0.02 * torch.randn(E, H, generator=g)).to(torch.bfloat16).to(DEV)
    w1 = (0.02 * torch.randn(E, 2 * F, H, generator=g)).to(torch.bfloat16).to(DEV)
    w2 = (0.02 * torch.randn(E, H, F, generator=g)).to(torch.bfloat16).to(DEV)
    return x, wr, w1, w2


@pytest.mark.parametrize("T,H,E,F,k,BM", [(300, 256, 16, 128, 4, None), (300, 256, 16, 96, 4, 256), (77, 512, 8, 192, 2, 128),
                                          (33, 2048, 128, 768, 8, None), (600, 2048, 8, 768, 2, 256),
                                          # enough tiles for the streaming form of the grouped kernels (one workgroup walks
                                          # many tiles): the smallest K it takes with ragged experts, and the full MoE shape
                                          (9000, 1024, 8, 704, 4, 256), (9000, 1024, 8, 768, 4, 256), (7000, 960, 8, 640, 4, 256),
                                          (16384, 2048, 128, 768, 8, None)])
def test_grouped_kernels_equal_the_dense_kernel_per_expert(T, H, E, F, k, BM):
    from isoexec_amd.ops.mm.mm_hip import linear_nt, router_gemm
    from isoexec_amd.ops.moe.moe_hip import experts_forward, permute, router_topk

    prims = DevicePrims(DEV)
    x, wr, w1, w2 = make(T, H, E, F, seed=T + F)
    logits = router_gemm(x, wr)
    logits[:, :2] += 2.0          # skewed load: some experts get ragged multi-tile segments, some get nothing
    idx, prob, _, _ = router_topk(logits, k, pre_softmax=True)
    p = permute(idx, prob, E, BM=BM)
    eo, inter = experts_forward(x, w1, w2, p, return_inter=True)
    offsets = p.offsets.cpu().numpy()
    st = p.sorted_token.long()
    pp = p.permuted_prob.cpu().numpy()
    checked = 0
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi == lo:
            continue
        xe = x.index_select(0, st[lo:hi])
        lin = bf16_to_np(linear_nt(xe, w1[e]))                      # bf16(x W1^T): gate columns then up columns
        gate, up = lin[:, :F], lin[:, F:]
        s = round_bf16(prims.silu_div(gate))
        h = round_bf16((s * up).astype(F32))
        a = round_bf16((h * pp[lo:hi, None]).astype(F32))
        assert same_bits(inter[lo:hi].cpu(), np_to_bf16(a)), f"fc1 epilogue, expert {e} rows {lo}:{hi}"
        assert same_bits(eo[lo:hi], linear_nt(inter[lo:hi].contiguous(), w2[e])), f"fc2, expert {e}"
        checked += hi - lo
    assert checked == T * k


def test_streamed_experts_with_a_pitched_activation_matrix():
    """The streaming kernels gather token rows through the caller's row pitch: a column slice of a wider matrix gives
    the bits of its contiguous copy (sizes that take the streaming form of both grouped GEMMs)."""
    from isoexec_amd.ops.mm.mm_hip import router_gemm
    from isoexec_amd.ops.moe.moe_hip import experts_forward, permute, router_topk

    T, H, E, F, k = 9000, 1024, 8, 768, 4
    x, wr, w1, w2 = make(T, H, E, F, seed=5)
    wide = torch.zeros(T, H + 192, dtype=torch.bfloat16, device=DEV)
    wide[:, 64:64 + H] = x
    xs = wide[:, 64:64 + H]
    assert xs.stride(0) == H + 192 and xs.data_ptr() % 16 == 0
    idx, prob, _, _ = router_topk(router_gemm(x, wr), k, pre_softmax=True)
    p = permute(idx, prob, E, BM=256)
    eo, inter = experts_forward(x, w1, w2, p, return_inter=True)
    eo2, inter2 = experts_forward(xs, w1, w2, p, return_inter=True)
    assert same_bits(inter, inter2) and same_bits(eo, eo2)


def fake_sequential_mlp(w1, w2, stacked=True):
    """What ``_batched_experts_forward`` reads of a ``SequentialMLP`` (the reference's own stand-in,
    ops/moe/tests/moe_fused_vs_bmm_gpu.py:26-44)."""
    cfg = SimpleNamespace(activation_func=torch.nn.functional.silu, activation_func_clamp_value=None, glu_linear_offset=0.0,
                          fp8=False, bias_activation_fusion=False, gated_linear_unit=True, add_bias_linear=False)
    pick = (lambda w, e: w[e]) if stacked else (lambda w, e: w[e].clone())
    experts = [SimpleNamespace(linear_fc1=SimpleNamespace(weight=pick(w1, e)), linear_fc2=SimpleNamespace(weight=pick(w2, e)))
               for e in range(w1.shape[0])]
    return SimpleNamespace(config=cfg, num_local_experts=w1.shape[0], local_experts=experts)


@pytest.mark.parametrize("stacked", [True, False])
def test_doors_with_the_reference_call_shapes(stacked):
    from isoexec_amd.ops.mm.mm_hip import router_gemm
    from isoexec_amd.ops.moe import moe_doors
    from isoexec_amd.ops.moe.moe_hip import combine, experts_forward, fused_router_dense, permute, router_topk

    T, H, E, F, k = 300, 256, 16, 128, 4
    x, wr, w1, w2 = make(T, H, E, F, seed=9)
    logits = router_gemm(x, wr)
    # TopKRouter.routing(logits) -> (routing_probs, routing_map)
    router = SimpleNamespace(topk=k, config=SimpleNamespace(moe_router_pre_softmax=False, moe_router_topk_scaling_factor=None))
    rprobs, rmap = moe_doors._make_sorted_topk_routing(None)(router, logits)
    dprobs, dmap = fused_router_dense(logits, k)
    assert same_bits(rprobs, dprobs) and torch.equal(rmap, dmap) and int(rmap.sum()) == T * k
    # dispatcher: dispatch_postprocess(hidden, probs) -> (permuted hidden, tokens_per_expert, permuted probs)
    disp = SimpleNamespace(routing_map=rmap, local_expert_indices=list(range(E)), config=SimpleNamespace(moe_router_topk=k))
    hidden, tpe, pprobs = moe_doors._dispatch_postprocess_fixed_shape(disp, x, rprobs)
    idx, prob, _, _ = router_topk(logits, k)
    p = permute(idx, prob, E)
    assert torch.equal(disp.reversed_local_input_permutation_mapping, p.sorted_token.long())
    assert torch.equal(tpe, p.counts.long()) and same_bits(pprobs, p.permuted_prob)
    assert same_bits(hidden, x.index_select(0, p.sorted_token.long()))
    # SequentialMLP.forward(permuted hidden, tokens_per_expert, permuted probs) -> (out, None)
    mlp = fake_sequential_mlp(w1, w2, stacked)
    out, bias = moe_doors._batched_experts_forward(mlp, hidden, tpe, pprobs)
    assert bias is None and same_bits(out, experts_forward(x, w1, w2, p))
    out_host_counts, _ = moe_doors._batched_experts_forward(mlp, hidden, tpe.cpu().to(torch.int32), pprobs)
    assert same_bits(out_host_counts, out)
    empty, _ = moe_doors._batched_experts_forward(mlp, hidden[:0], torch.zeros(E, dtype=torch.int64), pprobs[:0])
    assert empty.shape == (0, H)
    # moe_utils.unpermute(permuted_tokens, sorted_indices, restore_shape)
    got = moe_doors._deterministic_unpermute(out, disp.reversed_local_input_permutation_mapping, x.shape)
    assert same_bits(got, combine(out, p))
    assert moe_doors._deterministic_unpermute(out, disp.reversed_local_input_permutation_mapping, x.shape,
                                              isoexec_out_dtype=torch.float32).dtype is torch.float32
    assert moe_doors._fixed_order_combine(out[:-1], disp.reversed_local_input_permutation_mapping[:-1], x.shape) is None
    with pytest.raises(RuntimeError):
        moe_doors._deterministic_unpermute(out, disp.reversed_local_input_permutation_mapping, x.shape, fused=True)
    # a SequentialMLP the kernels do not serve says so
    mlp.config.add_bias_linear = True
    with pytest.raises(RuntimeError):
        moe_doors._batched_experts_forward(mlp, hidden, tpe, pprobs)


def test_unpermute_with_probs_and_layout_validation():
    """``moe_utils.unpermute(..., probs=, routing_map=)`` (moe_batch_invariant.py:366-385): bf16 rows times fp32 probs is
    an fp32 product, summed per token in ascending expert order in fp32, then cast. Expected values by the same eager
    torch expressions (elementwise IEEE products and sums: no reduction order of torch's own is involved)."""
    from isoexec_amd.ops.mm.mm_hip import router_gemm
    from isoexec_amd.ops.moe import moe_doors
    from isoexec_amd.ops.moe.moe_hip import fused_router_dense

    T, H, E, F, k = 70, 200, 16, 64, 4              # H not a multiple of 8: the element-wise load path too
    x, wr, w1, w2 = make(T, 256, E, F, seed=12)
    rprobs, rmap = fused_router_dense(router_gemm(x, wr), k)
    disp = SimpleNamespace(routing_map=rmap, local_expert_indices=list(range(E)), config=SimpleNamespace(moe_router_topk=k))
    _, _, _ = moe_doors._dispatch_postprocess_fixed_shape(disp, x, rprobs)
    sorted_indices = disp.reversed_local_input_permutation_mapping
    g = cpu_gen(13)
    moe_doors.reset_combine_validation()

    def eager(tokens, probs, out_dtype):
        pt = tokens
        if probs is not None:
            pp = probs.T.contiguous().masked_select(rmap.T.contiguous())
            pt = tokens * pp.unsqueeze(-1)
        rows = torch.argsort(sorted_indices, stable=True).view(T, k)
        acc = pt.index_select(0, rows[:, 0].contiguous())
        for j in range(1, k):
            acc = acc + pt.index_select(0, rows[:, j].contiguous())
        return acc.to(out_dtype)

    for width in (H, 256):
        tok16 = torch.randn(T * k, width, generator=g).to(torch.bfloat16).to(DEV)
        for tokens, probs, out_dtype in ((tok16, rprobs, None), (tok16, rprobs, torch.float32),
                                         (tok16, rprobs.to(torch.bfloat16), None), (tok16.float(), None, None),
                                         (tok16.float(), rprobs, torch.bfloat16), (tok16, None, None)):
            got = moe_doors._deterministic_unpermute(tokens, sorted_indices, (T, width), probs=probs,
                                                     routing_map=None if probs is None else rmap,
                                                     isoexec_out_dtype=out_dtype)
            want = eager(tokens, probs, tokens.dtype if out_dtype is None else out_dtype)
            assert got.dtype is want.dtype and same_bits(got, want), (width, tokens.dtype, probs is None, out_dtype)
    # a layout where the row count is a multiple of the token count but a token owns the wrong number of rows
    # (token dropping / padding) is refused on the first calls instead of summing the wrong rows
    moe_doors.reset_combine_validation()
    uneven = sorted_indices.clone()
    uneven[uneven == 3] = 4
    with pytest.raises(RuntimeError, match="do not each route to exactly topk"):
        moe_doors._deterministic_unpermute(tok16, uneven, (T, 256))
    with pytest.raises(RuntimeError, match="not a multiple"):
        moe_doors._deterministic_unpermute(tok16[:-1], sorted_indices[:-1], (T, 256))
    with pytest.raises(RuntimeError, match="not served"):
        moe_doors._deterministic_unpermute(tok16.half(), sorted_indices, (T, 256), probs=rprobs, routing_map=rmap)
    moe_doors.reset_combine_validation()


def test_block_map_keeps_every_tile_inside_the_row_buffers():
    """Per-expert counts live on the device; counts that add up to more rows than the buffers hold lose their tail,
    counts that add up to fewer leave the last rows in no tile; the experts' door refuses both on its first calls."""
    from isoexec_amd import _lib
    from isoexec_amd.ops.moe import moe_doors

    L = _lib.lib()
    E, BM, R = 6, 32, 100
    max_tiles = int(L.ix_moe_max_tiles(R, 1, E, BM))

    def block_map(counts, dtype):
        c = torch.tensor(counts, dtype=dtype, device=DEV)
        meta = torch.full((1 + 3 * max_tiles,), -7, dtype=torch.int32, device=DEV)
        off = torch.full((E + 1,), -7, dtype=torch.int32, device=DEV)
        assert L.ix_moe_block_map(c.data_ptr(), int(dtype is torch.int64), E, BM, R, off.data_ptr(), meta.data_ptr(),
                                  max_tiles, _lib.current_stream(torch.device(DEV))) == 0
        m = meta.cpu().tolist()
        n = m[0]
        tiles = [(m[1 + i], m[1 + max_tiles + i], m[1 + 2 * max_tiles + i]) for i in range(n)]
        return tiles, off.cpu().tolist()

    def expected(counts):
        tiles, off, row = [], [], 0
        for e, c in enumerate(counts):
            c = max(0, min(c, R - row))
            off.append(row)
            tiles += [(e, row + r0, min(BM, c - r0)) for r0 in range(0, c, BM)]
            row += c
        return tiles, off + [row]

    for counts in ([10, 0, 33, 7, 50, 0], [10, 0, 33, 7, 80, 5], [70, 70, 1, 0, 0, 9], [2 ** 31 - 1] * 6, [0] * 6,
                   [10, -4, 20, 0, 0, 3], [5, 5, 5, 5, 5, 5]):
        for dtype in (torch.int32, torch.int64):
            tiles, off = block_map(counts, dtype)
            assert (tiles, off) == expected(counts), counts
            assert all(0 <= r0 and n > 0 and r0 + n <= R for _, r0, n in tiles)
    tiles, _ = block_map([2 ** 40, 1, 1, 1, 1, 1], torch.int64)             # a count beyond 32 bits is still only "too many"
    assert tiles == [(0, 0, 32), (0, 32, 32), (0, 64, 32), (0, 96, 4)]
    # the door: a batch whose counts do not add up to its rows is refused while the first calls are being checked
    T, H, F = 72, 256, 128
    hidden, _, w1, w2 = make(T, H, E, F, seed=14)
    mlp = fake_sequential_mlp(w1, w2)
    pprobs = torch.ones(hidden.shape[0], device=DEV)
    moe_doors.reset_combine_validation()
    good = torch.tensor([12] * 6, device=DEV)
    out, _ = moe_doors._batched_experts_forward(mlp, hidden, good, pprobs)
    assert out.shape == hidden.shape
    for bad in ([12, 12, 12, 12, 12, 40], [12, 12, 12, 12, 12, 2]):
        with pytest.raises(RuntimeError, match="adding up to"):
            moe_doors._batched_experts_forward(mlp, hidden, torch.tensor(bad, device=DEV), pprobs)
    moe_doors.reset_combine_validation()


def test_operator_override_door():
    """aten::mm / addmm / bmm on the device key land on the fixed-order kernels: F.linear, torch.mm, torch.addmm,
    torch.bmm, 2-D and 3-D, with and without bias, forward and backward; what the kernels do not serve goes to the
    stock kernel and is counted; uninstalling brings the stock kernels back."""
    import torch.nn.functional as Fn

    from isoexec_amd.ops.mm import mm_hip

    g = cpu_gen(21)
    x = torch.randn(37, 256, generator=g).to(torch.bfloat16).to(DEV)
    w = (0.05 * torch.randn(96, 256, generator=g)).to(torch.bfloat16).to(DEV)
    b = torch.randn(96, generator=g).to(torch.bfloat16).to(DEV)
    want = mm_hip.linear_nt(x, w)
    want_b = mm_hip.linear_nt(x, w, b)
    stock = Fn.linear(x, w)
    mm_hip.reset_stats()
    assert mm_hip.install_mm_override(strict=False) and mm_hip.mm_override_installed()
    try:
        assert same_bits(Fn.linear(x, w), want) and mm_hip.stats()["mm"] == 1
        assert same_bits(torch.mm(x, w.t()), want) and same_bits(x @ w.t(), want) and mm_hip.stats()["mm"] == 3
        assert same_bits(Fn.linear(x, w, b), want_b) and same_bits(torch.addmm(b, x, w.t()), want_b)
        assert mm_hip.stats()["addmm"] == 2
        x3 = x.view(1, 37, 256).expand(3, 37, 256).contiguous()
        assert same_bits(Fn.linear(x3, w), want.expand(3, 37, 96))           # 3-D input folds into one mm
        w3 = torch.stack([w, w.roll(1, 0), w.flip(0)])
        got = torch.bmm(x3, w3.transpose(1, 2))
        assert mm_hip.stats()["bmm"] == 1
        for i in range(3):
            assert same_bits(got[i], mm_hip.linear_nt(x, w3[i]))              # bmm == mm, product by product
        assert mm_hip.stats()["operand_copies"] == 0                          # nothing above needed a copy
        # row m does not depend on how many rows share the call (the point of the override)
        assert same_bits(Fn.linear(x[5:6], w), want[5:6]) and same_bits(Fn.linear(x[:20], w), want[:20])
        # backward through the override: grad products are mm calls too (their row-major operands are copied)
        xg, wg = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
        Fn.linear(xg, wg).float().square().sum().backward()
        assert xg.grad.shape == x.shape and wg.grad.shape == w.shape and bool(torch.isfinite(wg.grad.float()).all())
        ref_gx = (2 * want.float()).to(torch.bfloat16).float() @ w.float()
        assert float((xg.grad.float() - ref_gx).abs().max()) <= 0.05 * float(ref_gx.abs().max())
        assert mm_hip.stats()["operand_copies"] >= 1
        # not served: fp16, and a K that is not a multiple of 8 -> the stock kernel, counted, same answer as stock
        before = mm_hip.stats()["declined"]
        h = torch.randn(4, 24, generator=g).to(DEV).half()
        assert torch.equal(h @ h.t(), torch.mm(h, h.t())) and mm_hip.stats()["declined"] == before + 2
        odd = torch.randn(5, 20, generator=g).to(torch.bfloat16).to(DEV)
        assert (odd @ odd.t()).shape == (5, 5) and mm_hip.stats()["declined"] == before + 3
        # fp32 products take the fp32 kernel (the router's gating product)
        f = torch.randn(9, 64, generator=g).to(DEV)
        served = mm_hip.stats()["mm"]
        assert same_bits(f @ f.t(), mm_hip.linear_f32_nt(f, f)) and mm_hip.stats()["mm"] == served + 1
        # what fell through can be turned into a refusal after the fact
        mm_hip.assert_none_declined(since=mm_hip.stats()["declined"])
        with pytest.raises(RuntimeError, match="stock kernel"):
            mm_hip.assert_none_declined(since=before)
        # strict mode (the default) refuses instead of falling through
        mm_hip.install_mm_override()
        with pytest.raises(RuntimeError):
            h @ h.t()
        mm_hip.install_mm_override(strict=False)
    finally:
        mm_hip.uninstall_mm_override()
    assert not mm_hip.mm_override_installed()
    served = dict(mm_hip.stats())
    assert same_bits(Fn.linear(x, w), stock) and mm_hip.stats() == served          # the stock kernel is back


@pytest.mark.parametrize("T,H,E,F,k", [(64, 2048, 128, 768, 8), (1, 2048, 128, 768, 8), (33, 512, 16, 1024, 4), (256, 1024, 8, 512, 2),
                                       (200, 768, 4, 1536, 2)])
def test_decode_kernels_read_fragment_packed_matrices_with_the_same_bits(T, H, E, F, k):
    """``pack_decode`` + ``ix_moe_experts_decode`` (weights streamed through registers from fragment-packed copies) against
    the 32-row ring tile reading the matrices in place: the packed copies hold exactly the values of the layout formula
    (checked on the host), and both grouped GEMMs give the same bits from them -- ragged tiles, tiles of 32 full rows,
    dead token lanes."""
    from isoexec_amd.ops.mm.mm_hip import router_gemm
    from isoexec_amd.ops.moe.moe_hip import experts_forward, pack_decode, permute, router_topk

    x, wr, w1, w2 = make(T, H, E, F, seed=50 + T)
    packed = pack_decode(w1, w2)
    assert packed is not None
    w1f, w2f = packed
    assert w1f.shape == w1.shape and w2f.shape == w2.shape
    # W1f [E][F/128][wave 4][H/64][b 2][s 4][g 2][r 32][8]: row b F + 128 nt + 32 wave + r, k = 64 kt + 32 g + 8 s + c
    got1 = w1f.view(E, F // 128, 4, H // 64, 2, 4, 2, 32, 8)                  # [e, nt, w, kt, b, s, g, r, c]
    src1 = w1.view(E, 2, F // 128, 4, 32, H // 64, 2, 4, 8)                    # [e, b, nt, w, r, kt, g, s, c]
    assert torch.equal(got1, src1.permute(0, 2, 3, 5, 1, 7, 6, 4, 8))
    # W2f [E][H/256][wave 4][F/64][b 2][s 4][g 2][r 32][8]: row 256 nt + 64 wave + 32 b + r
    got2 = w2f.view(E, H // 256, 4, F // 64, 2, 4, 2, 32, 8)                  # [e, nt, w, kt, b, s, g, r, c]
    src2 = w2.view(E, H // 256, 4, 2, 32, F // 64, 2, 4, 8)                    # [e, nt, w, b, r, kt, g, s, c]
    assert torch.equal(got2, src2.permute(0, 1, 2, 5, 3, 7, 6, 4, 8))
    idx, prob, _, _ = router_topk(router_gemm(x, wr), k, pre_softmax=True)
    p = permute(idx, prob, E, BM=32)
    want, want_inter = experts_forward(x, w1, w2, p, return_inter=True)
    got, got_inter = experts_forward(x, w1, w2, p, return_inter=True, packed=packed)
    assert same_bits(got_inter, want_inter) and same_bits(got, want)
    # a larger tile ignores the packed copies
    p256 = permute(idx, prob, E, BM=256)
    assert same_bits(experts_forward(x, w1, w2, p256, packed=packed), experts_forward(x, w1, w2, p256))
    assert pack_decode(w1[:, :, : H - 64].contiguous(), w2[:, : H - 64].contiguous()) is None   # H not a multiple of 256
