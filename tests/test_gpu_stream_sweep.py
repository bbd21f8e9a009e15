"""GPU: a seeded sweep of shapes through the streaming kernels (one workgroup walking many tiles) against the kernels
that take one tile per workgroup. The tile shape and the launch form choose who computes an element, never how, so
every case must agree bit for bit -- ragged row counts, K from the smallest the streaming form takes upwards, column
counts that leave a partial last tile, experts with no rows, expert widths on both sides of the second GEMM's threshold.
"""
import random

import pytest
import torch

from _util import same_bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def dense_cases(seed, n):
    rnd = random.Random(seed)
    out = []
    for _ in range(n):
        K = 64 * rnd.randint(11, 40)
        M = rnd.choice([256 * rnd.randint(1, 40) + rnd.choice([0, 0, 1, 17, 255]), rnd.randint(1, 5000)])
        N = 8 * rnd.randint(1, 600)
        out.append((M, K, N))
    return out


def moe_cases(seed, n):
    rnd = random.Random(seed)
    out = []
    for _ in range(n):
        H = 64 * rnd.randint(15, 34)
        F = 128 * rnd.choice([rnd.randint(1, 7), rnd.randint(6, 9)])
        E = rnd.choice([4, 8, 16, 60, 128])
        k = min(rnd.choice([1, 2, 4, 8]), E)
        T = rnd.randint(3000, 24000)
        out.append((T, H, E, F, k, rnd.choice([0.0, 1.0, 3.0])))
    return out


@pytest.mark.parametrize("M,K,N", dense_cases(7, 14))
def test_dense_streaming_tile_against_one_tile_per_workgroup(M, K, N):
    from isoexec_amd.ops.mm.mm_hip import linear_nt

    g = torch.Generator(device=DEV).manual_seed(M + K + N)
    a = torch.randn(M, K, device=DEV, generator=g).to(torch.bfloat16)
    w = (0.05 * torch.randn(N, K, device=DEV, generator=g)).to(torch.bfloat16)
    streamed = linear_nt(a, w, tile=8, want_row_max=True)
    single = linear_nt(a, w, tile=7, want_row_max=True)
    assert streamed is not None and single is not None
    assert same_bits(streamed[0], single[0]) and torch.equal(streamed[1], single[1])


@pytest.mark.parametrize("T,H,E,F,k,skew", moe_cases(11, 10))
def test_experts_256_row_tiles_against_128_row_tiles(T, H, E, F, k, skew):
    from isoexec_amd.ops.mm.mm_hip import router_gemm
    from isoexec_amd.ops.moe.moe_hip import experts_forward, permute, router_topk

    g = torch.Generator(device=DEV).manual_seed(T + H + F)
    x = torch.randn(T, H, device=DEV, generator=g).to(torch.bfloat16)
    wr = (0.05 * torch.randn(E, H, device=DEV, generator=g)).to(torch.bfloat16)
    w1 = (0.03 * torch.randn(E, 2 * F, H, device=DEV, generator=g)).to(torch.bfloat16)
    w2 = (0.03 * torch.randn(E, H, F, device=DEV, generator=g)).to(torch.bfloat16)
    logits = router_gemm(x, wr)
    logits[:, : max(1, E // 4)] += skew       # uneven load: ragged tiles, and with a strong skew experts without rows
    idx, prob, _, _ = router_topk(logits, k, pre_softmax=True)
    big = permute(idx, prob, E, BM=256)       # streaming kernels where there are 512 tiles or more
    small = permute(idx, prob, E, BM=128)     # always one tile per workgroup
    assert torch.equal(big.sorted_token, small.sorted_token)
    out_a, inter_a = experts_forward(x, w1, w2, big, return_inter=True)
    out_b, inter_b = experts_forward(x, w1, w2, small, return_inter=True)
    assert same_bits(inter_a, inter_b) and same_bits(out_a, out_b)
