"""GPU: the streaming form of the four-wave 256 x 256 GEMM tile (one workgroup per CU walks many tiles; the previous
tile's rounding, quad transposes and stores ride on the next tile's matrix instructions).

It is the same arithmetic per element as every other tile shape (one instruction, one K order, one rounding), so its
output must equal, bit for bit, the eight-wave tile (id 3) and the one-tile-per-workgroup four-wave tile (id 7), for
whole and partial tiles, with and without the row maximum, from one tile per workgroup (everything runs in the closing
flush) to dozens (everything rides on the next tile). Reference counterpart: the invariance gate of
ops/mm/mm_tiles.py:127-158 (one pinned, non-split-K schedule whatever M is)."""

import pytest
import torch

from _util import cpu_gen, same_bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def operands(M, K, N, seed):
    g = cpu_gen(seed)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16).to(DEV)
    w = (0.05 * torch.randn(N, K, generator=g)).to(torch.bfloat16).to(DEV)
    return a, w


@pytest.mark.parametrize("M,K,N", [(256, 704, 256),        # one tile, the fewest k-tiles the streaming form takes
                                   (300, 768, 520),        # partial row tile and partial column tile
                                   (2500, 1024, 1304),     # 60 tiles, most workgroups idle
                                   (4096, 2048, 4096),     # one tile per workgroup
                                   (70000, 768, 256),      # 274 tiles: some workgroups walk two
                                   (20100, 768, 4360),     # 79 x 18 tiles: the wide group shape, partial groups both ways
                                   (16384, 1536, 8192)])   # 2048 tiles: eight per workgroup
def test_streaming_tile_equals_the_other_tiles_bit_for_bit(M, K, N):
    from isoexec_amd.ops.mm.mm_hip import linear_nt

    a, w = operands(M, K, N, seed=M + N)
    ref, ref_max = linear_nt(a, w, tile=3, want_row_max=True)
    one, one_max = linear_nt(a, w, tile=7, want_row_max=True)
    got, got_max = linear_nt(a, w, tile=8, want_row_max=True)
    plain = linear_nt(a, w, tile=8)
    assert same_bits(one, ref) and torch.equal(one_max, ref_max)
    assert same_bits(got, ref) and same_bits(plain, ref)
    assert torch.equal(got_max, ref_max)
    assert torch.equal(got_max, ref.float().amax(dim=1))


def test_default_tile_streams_large_products_and_keeps_the_bits():
    """tile=0 sends a product with hundreds of tiles to the streaming form; a strided output view and the fp32 / bias
    variants (which the streaming form does not serve) still go through the one-tile kernels: same bits everywhere."""
    from isoexec_amd.ops.mm.mm_hip import linear_nt

    a, w = operands(8192, 2048, 16384, seed=5)
    ref = linear_nt(a, w, tile=3)
    assert same_bits(linear_nt(a, w), ref)
    bias = (0.1 * torch.randn(16384, generator=cpu_gen(6))).to(torch.bfloat16).to(DEV)
    assert same_bits(linear_nt(a, w, bias), linear_nt(a, w, bias, tile=3))
    f32 = linear_nt(a, w, out_dtype=torch.float32)
    assert same_bits(f32.to(torch.bfloat16), ref)


def test_streaming_tile_declines_what_it_does_not_serve():
    from isoexec_amd.ops.mm.mm_hip import linear_nt

    a, w = operands(512, 640, 512, seed=7)   # ten k-tiles: one short of what the deferred epilogue needs
    assert linear_nt(a, w, tile=8) is None
    assert linear_nt(a, w, tile=8, out_dtype=torch.float32) is None
    assert same_bits(linear_nt(a, w, tile=4), linear_nt(a, w, tile=3))   # the default big tile falls back to one tile per workgroup
