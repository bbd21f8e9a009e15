"""The streaming form of the dense product for at most 64 rows (``ix_gemm_bf16_nt_decode``) against the tile kernels
(``ix_gemm_bf16_nt``), bit for bit, through the C ABI: the same matrix instruction, K order and rounding, so the two
must agree on every element whatever the shape; and against the integer known answer, which no order can move."""

import pytest
import torch

from _util import cpu_gen, same_bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def operands(m, n, k, seed, pitch=0):
    g = cpu_gen(seed)
    x = torch.randn(m, k + pitch, generator=g).to(torch.bfloat16).to(DEV)[:, :k]
    w = (torch.randn(n, k, generator=g) * 0.05).to(torch.bfloat16).to(DEV)
    return x, w


@pytest.mark.parametrize("m", [1, 7, 32, 33, 64])
@pytest.mark.parametrize("n,k", [(96, 1024), (2048, 4096), (12352, 2048), (5120, 3072), (65568, 2048)])
def test_streaming_form_equals_the_tile_kernels(m, n, k):
    from isoexec_amd.ops.mm.mm_hip import PackedWeight, linear_nt, linear_nt_decode, pack_nt_decode

    x, w = operands(m, n, k, seed=m + n, pitch=64 if m == 33 else 0)      # one case with a row pitch above K
    packed = pack_nt_decode(w)
    assert isinstance(packed, PackedWeight) and packed.packed.numel() == n * k
    want = linear_nt(x, w)
    got = linear_nt_decode(x, packed)
    assert got is not None and same_bits(got, want)
    assert same_bits(linear_nt(x, packed), want)                            # the door picks the streaming form itself
    # and every row is what it is alone (the product does not depend on what else is in the batch)
    if m > 1:
        assert same_bits(linear_nt_decode(x[m - 1:m], packed), want[m - 1:m])


def test_integer_known_answer():
    from isoexec_amd.ops.mm.mm_hip import linear_nt_decode, pack_nt_decode

    g = cpu_gen(5)
    m, n, k = 64, 4096, 2048
    x = torch.randint(-3, 4, (m, k), generator=g)
    w = torch.randint(-3, 4, (n, k), generator=g)
    want = (x.double() @ w.double().T)                                      # |sum| <= 9 K < 2^24: exact in fp32
    got = linear_nt_decode(x.to(torch.bfloat16).to(DEV), pack_nt_decode(w.to(torch.bfloat16).to(DEV)))
    assert torch.equal(got.cpu(), want.to(torch.bfloat16))


def test_what_the_form_does_not_serve_is_declined_and_the_door_falls_back():
    from isoexec_amd.ops.mm.mm_hip import linear_nt, linear_nt_decode, pack_nt_decode

    assert pack_nt_decode(torch.zeros(48, 2048, dtype=torch.bfloat16, device=DEV)) is None      # N not a multiple of 32
    assert pack_nt_decode(torch.zeros(64, 512, dtype=torch.bfloat16, device=DEV)) is None       # K not served
    assert pack_nt_decode(torch.zeros(64, 2048, dtype=torch.float32, device=DEV)) is None
    x, w = operands(65, 256, 2048, seed=3)
    packed = pack_nt_decode(w)
    assert linear_nt_decode(x, packed) is None                                                   # more than 64 rows
    want = linear_nt(x, w)
    assert same_bits(linear_nt(x, packed), want)                                                 # the door uses the weight itself
    bias = torch.randn(256).to(torch.bfloat16).to(DEV)
    assert same_bits(linear_nt(x[:8], packed, bias), linear_nt(x[:8], w, bias))
    out, row_max = linear_nt(x[:8], packed, want_row_max=True)
    assert same_bits(out, want[:8]) and torch.equal(row_max, want[:8].float().amax(dim=1))
    assert same_bits(linear_nt(x[:8], packed, out_dtype=torch.float32), linear_nt(x[:8], w, out_dtype=torch.float32))
