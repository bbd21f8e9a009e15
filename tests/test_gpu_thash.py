"""Digests computed by the HIP library against the CPU checker (oracle/thash.py), bit for bit: an equality suite over
dtypes, shapes that straddle the group of 8 and a workgroup's share, ladders, segmentations, layouts and alignments,
plus the vectors of the reference's own eager implementation and size-independent properties at full size.
(The reference's suite of the same kind: isoexec/debug/tests/test_thash_gpu.py:51-142.)"""

import ctypes
import json
import os

import numpy as np
import pytest
import torch

from isoexec_amd._lib import check, current_stream, lib
from isoexec_amd.debug import thash
from oracle import thash as OT

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
HERE = os.path.dirname(os.path.abspath(__file__))

NAMES = ["bfloat16", "float16", "float32", "float64", "int8", "uint8", "int16", "int32", "int64", "bool",
         "float8_e4m3fn", "float8_e5m2", "uint16", "uint32"]
SHAPES = [(1,), (7,), (8,), (9,), (1, 63, 3, 5), (33, 17), (1, 4096), (4097,), (3, 1, 1), (129, 65), (8193, 9)]
NP_VIEW = {1: np.int8, 2: np.int16, 4: np.int32, 8: np.int64}


def sample(name, shape, seed=0):
    g = torch.Generator().manual_seed(seed)
    dtype = getattr(torch, name)
    if name == "bool":
        return torch.randint(0, 2, shape, generator=g).to(torch.bool)
    if dtype.is_floating_point:
        return (torch.randn(shape, generator=g) * 7).to(dtype)
    if name in ("uint16", "uint32"):
        return torch.randint(0, 30000, shape, generator=g).to(torch.int32).to(dtype)
    return torch.randint(-100 if dtype.is_signed else 0, 100, shape, generator=g).to(dtype)


def image_of(t):
    """(integer image as numpy, dtype name, shape) of a host tensor, for the checker."""
    name = str(t.dtype).replace("torch.", "")
    t = t.contiguous()
    raw = t.reshape(-1).view(torch.uint8).numpy() if t.numel() else np.zeros(0, np.uint8)
    width = {"bool": 1}.get(name, min(t.element_size(), 8))
    view = np.uint8 if name in ("uint8", "bool") else NP_VIEW[width]
    return raw.view(view), name, tuple(t.shape)


@pytest.mark.parametrize("name", NAMES)
def test_digest_ladder_and_segments_equal_the_checker(name):
    for number, shape in enumerate(SHAPES):
        host = sample(name, shape, seed=number)
        iv, nm, shp = image_of(host)
        dev = host.to(DEV)
        assert thash.tensor_digest(dev) == OT.tensor_digest(iv, nm, shp), (name, shape)
        assert thash.tensor_digest(dev, seed=77) == OT.tensor_digest(iv, nm, shp, seed=77), (name, shape)
        assert thash.digest_ladder(dev) == OT.digest_ladder(iv, nm, shp), (name, shape)
        for k in thash.ladder_for(dev.dtype)[:2]:
            assert thash.tensor_digest(dev, k=k) == OT.tensor_digest(iv, nm, shp, k=k), (name, shape, k)
        for rps in (1, 3, 16, 4096):
            got = thash.segment_digests(dev, rows_per_segment=rps, seed=5)
            assert got == OT.segment_digests(iv, nm, shp, rows_per_segment=rps, seed=5), (name, shape, rps)


def test_reference_vectors_through_the_device_path():
    with open(os.path.join(HERE, "golden", "thash_vectors.json")) as fh:
        cases = json.load(fh)["cases"]
    for case in cases:
        name, shape, seed = case["dtype"], tuple(case["shape"]), case["seed"]
        view = {"int8": torch.int8, "uint8": torch.uint8, "int16": torch.int16, "int32": torch.int32,
                "int64": torch.int64}[OT.DTYPES[name][0]]
        flat = torch.tensor(case["image"], dtype=view)
        t = (flat.to(torch.bool) if name == "bool" else flat.view(getattr(torch, name))).reshape(shape).to(DEV)
        assert f"{thash.tensor_digest(t, seed=seed):016x}" == case["digest"], (name, shape)
        assert thash.digest_ladder(t, seed=seed) == case["ladder"], (name, shape)
        for rps, want in case["segments"].items():
            assert thash.segment_digests(t, rows_per_segment=int(rps), seed=seed) == want, (name, shape, rps)
        if "segments_k2" in case:
            assert thash.segment_digests(t, rows_per_segment=2, k=2, seed=seed) == case["segments_k2"]


def test_complex_images():
    for name, shape in (("complex64", (9, 5)), ("complex128", (7, 3))):
        g = torch.Generator().manual_seed(3)
        host = torch.randn(shape + (2,), generator=g, dtype=torch.float32 if name == "complex64" else torch.float64)
        host = torch.view_as_complex(host)
        iv = torch.view_as_real(host).contiguous().view(torch.int64).reshape(-1).numpy()
        dev = host.to(DEV)
        assert thash.tensor_digest(dev) == OT.tensor_digest(iv, name, shape)
        assert thash.segment_digests(dev, rows_per_segment=2) == OT.segment_digests(iv, name, shape, rows_per_segment=2)
        assert set(thash.digest_ladder(dev)) == {"full"}


def test_logical_order_not_layout_and_unaligned_views():
    host = sample("bfloat16", (64, 96), seed=1)
    dev = host.to(DEV)
    base = thash.tensor_digest(dev)
    assert thash.tensor_digest(dev.t().contiguous().t()) == base                  # strided view, same contents
    assert thash.tensor_digest(dev[:, ::2]) == thash.tensor_digest(dev[:, ::2].contiguous())
    iv, nm, _ = image_of(host.t())
    assert thash.tensor_digest(dev.t()) == OT.tensor_digest(iv, nm, (96, 64)) != base
    # a contiguous view whose first byte is 2 bytes past a 16-byte boundary: element-wise loads
    flat = dev.reshape(-1)
    for start in (1, 3, 5):
        piece = flat[start:start + 4001]
        ivp, nm, shp = image_of(host.reshape(-1)[start:start + 4001])
        assert piece.data_ptr() % 16 != 0
        assert thash.tensor_digest(piece) == OT.tensor_digest(ivp, nm, shp)
        assert thash.digest_ladder(piece) == OT.digest_ladder(ivp, nm, shp)
        assert thash.segment_digests(piece, rows_per_segment=333) == OT.segment_digests(ivp, nm, shp, rows_per_segment=333)


def test_sensitivity():
    t = sample("bfloat16", (64, 64), seed=2).to(DEV)
    base = thash.tensor_digest(t)
    flipped = t.clone()
    flipped.reshape(-1).view(torch.int16)[1234] ^= 1
    assert thash.tensor_digest(flipped) != base
    swapped = t.clone()
    swapped[0, 0], swapped[0, 1] = t[0, 1].clone(), t[0, 0].clone()
    assert (swapped != t).any() and thash.tensor_digest(swapped) != base            # a swap inside one group of 8
    assert thash.tensor_digest(t.flip(0).contiguous()) != base
    assert thash.tensor_digest(t.view(torch.int16)) != base                          # same bytes, other dtype
    assert thash.tensor_digest(t.reshape(32, 128)) != base
    a = torch.randn(16, 32, device=DEV)
    b = a.clone()
    b[5, 7] += 1.0
    sa, sb = thash.segment_digests(a, rows_per_segment=4), thash.segment_digests(b, rows_per_segment=4)
    assert thash.first_divergent_segments(sa, sb) == [1]


def test_ladder_brackets_a_flipped_mantissa_bit():
    for bit in range(7):
        a = (torch.rand(50, generator=torch.Generator().manual_seed(bit)) + 0.5).to(torch.bfloat16).to(DEV)
        u = a.clone()
        u.view(torch.int16)[7] ^= 1 << bit
        la, lb = thash.digest_ladder(a), thash.digest_ladder(u)
        assert la["full"] != lb["full"]
        assert [k for k in (6, 4, 2, 0) if la[f"k{k}"] == lb[f"k{k}"]] == [k for k in (6, 4, 2, 0) if bit < 7 - k]


def test_empty_and_scalar():
    for host in (torch.empty(0, 8), torch.tensor(3.5), torch.empty(0, 4, dtype=torch.bfloat16)):
        iv, nm, shp = image_of(host)
        dev = host.to(DEV)
        want = OT.tensor_digest(iv, nm, shp)
        assert thash.tensor_digest(dev) == want
        assert thash.segment_digests(dev, rows_per_segment=4) == [f"{want:016x}"]
    assert thash.tensor_digest(torch.empty(0, 8, device=DEV)) != thash.tensor_digest(torch.empty(0, 4, device=DEV))


def test_many_workgroups_and_many_segments_equal_the_checker():
    g = torch.Generator().manual_seed(11)
    host = (torch.randn(4096, 2048, generator=g) * 3).to(torch.bfloat16)           # 8.4 M elements: partial sums + finish
    iv, nm, shp = image_of(host)
    dev = host.to(DEV)
    assert thash.tensor_digest(dev) == OT.tensor_digest(iv, nm, shp)
    assert thash.digest_ladder(dev) == OT.digest_ladder(iv, nm, shp)
    for rps in (1, 64, 1500):
        assert thash.segment_digests(dev, rows_per_segment=rps) == OT.segment_digests(iv, nm, shp, rows_per_segment=rps)
    wide = torch.randn(70000, 24, generator=g)                                       # more slabs than a grid has rows
    iv, nm, shp = image_of(wide)
    assert thash.segment_digests(wide.to(DEV), rows_per_segment=1) == OT.segment_digests(iv, nm, shp, rows_per_segment=1)


def _sums(x, elem_bytes, count, masks, salt=0x1234):
    handle = lib()
    need = handle.ix_digest_workspace_words(1, count, len(masks))
    work = torch.empty(max(1, need), dtype=torch.int64, device=x.device)
    out = torch.empty(len(masks), dtype=torch.int64, device=x.device)
    arr = (ctypes.c_uint64 * 8)(*masks)
    check(handle.ix_digest_sums(x.data_ptr(), elem_bytes, count, salt, arr, len(masks), work.data_ptr(), need,
                                out.data_ptr(), current_stream(x.device)), "ix_digest_sums")
    return [v & OT.U64 for v in out.tolist()]


def test_full_size_properties_through_the_c_abi():
    """[4096, 151936] bf16 logits (1.24 GB): disjoint masks add up, one pass over eight masks equals eight passes,
    masks that reach into the sign extension are honoured, a single flipped bit moves the sum by that bit's weight."""
    rows, vocab = 4096, 151936
    x = torch.empty(rows, vocab, dtype=torch.bfloat16, device=DEV)
    x.view(torch.int16).random_(-32768, 32767, generator=torch.Generator(device=DEV).manual_seed(4))
    n = x.numel()
    full, hi, lo, wide, signs = _sums(x, 2, n, [0xFFFF, 0xFF00, 0x00FF, OT.U64, 0xFFFFFFFFFFFF0000])
    assert (hi + lo) & OT.U64 == full
    assert (full + signs) & OT.U64 == wide
    singles = [_sums(x, 2, n, [m])[0] for m in (0xFFFF, 0xFF00, 0x00FF)]
    assert singles == [full, hi, lo]
    eight = _sums(x, 2, n, [0xFFFF, 0xFFFE, 0xFFFC, 0xFFF0, 0xFFC0, 0xFF80, 0xFF00, 0x8000])
    assert eight[0] == full and eight[6] == hi and len(set(eight)) == 8
    position = 3 * vocab + 12345
    before = int(x.view(torch.int16).reshape(-1)[position].item()) & 0xFFFF
    x.view(torch.int16).reshape(-1)[position] ^= 0x10
    after = before ^ 0x10
    weight = int(OT.weights(position, 1, 0x1234)[0])
    assert _sums(x, 2, n, [0xFFFF])[0] == (full + (after - before) * weight) & OT.U64
    # the module on the same tensor: every slab but the touched one is unchanged by the flip back
    seg_a = thash.segment_digests(x, rows_per_segment=512)
    x.view(torch.int16).reshape(-1)[position] ^= 0x10
    seg_b = thash.segment_digests(x, rows_per_segment=512)
    assert thash.first_divergent_segments(seg_a, seg_b) == [0] and len(seg_a) == 8


def test_bad_arguments_are_refused_not_launched():
    handle = lib()
    x = torch.zeros(64, dtype=torch.int32, device=DEV)
    out = torch.zeros(8, dtype=torch.int64, device=DEV)
    arr = (ctypes.c_uint64 * 8)(*([1] * 8))
    st = current_stream(x.device)
    assert handle.ix_digest_sums(x.data_ptr(), 3, 64, 0, arr, 1, None, 0, out.data_ptr(), st) < 0       # element size
    assert handle.ix_digest_sums(x.data_ptr(), 4, 64, 0, arr, 9, None, 0, out.data_ptr(), st) < 0       # too many masks
    assert handle.ix_digest_sums(x.data_ptr(), 4, 64, 0, arr, 0, None, 0, out.data_ptr(), st) < 0
    assert handle.ix_digest_sums(x.data_ptr() + 2, 4, 8, 0, arr, 1, None, 0, out.data_ptr(), st) < 0    # misaligned element
    assert handle.ix_digest_segment_sums(x.data_ptr(), 4, 64, 3, 16, 0, 1, None, 0, out.data_ptr(), st) < 0  # 64/16 = 4 runs
    big = 1 << 24
    assert handle.ix_digest_workspace_words(1, big, 1) > 0
    y = torch.zeros(big, dtype=torch.int8, device=DEV)
    assert handle.ix_digest_sums(y.data_ptr(), 1, big, 0, arr, 1, None, 0, out.data_ptr(), st) < 0      # workspace missing
    torch.cuda.synchronize()
