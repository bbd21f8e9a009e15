"""GPU: the permutation entry point that allocates nothing (its tables live in a file-scope device array) gives the
integers of ix_moe_permute, on two calls in a row, the second smaller (it must not see what the first left behind)."""

import ctypes

import numpy as np
import pytest
import torch

from _util import cpu_gen

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _routing(T, E, k, seed):
    from isoexec_amd.ops.moe.moe_hip import router_topk

    logits = torch.randn(T, E, generator=cpu_gen(seed))
    logits[:, :4] += 3.0
    idx, prob, _, _ = router_topk(logits.to(DEV), k)
    return idx.contiguous(), prob.contiguous()


def _buffers(L, T, E, k, BM):
    i32 = dict(dtype=torch.int32, device=DEV)
    max_tiles = int(L.ix_moe_max_tiles(T, k, E, BM))
    # poisoned, so that an entry a call failed to write shows up in the comparison
    return max_tiles, dict(
        counts=torch.full((E,), -7, **i32), offsets=torch.full((E + 1,), -7, **i32),
        sorted_token=torch.full((T * k,), -7, **i32),
        permuted_prob=torch.full((T * k,), -7.0, dtype=torch.float32, device=DEV),
        combine_rows=torch.full((T, k), -7, **i32), tile_meta=torch.full((1 + 3 * max_tiles,), -7, **i32))


def _call(L, name, idx, prob, T, E, k, BM, scratch):
    max_tiles, b = _buffers(L, T, E, k, BM)
    stream = torch.cuda.current_stream().cuda_stream
    args = [idx.data_ptr(), prob.data_ptr(), T, E, k, BM, b["counts"].data_ptr(), b["offsets"].data_ptr(),
            b["sorted_token"].data_ptr(), b["permuted_prob"].data_ptr(), b["combine_rows"].data_ptr(),
            b["tile_meta"].data_ptr(), max_tiles]
    if scratch is not None:
        args.append(scratch.data_ptr())
    rc = getattr(L, name)(*args, stream)
    assert rc == 0, (name, rc)
    torch.cuda.synchronize()
    out = {n: t.cpu().numpy() for n, t in b.items()}
    meta = out.pop("tile_meta")
    nt = int(meta[0])
    out["n_tiles"] = np.array([nt])
    for i, n in enumerate(("tile_expert", "tile_row0", "tile_nrows")):
        out[n] = meta[1 + i * max_tiles: 1 + i * max_tiles + nt]
    return out


@pytest.mark.parametrize("sizes", [((2000, 128, 8, 256), (700, 128, 8, 256)), ((16384, 128, 8, 256), (300, 16, 4, 32)),
                                   ((900, 60, 2, 128), (40, 60, 2, 32))])
def test_static_scratch_permutation_equals_workspace_permutation(sizes):
    from isoexec_amd import _lib

    L = _lib.lib()
    for n, (T, E, k, BM) in enumerate(sizes):      # two calls in a row, the second with a smaller input
        idx, prob = _routing(T, E, k, seed=10 * T + n)
        scratch = torch.full((max(1, int(L.ix_moe_permute_scratch_ints(T, E))),), -1, dtype=torch.int32, device=DEV)
        want = _call(L, "ix_moe_permute", idx, prob, T, E, k, BM, scratch)
        got = _call(L, "ix_moe_permute_static", idx, prob, T, E, k, BM, None)
        assert want["counts"].sum() == T * k and want["n_tiles"][0] > 0
        for name in want:
            assert np.array_equal(got[name].view(np.uint32), want[name].view(np.uint32)), (name, T, E, k, BM)


def test_static_scratch_permutation_allocates_nothing():
    """What the entry point exists for: after set-up, calls move neither the device's free memory (the runtime's own
    figure, hipMemGetInfo) nor torch's allocator; the workspace form needs its scratch tensor for the same input."""
    from isoexec_amd import _lib

    L = _lib.lib()
    assert L.ix_moe_permute_static_init() == 0 and L.ix_moe_permute_static_init() == 0
    T, E, k, BM = 5000, 128, 8, 256
    idx, prob = _routing(T, E, k, seed=77)
    max_tiles, b = _buffers(L, T, E, k, BM)
    stream = torch.cuda.current_stream().cuda_stream
    args = [idx.data_ptr(), prob.data_ptr(), T, E, k, BM, b["counts"].data_ptr(), b["offsets"].data_ptr(),
            b["sorted_token"].data_ptr(), b["permuted_prob"].data_ptr(), b["combine_rows"].data_ptr(),
            b["tile_meta"].data_ptr(), max_tiles, stream]
    assert L.ix_moe_permute_static(*args) == 0
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    alloc0, reserved0 = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    for _ in range(20):
        assert L.ix_moe_permute_static(*args) == 0
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0 and torch.cuda.memory_allocated() == alloc0 and torch.cuda.memory_reserved() == reserved0
    assert int(b["counts"].sum()) == T * k


def test_static_scratch_permutation_refuses_what_does_not_fit():
    """Host-side check only: nothing is launched for an input beyond the array."""
    from isoexec_amd import _lib

    L = _lib.lib()
    limit = int(L.ix_moe_permute_static_max_ints())
    assert limit == 256 * 1024
    T, E = 256 * 1100, 128
    assert int(L.ix_moe_permute_scratch_ints(T, E)) > limit
    one = torch.zeros(1, dtype=torch.int32, device=DEV)
    p = one.data_ptr()
    rc = L.ix_moe_permute_static(p, p, T, E, 8, 256, p, p, p, p, p, p, int(L.ix_moe_max_tiles(T, 8, E, 256)), None)
    assert rc == -3
    assert L.ix_moe_permute_static(p, p, -1, E, 8, 256, p, p, p, p, p, p, 0, None) == -1
