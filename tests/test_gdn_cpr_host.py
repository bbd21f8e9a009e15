"""Host metadata of the chunk-boundary GatedDeltaNet forward (reference ops/gdn/gdn_cpr.py:25-51,187-222): pure
integer bookkeeping, checked against hand-written vectors and a brute-force walk."""

import numpy as np
import torch

from isoexec_amd.ops.gdn import gdn_cpr


def test_chunked_cu_seqlens_and_indices_hand_vector():
    cu = torch.tensor([0, 5, 5, 69, 70], dtype=torch.int32)  # lengths 5, 0, 64, 1
    cu_c, idx, n = gdn_cpr.chunked_cu_seqlens_and_indices(cu, 32, "cpu")
    assert cu_c.dtype is torch.int32 and idx.dtype is torch.int32
    assert cu_c.tolist() == [0, 5, 37, 69, 70]        # chunks: 5 | 32 32 | 1 (the empty sequence has none)
    assert n == 4 and idx.shape == (4, 32)
    assert idx[:, 0].tolist() == [1, 2, 3, 4]          # pool rows count from 1: row 0 is the null row
    assert not idx[:, 1:].any()                         # only column 0 is set


def test_chunk_meta_against_a_brute_force_walk():
    rng = np.random.default_rng(3)
    for chunk in (2, 16, 64):
        lens = rng.integers(0, 200, size=9).tolist()
        idx, off = gdn_cpr.host_chunk_meta(lens, chunk, "cpu")
        want_idx, want_off = [], [0]
        for s, n in enumerate(lens):
            nc = 0
            for pos in range(0, n, chunk):
                want_idx.append([s, nc])
                nc += 1
            want_off.append(want_off[-1] + nc)
        assert idx.dtype is torch.int32 and off.dtype is torch.int64   # offsets are int64 whatever the index dtype
        assert idx.tolist() == want_idx and off.tolist() == want_off
        cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32)
        cu_c, sidx, n = gdn_cpr.chunked_cu_seqlens_and_indices(cu, chunk, "cpu")
        assert n == len(want_idx) and sidx.shape == (n, chunk)
        seg = np.diff(cu_c.numpy())
        assert seg.sum() == sum(lens) and (seg > 0).all() and (seg <= chunk).all()
        # every chunk but a sequence's last is full
        k = 0
        for s, nlen in enumerate(lens):
            nc = -(-nlen // chunk)
            assert (seg[k:k + nc - 1] == chunk).all() if nc > 1 else True
            k += nc
    assert gdn_cpr.host_chunk_meta([], 16, "cpu")[0].shape == (0, 2)


def test_chunk_meta_is_cached_and_sequence_metadata_memoized(monkeypatch):
    a = gdn_cpr.host_chunk_meta([3, 70], 32, "cpu")
    b = gdn_cpr.host_chunk_meta([3, 70], 32, "cpu")
    assert a[0] is b[0] and a[1] is b[1]
    cu = torch.tensor([0, 3, 73], dtype=torch.int32)
    before = gdn_cpr.seq_meta_census()
    m1 = gdn_cpr.sequence_metadata(cu, 32, "cpu")
    m2 = gdn_cpr.sequence_metadata(cu, 32, "cpu")
    after = gdn_cpr.seq_meta_census()
    assert m1 is m2 and after["built"] == before["built"] + 1 and after["served"] == before["served"] + 1
    assert m1[0] == [3, 70] and m1[4] == 4 and torch.equal(m1[1], cu) and m1[1] is not cu
    cu[2] = 80  # an in-place edit bumps the version: the memo must not serve the stale entry
    m3 = gdn_cpr.sequence_metadata(cu, 32, "cpu")
    assert m3[0] == [3, 77] and m3[2].tolist() == [0, 3, 35, 67, 80]
    monkeypatch.setenv("SKYRL_ISOEXEC_GDN_SEQ_META_CACHE", "0")
    d0 = gdn_cpr.seq_meta_census()["declined"]
    gdn_cpr.sequence_metadata(cu, 32, "cpu")
    assert gdn_cpr.seq_meta_census()["declined"] == d0 + 1


def test_state_pool_widens_the_snapshot_behind_a_null_row():
    h = torch.arange(2 * 3 * 2 * 2 * 2, dtype=torch.float32).reshape(2, 3, 2, 2, 2).to(torch.bfloat16)
    pool = gdn_cpr._state_pool(h, 5, "cpu")
    assert pool.dtype is torch.float32 and pool.shape == (6, 2, 2, 2)
    assert not pool[0].any() and torch.equal(pool[1:], h.reshape(6, 2, 2, 2)[:5].float())


def test_kernel_selector_vocabulary_default_and_refusal(monkeypatch):
    """core/gdn_kernel_env.py of the reference: empty -> recurrent, unknown names refuse (a typo must not fall
    back), a retired spelling names its successor, and the trainer override is None unless set."""
    import pytest

    from isoexec_amd.core import gdn_kernel_env as env

    monkeypatch.delenv(env.KERNEL_ENV, raising=False)
    monkeypatch.delenv(env.TRAINER_KERNEL_ENV, raising=False)
    assert env.gdn_kernel_mode() == "recurrent" and env.gdn_trainer_kernel_override() is None
    for raw, want in ((" CPR ", "cpr"), ("recurrent", "recurrent"), ("chunk", "chunk"), ("", "recurrent")):
        monkeypatch.setenv(env.KERNEL_ENV, raw)
        assert env.gdn_kernel_mode() == want
    monkeypatch.setenv(env.KERNEL_ENV, "chunk_synced")
    with pytest.raises(ValueError, match="renamed to 'cpr'"):
        env.gdn_kernel_mode()
    monkeypatch.setenv(env.KERNEL_ENV, "recurent")
    with pytest.raises(ValueError, match="names no delta-rule kernel"):
        env.gdn_kernel_mode()
    monkeypatch.setenv(env.KERNEL_ENV, "recurrent")
    monkeypatch.setenv(env.TRAINER_KERNEL_ENV, "cpr")
    assert env.gdn_trainer_kernel_override() == "cpr"
    from isoexec_amd.ops.gdn import gdn_ops

    assert gdn_ops.recurrent_mode() and not gdn_ops.cpr_mode() and gdn_ops.fla_chunk_size() == 64
