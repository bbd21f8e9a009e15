"""Host side of the digest module (no GPU): vocabulary, masks, header, walking a region's outputs, and the refusal
of tensors the HIP library cannot reach. The expectations are those of the reference's own CPU tests
(isoexec/debug/tests/test_thash_cpu.py:206-222, 246-273, 339-350) and the golden vectors' header conventions."""

import json
import os

import pytest
import torch

from isoexec_amd import debug
from isoexec_amd._lib import IsoExecLibraryError
from isoexec_amd.debug import thash
from oracle import thash as OT

HERE = os.path.dirname(os.path.abspath(__file__))


def test_ladders_follow_the_dtype():
    assert thash.ladder_for(torch.bfloat16) == (6, 4, 2, 0)
    assert max(thash.ladder_for(torch.float32)) == 22
    assert max(thash.ladder_for(torch.float64)) == 48
    assert thash.ladder_for(torch.float16) == (9, 7, 5, 3, 1, 0)
    assert thash.ladder_for(torch.int32) == () and thash.mantissa_bits(torch.bool) is None
    assert thash.mantissa_bits(torch.float8_e4m3fn) == 3 and thash.ladder_for(torch.float8_e5m2) == (1, 0)


def test_masks_and_kept_bits_agree_with_the_checker():
    for dtype, kind in thash._KINDS.items():
        name = str(dtype).replace("torch.", "")
        assert kind.code == OT.DTYPES[name][3], name
        for k in (None,) + thash.ladder_for(dtype) + (60,):
            assert thash._mask_for(kind, k) == OT.and_mask(name, k), (name, k)


def test_header_agrees_with_the_checker_and_separates_shapes():
    for shape in ((), (1,), (6, 8), (8, 6), (0, 4), (1, 63, 3, 5)):
        t = torch.empty(shape, dtype=torch.bfloat16)
        kind = thash._KINDS[t.dtype]
        for kept, seed in ((7, 0), (2, 0), (7, 99), (-1, 3)):
            assert thash._header(t, kind, kept, seed) == OT.header(shape, "bfloat16", kept, seed)
    a = thash._header(torch.empty(6, 8), thash._KINDS[torch.float32], 23, 0)
    assert a != thash._header(torch.empty(8, 6), thash._KINDS[torch.float32], 23, 0)
    assert a != thash._header(torch.empty(48), thash._KINDS[torch.float32], 23, 0)


def test_segment_axis_is_the_first_axis_with_rows():
    assert thash.segment_axis(torch.zeros(1, 64, 4, 8)) == 1
    assert thash.segment_axis(torch.zeros(64, 1, 2048)) == 0
    assert thash.segment_axis(torch.zeros(1, 1, 1)) == 0
    assert thash.segment_axis(torch.zeros(7)) == 0


def test_region_outputs_are_walked_in_order():
    t1, t2 = torch.zeros(2), torch.ones(3)
    assert [p for p, _ in thash.iter_tensor_outputs(t1)] == ["0"]
    assert [p for p, _ in thash.iter_tensor_outputs((t1, None, t2))] == ["0", "2"]
    assert list(thash.iter_tensor_outputs("nope")) == [] and list(thash.iter_tensor_outputs(None)) == []
    assert [p for p, _ in thash.iter_tensor_outputs((t1, (t1, t2)))] == ["0", "1.0", "1.1"]
    assert [p for p, _ in thash.iter_tensor_outputs({"h": t1, "aux": [t2]})] == ["h", "aux.0"]
    assert [p for p, _ in thash.iter_tensor_outputs([(t1, {"x": t2}), t1])] == ["0.0", "0.1.x", "1"]
    deep = (((t1,),),)
    assert list(thash.iter_tensor_outputs(deep, max_depth=2)) == [("0.0", None)]


def test_divergent_segments():
    assert thash.first_divergent_segments(["a", "b", "c"], ["a", "x", "c"]) == [1]
    assert thash.first_divergent_segments(["a"], ["a"]) == []
    assert thash.first_divergent_segments(["a"], ["a", "b"]) == [0, 1]


def test_host_tensors_and_unknown_dtypes_are_refused():
    with pytest.raises(IsoExecLibraryError, match="no CPU fallback"):
        thash.tensor_digest(torch.zeros(4))
    with pytest.raises(IsoExecLibraryError):
        thash.segment_digests(torch.zeros(4, 4), rows_per_segment=2)
    exotic = next((getattr(torch, n) for n in ("float8_e8m0fnu", "bits8", "float4_e2m1fn_x2")
                   if getattr(torch, n, None) is not None and getattr(torch, n) not in thash._KINDS), None)
    if exotic is not None:
        with pytest.raises((TypeError, IsoExecLibraryError)):
            thash.tensor_digest(torch.zeros(4).to(exotic))


def test_package_reexports_lazily():
    assert debug.tensor_digest is thash.tensor_digest and debug.preload_digest is thash.preload
    assert "segment_digests" in debug.__all__
    with pytest.raises(AttributeError):
        debug.no_such_name


def test_workspace_sizing_is_host_arithmetic():
    from isoexec_amd._lib import lib

    handle = lib()
    assert handle.ix_digest_workspace_words(1, 100, 1) == 0            # one workgroup writes the result itself
    big = handle.ix_digest_workspace_words(1, 1 << 26, 5)
    assert big > 0 and big % 5 == 0 and big <= 2048 * 5
    assert handle.ix_digest_workspace_words(100000, 2048, 1) == 0      # many small segments: one workgroup each
    assert handle.ix_digest_workspace_words(4, 1 << 24, 1) == 4 * 512
