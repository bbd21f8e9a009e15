"""The build's check of the device assembly (csrc/asm_hazards.py): each rule on a few lines written by hand.

The compiler does not place wait states around instructions inside an ``asm`` statement; the check is what keeps a
reloaded scalar register from being read too early by such a load (the cause of two GPU memory faults of an earlier
build of the streaming expert GEMM), so it gets tests of its own: every rule must fire on the pattern it is for and
stay quiet on the legal neighbour of that pattern.
"""
import importlib.util
import os
import subprocess
import sys

import pytest

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "skyrl-isoexec_amd", "csrc")
spec = importlib.util.spec_from_file_location("asm_hazards", os.path.join(CSRC, "asm_hazards.py"))
asm_hazards = importlib.util.module_from_spec(spec)
spec.loader.exec_module(asm_hazards)


def scan(tmp_path, body):
    p = tmp_path / "k.s"
    p.write_text("k_test:                                 ; @k_test\n" + body + ".Lfunc_end0:\n")
    return asm_hazards.scan(str(p))


def asm(*lines):
    return "\t;;#ASMSTART\n" + "".join(f"\t{l}\n" for l in lines) + "\t;;#ASMEND\n"


DMA = ("s_mov_b32 m0, s9", "s_nop 0", "buffer_load_dwordx4 v39, s[16:19], s20 offen lds")


def test_reloaded_scalar_offset_needs_five_wait_states(tmp_path):
    # the pattern of the faulting build: spill reload, then the load two wait states later
    bad = "\tv_readlane_b32 s20, v221, 18\n" + asm(*DMA)
    found = scan(tmp_path, bad)
    assert len(found) == 1 and "reads s[20] 2 wait states after" in found[0]
    # three more idle states in the statement: legal
    assert scan(tmp_path, "\tv_readlane_b32 s20, v221, 18\n" + asm(DMA[0], "s_nop 3", DMA[2])) == []
    # five unrelated instructions in between: legal
    filler = "".join(f"\tv_add_u32_e32 v{i}, v{i}, v{i}\n" for i in range(3))
    assert scan(tmp_path, "\tv_readlane_b32 s20, v221, 18\n" + filler + asm(*DMA)) == []
    # a scalar instruction writing the same register is no hazard
    assert scan(tmp_path, "\ts_add_i32 s20, s20, s4\n" + asm(*DMA)) == []


def test_descriptor_words_moved_by_a_vector_instruction(tmp_path):
    store = "buffer_store_dwordx4 v[172:175], v75, s[4:7], 0 offen"
    bad = "\tv_readfirstlane_b32 s4, v108\n\tv_readfirstlane_b32 s5, v107\n\tv_readfirstlane_b32 s6, v106\n" + asm(store)
    assert len(scan(tmp_path, bad)) == 3
    good = "\tv_readfirstlane_b32 s4, v108\n\tv_readfirstlane_b32 s5, v107\n\tv_readfirstlane_b32 s6, v106\n" + asm("s_nop 4", store)
    assert scan(tmp_path, good) == []
    # a compare that writes a scalar pair counts as well
    assert len(scan(tmp_path, "\tv_cmp_lt_u32_e64 s[4:5], v1, v2\n" + asm(store))) == 1
    # the same store emitted by the compiler itself (outside an asm statement) is the compiler's business
    assert scan(tmp_path, "\tv_readfirstlane_b32 s4, v108\n\t" + store + "\n") == []


def test_m0_needs_one_wait_state_before_a_load_to_lds(tmp_path):
    assert len(scan(tmp_path, asm("s_mov_b32 m0, s9", "buffer_load_dwordx4 v39, s[16:19], s20 offen lds"))) == 1
    assert scan(tmp_path, asm(*DMA)) == []


def test_the_walk_follows_jumps_to_a_branch_target(tmp_path):
    # the instruction above the label is harmless, the one in front of the jump is not
    body = ("\tv_readlane_b32 s20, v221, 18\n\ts_branch .LBB0_2\n.LBB0_1:\n\ts_add_i32 s20, s20, s4\n.LBB0_2:\n" + asm(*DMA))
    found = scan(tmp_path, body)
    assert len(found) == 1 and "v_readlane_b32 s20" in found[0]
    body_ok = ("\ts_mov_b32 s20, s7\n\ts_branch .LBB0_2\n.LBB0_1:\n\ts_add_i32 s20, s20, s4\n.LBB0_2:\n" + asm(*DMA))
    assert scan(tmp_path, body_ok) == []


def test_uncounted_load_must_be_retired_and_untouched(tmp_path):
    load = asm("global_load_dword v8, v1, s[26:27]")
    dmas = "".join(asm(*DMA) for _ in range(8))
    take = asm("; ix_landed v8")
    wait = "\ts_waitcnt vmcnt(8) lgkmcnt(0)\n"
    assert scan(tmp_path, load + dmas + wait + take) == []
    # the wait leaves more operations in flight than were issued after the load: it may still be one of them
    found = scan(tmp_path, load + "".join(asm(*DMA) for _ in range(7)) + wait + take)
    assert len(found) == 1 and "no wait since its load" in found[0]
    # a copy of the register before it has landed
    found = scan(tmp_path, load + "\tv_mov_b32_e32 v9, v8\n" + dmas + wait + take)
    assert len(found) == 1 and "touches v8" in found[0]
    # also as part of a register range
    found = scan(tmp_path, load + "\tds_write_b128 v2, v[6:9]\n" + dmas + wait + take)
    assert len(found) == 1 and "touches v8" in found[0]
    # never taken into use
    assert any("never taken into use" in f for f in scan(tmp_path, load + dmas + wait))
    # a marker without a load
    assert any("without an uncounted load" in f for f in scan(tmp_path, take))
    # control flow between the load and its use: the file order is not the execution order, the rule says so
    found = scan(tmp_path, load + dmas + ".LBB0_3:\n" + wait + take)
    assert len(found) == 1 and "label .LBB0_3" in found[0] and "not straight-line" in found[0]
    found = scan(tmp_path, load + dmas + "\ts_cbranch_scc1 .LBB0_9\n" + wait + take)
    assert len(found) == 1 and "s_cbranch_scc1" in found[0]
    # the same label or branch outside the window is nobody's business
    assert scan(tmp_path, ".LBB0_3:\n" + load + dmas + wait + take + "\ts_cbranch_scc1 .LBB0_3\n") == []


def test_accumulator_read_waits_for_the_matrix_pipeline(tmp_path):
    mfma = "\tv_mfma_f32_32x32x16_bf16 a[240:255], v[64:67], v[12:15], a[240:255]\n"
    read = asm("v_accvgpr_read_b32 v5, a241")
    assert len(scan(tmp_path, mfma + read)) == 1
    assert scan(tmp_path, mfma + asm("s_nop 15", "s_nop 15") + read) == []
    # fifteen other matrix instructions and their companions in between (the streaming kernels' distance): legal
    others = "".join(f"\tv_mfma_f32_32x32x16_bf16 a[{16 * i}:{16 * i + 15}], v[64:67], v[12:15], a[{16 * i}:{16 * i + 15}]\n"
                     "\tds_read_b128 v[0:3], v9\n" for i in range(14))
    assert scan(tmp_path, mfma + others + read) == []
    # a read of another block right behind it is no hazard of this instruction
    assert scan(tmp_path, mfma + asm("v_accvgpr_read_b32 v5, a17")) == []


def test_built_assembly_is_clean_when_present():
    files = [os.path.join(CSRC, f) for f in ("ix_gemm.dev.s", "ix_moe.dev.s", "ix_attn.dev.s")]
    if not all(os.path.exists(f) for f in files):
        pytest.skip("device assembly not built here (make check writes it)")
    r = subprocess.run([sys.executable, os.path.join(CSRC, "asm_hazards.py")] + files, capture_output=True, text=True)
    assert r.returncode == 0, r.stdout[-2000:]
