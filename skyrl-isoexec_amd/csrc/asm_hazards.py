#!/usr/bin/env python3
"""Checks the compiler's device assembly for wait-state rules that the compiler does not apply to inline assembly.

The compiler's hazard recogniser inserts the idle states the instruction set asks for between two instructions it
emitted itself, but it does not look inside an ``asm`` statement. The vector-memory instructions of this library's
matrix kernels are inline assembly (loads straight into LDS, stores through a descriptor), so two documented rules are
on the source to keep:

* a scalar register written by a vector instruction (``v_readfirstlane_b32``, ``v_readlane_b32`` -- which is also how the
  compiler reloads a spilled scalar register -- or a vector compare) must not be read by a vector-memory instruction in
  the next 5 wait states: the memory instruction would use the OLD value as descriptor word or scalar offset, i.e. an
  address the range check never saw;
* M0 written by a scalar instruction must not be read by a load-to-LDS in the next wait state.

Usage: ``asm_hazards.py file.s [file.s ...]`` on the output of ``hipcc -S --offload-device-only`` (``make check``
drives it). Exit status 1 and one line per finding if a rule is broken. The scan walks each function's lines upwards
from every inline-assembly memory instruction; a branch target closer than the five wait states is a finding of its own,
because the instructions that jump there are not on the lines above it.
"""
import re
import sys

VMEM = re.compile(r"^(buffer_|global_|flat_|scratch_|tbuffer_)")
VALU_SGPR_DEF = re.compile(r"^(v_readlane_b32|v_readfirstlane_b32)\s+(s\d+|s\[\d+:\d+\]|vcc_lo|vcc_hi|vcc)")
VCMP_E64 = re.compile(r"^v_cmpx?_\w+_e64\s+(s\[\d+:\d+\]|vcc)")
VCMP_E32 = re.compile(r"^v_cmpx?_\w+_e32\s")
VALU_CARRY = re.compile(r"^v_(add_co|sub_co|subrev_co|addc_co|subb_co|subbrev_co|div_scale|mad_u64_u32|mad_i64_i32)\w*\s+\S+,\s*(s\[\d+:\d+\]|vcc)")
VMEM_SGPR_WAIT = 5
M0_LDS_WAIT = 1


def sregs(text):
    """Scalar registers named in an operand string, as a set of numbers (vcc = 106, 107; m0 = 124)."""
    out = set()
    for m in re.finditer(r"\bs\[(\d+):(\d+)\]", text):
        out.update(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"\bs(\d+)\b", text):
        out.add(int(m.group(1)))
    if re.search(r"\bvcc_lo\b", text):
        out.add(106)
    if re.search(r"\bvcc_hi\b", text):
        out.add(107)
    if re.search(r"\bvcc\b", text):
        out.update((106, 107))
    if re.search(r"\bm0\b", text):
        out.add(124)
    return out


def valu_sgpr_defs(ins):
    """Scalar registers that the vector instruction `ins` writes."""
    m = VALU_SGPR_DEF.match(ins) or VCMP_E64.match(ins)
    if m:
        return sregs(m.group(m.lastindex))
    if VCMP_E32.match(ins):
        return {106, 107}
    m = VALU_CARRY.match(ins)
    if m:
        return sregs(m.group(2))
    return set()


def wait_states(ins):
    m = re.match(r"^s_nop\s+(\d+)", ins)
    return int(m.group(1)) + 1 if m else 1


def scan(path):
    findings = []
    func = "?"
    in_asm = False
    hist = []  # (instruction, from inline asm, source line number), oldest first, of the current function
    for ln, raw in enumerate(open(path), 1):
        s = raw.strip()
        if s.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if s.startswith(";;#ASMEND"):
            in_asm = False
            continue
        m = re.match(r"^([A-Za-z_][\w$.]*):\s*(;.*)?$", raw)
        if m and not raw.startswith(".L"):
            func = m.group(1)
            hist = []
            continue
        if re.match(r"^\.LBB\w+:", raw):
            hist.append(("<label>", False, ln))  # a branch target: what ran before it is not on the lines above
            continue
        if not raw.startswith("\t") or s.startswith(";") or s.startswith("."):
            continue
        ins = s.split(";")[0].strip()
        if not ins:
            continue
        if in_asm and VMEM.match(ins):
            ops = ins.split(None, 1)[1] if " " in ins else ""
            used = sregs(ops)
            lds_dma = bool(re.search(r"\blds\b", ops))
            dist = 0
            for pins, _, pln in reversed(hist):
                if dist >= VMEM_SGPR_WAIT:
                    break
                if pins == "<label>":
                    if used - {124}:
                        findings.append(f"{path}:{ln}: {func}: '{ins}' sits {dist} wait states after the branch target of "
                                        f"line {pln}: the code that jumps there is not checked")
                    continue
                hit = valu_sgpr_defs(pins) & used
                if hit:
                    findings.append(f"{path}:{ln}: {func}: '{ins}' reads s{sorted(hit)} {dist} wait states after "
                                    f"'{pins}' (line {pln}); {VMEM_SGPR_WAIT} needed")
                if lds_dma and dist < M0_LDS_WAIT and re.match(r"^s_\w+\s+m0\b", pins):
                    findings.append(f"{path}:{ln}: {func}: '{ins}' reads m0 {dist} wait states after '{pins}'")
                dist += wait_states(pins)
        hist.append((ins, in_asm, ln))
        if len(hist) > 16:
            hist.pop(0)
    return findings


def main(argv):
    bad = []
    for p in argv[1:]:
        bad += scan(p)
    for f in bad:
        print(f)
    print(f"asm_hazards: {len(argv) - 1} files, {len(bad)} findings")
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
