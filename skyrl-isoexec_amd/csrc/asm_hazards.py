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

* an accumulation register written by a matrix instruction must not be read by an inline-assembly
  ``v_accvgpr_read_b32`` before the matrix pipeline has delivered it: 19 wait states cover the longest instruction
  (the kernels place ``s_nop 15`` twice in front of the first read).

A last rule is this library's own. ``ix_load4_uncounted`` issues ``global_load_dword vN`` from inline assembly, so the
compiler believes vN holds the value at once; the value is taken into use through ``ix_landed`` (which leaves the
comment ``; ix_landed vN`` in the assembly). Between the two
* no instruction may mention vN (a copy or a spill would move a value that has not arrived), and
* there must be an ``s_waitcnt vmcnt(n)`` with at least n vector-memory instructions issued after the load (they
  retire in order, so that wait has retired the load);
* and no label, branch or jump may lie between the load and its ``ix_landed``: this rule is judged on the lines in
  their order in the file, which is only the order of execution for straight-line code.

The rules cover the instruction classes the inline assembly of this library uses today. A NEW class of inline-assembly
instruction (an LDS instruction that reads M0, a scalar load whose result feeds a vector-memory instruction, a
different matrix instruction with its own latency, ...) gets its own rule here and a case in tests/test_asm_hazards.py
before the kernel that contains it runs on a GPU for the first time.

Usage: ``asm_hazards.py file.s [file.s ...]`` on the output of ``hipcc -S --offload-device-only`` (``make check``
drives it). Exit status 1 and one line per finding if a rule is broken. The scan walks upwards from every
inline-assembly memory instruction, at a branch target along the lines above it and along every jump to it.
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
MFMA_AGPR_WAIT = 19
ACC_READ = re.compile(r"^v_accvgpr_read_b32\s+v\d+,\s*a(\d+)")
MFMA_DEF = re.compile(r"^v_mfma_\w+\s+a\[(\d+):(\d+)\]")


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


def vregs(text):
    out = set()
    for m in re.finditer(r"\bv\[(\d+):(\d+)\]", text):
        out.update(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"\bv(\d+)\b", text):
        out.add(int(m.group(1)))
    return out


def scan(path):
    findings = []
    func = "?"
    in_asm = False
    hist = []  # (instruction, from inline asm, source line number), oldest first, of the current function
    flying = {}  # vector register -> [line of its uncounted load, vector-memory instructions issued since, retired]

    pending_checks = []  # indices into hist of the inline-assembly memory instructions of the current function
    acc_checks = []      # and of its inline-assembly accumulator reads

    def check_operands():
        """Walks upwards from every inline-assembly memory instruction, through the function's jumps as well."""
        jumps = {}
        for i, (pins, _, _) in enumerate(hist):
            m = re.match(r"^s_c?branch\w*\s+(\.LBB\w+)", pins)
            if m:
                jumps.setdefault(m.group(1), []).append(i)
        for at in pending_checks:
            ins, _, ln = hist[at]
            ops = ins.split(None, 1)[1] if " " in ins else ""
            used = sregs(ops)
            lds_dma = bool(re.search(r"\blds\b", ops))
            seen = set()
            stack = [(at - 1, 0)]
            while stack:
                i, dist = stack.pop()
                arrived_by_jump = i != at - 1
                while i >= 0 and dist < VMEM_SGPR_WAIT and (i, dist) not in seen:
                    seen.add((i, dist))
                    pins, _, pln = hist[i]
                    if re.match(r"^s_branch\b", pins) and not arrived_by_jump:
                        break  # nothing falls through an unconditional jump
                    arrived_by_jump = False
                    if pins.startswith("<label> "):
                        for j in jumps.get(pins[8:], []):
                            stack.append((j, dist))  # the jump itself is one wait state: counted when it is visited
                        i -= 1  # and the line above the label
                        continue
                    hit = valu_sgpr_defs(pins) & used
                    if hit:
                        findings.append(f"{path}:{ln}: {func}: '{ins}' reads s{sorted(hit)} {dist} wait states after "
                                        f"'{pins}' (line {pln}); {VMEM_SGPR_WAIT} needed")
                    if lds_dma and dist < M0_LDS_WAIT and re.match(r"^s_\w+\s+m0\b", pins):
                        findings.append(f"{path}:{ln}: {func}: '{ins}' reads m0 {dist} wait states after '{pins}'")
                    dist += wait_states(pins)
                    i -= 1
        pending_checks.clear()
        # accumulator reads from inline assembly: straight up the lines (these sit in straight-line epilogue code)
        for at in acc_checks:
            ins, _, ln = hist[at]
            reg = int(ACC_READ.match(ins).group(1))
            dist, i = 0, at - 1
            while i >= 0 and dist < MFMA_AGPR_WAIT:
                pins, _, pln = hist[i]
                m = MFMA_DEF.match(pins)
                if m and int(m.group(1)) <= reg <= int(m.group(2)):
                    findings.append(f"{path}:{ln}: {func}: '{ins}' {dist} wait states after '{pins[:60]}' (line {pln}); "
                                    f"{MFMA_AGPR_WAIT} needed")
                    break
                if not pins.startswith("<label> "):
                    dist += wait_states(pins)
                i -= 1
        acc_checks.clear()

    def close_function():
        check_operands()
        for reg, (lln, _, _) in flying.items():
            findings.append(f"{path}:{lln}: {func}: uncounted load into v{reg} is never taken into use (ix_landed)")
        flying.clear()

    for ln, raw in enumerate(open(path), 1):
        s = raw.strip()
        m = re.match(r"^;\s*ix_landed\s+v(\d+)", s)
        if in_asm and m:
            reg = int(m.group(1))
            if reg not in flying:
                findings.append(f"{path}:{ln}: {func}: ix_landed v{reg} without an uncounted load into it on the lines above")
            else:
                if not flying[reg][2]:
                    findings.append(f"{path}:{ln}: {func}: v{reg} taken into use, but no wait since its load (line "
                                    f"{flying[reg][0]}) has retired it")
                del flying[reg]
            continue
        if s.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if s.startswith(";;#ASMEND"):
            in_asm = False
            continue
        m = re.match(r"^([A-Za-z_][\w$.]*):\s*(;.*)?$", raw)
        if m and not raw.startswith(".L"):
            close_function()
            func = m.group(1)
            hist = []
            continue
        m = re.match(r"^(\.LBB\w+):", raw)
        if m:
            for reg, st in flying.items():
                findings.append(f"{path}:{ln}: {func}: label {m.group(1)} between the uncounted load into v{reg} (line "
                                f"{st[0]}) and its ix_landed: not straight-line code, the in-flight rule cannot be judged")
            hist.append(("<label> " + m.group(1), False, ln))
            continue
        if not raw.startswith("\t") or s.startswith(";") or s.startswith("."):
            continue
        ins = s.split(";")[0].strip()
        if not ins:
            continue
        # uncounted loads in flight: nobody touches the register, and a wait has to retire it
        touched = vregs(ins)
        for reg in list(flying):
            if reg in touched:
                findings.append(f"{path}:{ln}: {func}: '{ins}' touches v{reg} while the uncounted load of line "
                                f"{flying[reg][0]} is in flight")
        if re.match(r"^s_c?branch|^s_setpc|^s_swappc|^s_call", ins):
            for reg, st in flying.items():
                findings.append(f"{path}:{ln}: {func}: '{ins}' between the uncounted load into v{reg} (line {st[0]}) and "
                                f"its ix_landed: not straight-line code, the in-flight rule cannot be judged")
        m = re.match(r"^s_waitcnt\b.*\bvmcnt\((\d+)\)", ins)
        if m:
            for st in flying.values():
                if int(m.group(1)) <= st[1]:
                    st[2] = True
        if VMEM.match(ins):
            for st in flying.values():
                st[1] += 1
            m = re.match(r"^global_load_dword\s+v(\d+),", ins)
            if in_asm and m:
                flying[int(m.group(1))] = [ln, 0, False]
        if in_asm and ACC_READ.match(ins):
            acc_checks.append(len(hist))
        if in_asm and VMEM.match(ins):
            pending_checks.append(len(hist))  # checked when the function is complete (its jumps are known then)
        hist.append((ins, in_asm, ln))
    close_function()
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
