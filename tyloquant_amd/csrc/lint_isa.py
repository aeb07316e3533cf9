#!/usr/bin/env python3
"""Checks the gfx950 assembly of the kernels for the two hazards their inline-assembly dot products can run into.

The DPP dot products (v_dot2c_f32_f16_dpp ... row_newbcast) are written as inline assembly, so the compiler's hazard
recognizer does not know what they are.  Two rules of the target then rest on the source code alone:

  1. a VGPR written by a vector-ALU instruction may be read through DPP only two issue slots later;
  2. the result of a dot instruction may feed the accumulator of the same dot opcode at once, but any other
     instruction that reads it has to stay three issue slots behind.

This script reads the device assembly the build keeps (one .s per source file) and fails on either pattern, whichever
way it came about (instruction scheduling, a register copy the allocator put in).  s_nop N counts as N + 1 slots.
Usage: lint_isa.py file.s [...]
"""
import re
import sys

DPP = re.compile(r"^(v_\w+_dpp)\s+(v\d+|v\[\d+:\d+\]),\s*(v\d+)")
DOT = re.compile(r"^(v_dot\w+)\s+(v\d+),")
VALU_DST = re.compile(r"^v_\w+\s+(v\d+|v\[(\d+):(\d+)\])")
REG = re.compile(r"\bv(\d+)\b|\bv\[(\d+):(\d+)\]")


def regs_of(text):
    out = set()
    for m in REG.finditer(text):
        if m.group(1) is not None:
            out.add(int(m.group(1)))
        else:
            out.update(range(int(m.group(2)), int(m.group(3)) + 1))
    return out


def written(line):
    m = VALU_DST.match(line)
    if not m or line.startswith("v_cmp") or line.startswith("v_readlane") or line.startswith("v_readfirstlane"):
        return set()
    return regs_of(m.group(1))


def lint(path):
    errors = []
    kernel = "?"
    window = []  # (slots_ago_base, line) of recent instructions, newest last
    for raw in open(path):
        line = raw.split(";")[0].strip()
        if line.endswith(":") and line.startswith("_Z"):
            kernel = line.rstrip(":")
            window = []
            continue
        if not line or line.startswith((".", "//")) or line.endswith(":"):
            continue
        nop = re.match(r"^s_nop\s+(\d+)", line)
        slots = int(nop.group(1)) + 1 if nop else 1
        # rule 1: the DPP source of this instruction against vector-ALU writes in the two slots before it
        m = DPP.match(line)
        if m:
            src = int(m.group(3)[1:])
            dist = 0
            for s_, prev in reversed(window):
                if dist >= 2:
                    break
                if src in written(prev):
                    errors.append(f"{path}: {kernel}: DPP source v{src} written {dist} slot(s) before: '{prev}' -> '{line}'")
                dist += s_
        # rule 2: readers of a dot result within three slots (the same opcode accumulating into it is exempt)
        dist = 0
        for s_, prev in reversed(window):
            if dist >= 3:
                break
            d = DOT.match(prev)
            if d:
                dst = int(d.group(2)[1:])
                mine = DOT.match(line)
                same_acc = mine and mine.group(1).replace("_dpp", "") == d.group(1).replace("_dpp", "") and int(mine.group(2)[1:]) == dst
                operands = line.split(None, 1)[1] if " " in line else ""
                reads = regs_of(operands.split(",", 1)[1]) if "," in operands and line.startswith("v_") else regs_of(operands)
                if same_acc:
                    reads = regs_of(",".join(operands.split(",")[1:])) - {dst} if dst not in regs_of(",".join(operands.split(",")[1:3])) else {dst}
                    if dst in reads:
                        errors.append(f"{path}: {kernel}: dot result v{dst} read as a source {dist} slot(s) later: '{prev}' -> '{line}'")
                elif dst in reads and not line.startswith("s_"):
                    errors.append(f"{path}: {kernel}: dot result v{dst} read {dist} slot(s) later: '{prev}' -> '{line}'")
            dist += s_
        window.append((slots, line))
        if len(window) > 8:
            window.pop(0)
    return errors


def main():
    bad = []
    for p in sys.argv[1:]:
        bad += lint(p)
    for e in bad[:40]:
        print(e)
    if bad:
        print(f"lint_isa: {len(bad)} hazard(s)")
        return 1
    print(f"lint_isa: {len(sys.argv) - 1} file(s) clean")
    return 0


if __name__ == "__main__":
    sys.exit(main())
