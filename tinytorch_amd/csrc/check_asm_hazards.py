#!/usr/bin/env python3
"""Scans the compiler's assembly listing of a kernel source for a hazard that its asm statements can create.

    python3 check_asm_hazards.py file.s [file.s ...]      (exit status 1 if anything is found)

On gfx9-family chips a scalar register written by a vector instruction (v_readlane of a spilled scalar register,
v_readfirstlane, a compare with a scalar destination) may be read as the address of a vector-memory instruction only
five wait states later.  The compiler inserts the wait states itself for its own instructions, but its hazard pass does
not look into asm statements: a `global_load ... , s[n:n+1]` at the start of a statement, right behind the restore of
s[n:n+1], reads the old value.  The direct global->LDS loads and the Q loads of the kernels here are such statements;
they carry `s_nop`s of their own, and this check holds every listing to it.

Two passes over a listing:
  1. forward from every vector instruction that writes scalar registers: a vector-memory instruction (asm-issued or
     not) that reads one of them within five wait states is reported;
  2. every instruction between the compiler's `;;#ASMSTART` / `;;#ASMEND` markers is classified.  A vector-memory
     instruction with a scalar base must have five wait states of instructions behind it that provably do not write its
     base (a label, a branch or the start of the function inside that window ends the proof: reported).  A scalar-memory
     instruction, or a mnemonic this script does not know, is reported as unclassified: nothing asm-issued passes
     because a pattern failed to match it.
"""
import re
import sys

VMEM = ("global_", "buffer_", "flat_", "scratch_", "tbuffer_")
# what an asm statement may hold besides vector-memory instructions: vector ALU / matrix, LDS, scalar ALU and control
PLAIN = ("v_", "ds_", "s_")
SMEM = ("s_load", "s_buffer_load", "s_store", "s_buffer_store", "s_scratch_", "s_atomic", "s_buffer_atomic", "s_dcache")
WAIT_STATES = 5


def sregs(text):
    out = set()
    for m in re.finditer(r"\bs(\d+)\b|\bs\[(\d+):(\d+)\]", text):
        if m.group(1):
            out.add(int(m.group(1)))
        else:
            out.update(range(int(m.group(2)), int(m.group(3)) + 1))
    return out


def operands(ins):
    return ins.split(None, 1)[1] if " " in ins else ""


def scalar_dests(ins):
    """Scalar registers a vector instruction writes (none for anything else)."""
    if not ins.startswith("v_"):
        return set()
    ops = [o.strip() for o in operands(ins).split(",")]
    dst = sregs(ops[0]) if ops else set()
    if "_co_" in ins and len(ops) > 1:  # carry-out in the second operand
        dst |= sregs(ops[1])
    return dst


def cost(ins):
    return int(ins.split()[1]) + 1 if ins.startswith("s_nop") else 1


def parse(path):
    """-> list of (line number, text, issued by an asm statement); labels are kept as text ending in ':'."""
    ins, in_asm = [], False
    for i, line in enumerate(open(path).read().split("\n")):
        if "#ASMSTART" in line:
            in_asm = True
            continue
        if "#ASMEND" in line:
            in_asm = False
            continue
        t = line.split(";")[0].strip()
        if not t or t.startswith(".") and not t.endswith(":"):
            continue
        ins.append((i + 1, t, in_asm))
    return ins


def scan(path):
    ins = parse(path)
    found = []
    # pass 1: forward from scalar writes by vector instructions
    for k, (i, t, _) in enumerate(ins):
        dst = scalar_dests(t)
        if not dst:
            continue
        waited = 0
        for j, u, _ in ins[k + 1:k + 12]:
            if u.endswith(":"):
                continue
            if u.startswith(VMEM) and waited < WAIT_STATES and sregs(operands(u)) & dst:
                found.append("%s:%d: %s  ->  line %d: %s  (%d wait states)" % (path, i, t, j, u, waited))
            waited += cost(u)
            if waited >= WAIT_STATES:
                break
    # pass 2: everything an asm statement issues
    for k, (i, t, in_asm) in enumerate(ins):
        if not in_asm or t.endswith(":"):
            continue
        if t.startswith(SMEM):
            found.append("%s:%d: %s  (asm-issued scalar-memory instruction: unclassified)" % (path, i, t))
            continue
        if t.startswith(VMEM):
            base = sregs(operands(t))
            if not base:
                continue
            waited, proven = 0, False
            for j, u, _ in reversed(ins[max(0, k - 16):k]):
                if u.endswith(":") or u.startswith(("s_cbranch", "s_branch", "s_setpc", "s_swappc", "s_endpgm")):
                    break  # other paths may lead here: nothing is known about what ran before
                if scalar_dests(u) & base:
                    break
                waited += cost(u)
                if waited >= WAIT_STATES:
                    proven = True
                    break
            if not proven:
                found.append("%s:%d: %s  (scalar base %s: only %d wait states provably free of a vector write)"
                             % (path, i, t, sorted(base), waited))
            continue
        if not t.startswith(PLAIN):
            found.append("%s:%d: %s  (asm-issued instruction this check cannot classify)" % (path, i, t))
    return found


def main():
    found = []
    for path in sys.argv[1:]:
        found += scan(path)
    for f in found:
        print(f)
    print("%d finding(s)" % len(found))
    return 1 if found else 0


if __name__ == "__main__":
    sys.exit(main())
