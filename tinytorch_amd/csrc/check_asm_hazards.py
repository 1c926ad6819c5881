#!/usr/bin/env python3
"""Scans the compiler's assembly listing of a kernel source for a hazard that its asm statements can create.

    python3 check_asm_hazards.py file.s [file.s ...]      (exit status 1 if any is found)

On gfx9-family chips a scalar register written by a vector instruction (v_readlane of a spilled scalar register,
v_readfirstlane) may be read as the address of a vector-memory instruction only five wait states later.  The compiler
inserts the wait states itself for its own instructions, but its hazard pass does not look into asm statements: a
`global_load ... , s[n:n+1]` at the start of a statement, right behind the restore of s[n:n+1], reads the old value.
The direct global->LDS loads and the Q loads of the kernels here are such statements; they carry `s_nop`s of their
own, and this check holds every listing to it.
"""
import re
import sys


def sregs(text):
    out = set()
    for m in re.finditer(r"\bs(\d+)\b|s\[(\d+):(\d+)\]", text):
        if m.group(1):
            out.add(int(m.group(1)))
        else:
            out.update(range(int(m.group(2)), int(m.group(3)) + 1))
    return out


def scan(path):
    ins = []
    for i, line in enumerate(open(path).read().split("\n")):
        t = line.split(";")[0].strip()
        if t and not t.endswith(":") and not t.startswith("."):
            ins.append((i + 1, t))
    found = []
    for k, (i, t) in enumerate(ins):
        if not (t.startswith("v_readlane") or t.startswith("v_readfirstlane")):
            continue
        dst = sregs(t.split(",")[0])
        waited = 0
        for j, u in ins[k + 1:k + 12]:
            if u.startswith("s_nop"):
                waited += int(u.split()[1]) + 1
            else:
                if u.split("_")[0] in ("global", "buffer", "flat", "scratch") and waited < 5:
                    if sregs(u.split(None, 1)[1] if " " in u else "") & dst:
                        found.append("%s:%d: %s  ->  line %d: %s  (%d wait states)" % (path, i, t, j, u, waited))
                waited += 1
            if waited >= 5:
                break
    return found


def main():
    found = []
    for path in sys.argv[1:]:
        found += scan(path)
    for f in found:
        print(f)
    print("%d hazard(s)" % len(found))
    return 1 if found else 0


if __name__ == "__main__":
    sys.exit(main())
