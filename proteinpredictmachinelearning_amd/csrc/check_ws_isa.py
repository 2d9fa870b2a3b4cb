#!/usr/bin/env python3
"""Build step: checks the gfx950 assembly of q8.hip before the object is linked.

The weight-stationary Q8 kernels keep the activation tile in flight in VGPRs that only inline
assembly names (the top 16/32/64 of the wave's register budget).  The register allocator is kept
out of them by a kernel attribute, but two things can still put compiler-owned data there, and
either one ends in corrupted addresses and a memory fault on the GPU:

  * scalar-register spills: they go into lanes of a VGPR the compiler picks outside the budget
    (v_writelane_b32 / v_readlane_b32);
  * a change of the attribute's meaning between compiler versions.

So for every fast instance (template argument DUMP = false) this script requires: no lane
spills, no scratch memory, no compiler-written instruction naming a staging register, and a
kernel descriptor that gives the wave its whole register budget.  The
diagnostic instances (DUMP = true) must not contain the staging loads at all.

usage: check_ws_isa.py <q8 device assembly (.s)>     exit status 0 = all kernels pass
"""
import re
import sys

KERNEL = re.compile(r"^(_ZN\S*?(q8_linear_ws(\d*)_kernel)ILi(\d+)ELi(\d+)ELi(\d+)ELi(\d+)ELb([01])E\S*):")
VREG = re.compile(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b")
STAGING_BY_NAME = {"": 16, "32": 32, "64": 64}      # q8_linear_ws<suffix>_kernel
BUDGET_BY_NAME = {"": 256, "32": 256, "64": 256}   # registers of one wave


def check(path):
    lines = open(path).read().split("\n")
    problems, seen = [], 0
    i = 0
    while i < len(lines):
        m = KERNEL.match(lines[i])
        if not m:
            i += 1
            continue
        suffix, dump = m.group(3), m.group(8) == "1"
        label = "%s<%s,%s,%s,%s,%s>" % (m.group(2), m.group(4), m.group(5), m.group(6), m.group(7), "true" if dump else "false")
        stage0 = BUDGET_BY_NAME[suffix] - STAGING_BY_NAME[suffix]
        seen += 1
        in_asm = False
        owned = 0                      # from the kernel descriptor, which sits between the code and .Lfunc_end
        i += 1
        while i < len(lines) and ".Lfunc_end" not in lines[i]:
            if ".amdhsa_next_free_vgpr" in lines[i]:
                owned = int(lines[i].split()[-1])
            text = lines[i].split(";")[0].strip() if "ASM" not in lines[i] else lines[i]
            if "ASMSTART" in text:
                in_asm = True
            elif "ASMEND" in text:
                in_asm = False
            elif text:
                if in_asm:
                    if dump and text.startswith("global_load"):
                        problems.append("%s: diagnostic instance contains a staging load: %s" % (label, text))
                elif not dump:
                    if "v_writelane" in text or "v_readlane" in text:
                        problems.append("%s: scalar spill into a vector register: %s" % (label, text))
                    if text.startswith("scratch_"):
                        problems.append("%s: scratch memory in a fast instance: %s" % (label, text))
                    for r in VREG.finditer(text):
                        hi = int(r.group(2) or r.group(3))
                        if hi >= stage0:
                            problems.append("%s: compiler code names staging register v%d: %s" % (label, hi, text))
            i += 1
        if not dump and owned < BUDGET_BY_NAME[suffix]:
            problems.append("%s: the wave owns %d registers, the staging needs %d" % (label, owned, BUDGET_BY_NAME[suffix]))
    if seen == 0:
        problems.append("no q8_linear_ws kernel found in %s" % path)
    return seen, problems


if __name__ == "__main__":
    n, bad = check(sys.argv[1])
    for p in bad[:40]:
        print("check_ws_isa: " + p, file=sys.stderr)
    if bad:
        print("check_ws_isa: %d problem(s) in %d kernels" % (len(bad), n), file=sys.stderr)
        sys.exit(1)
    print("check_ws_isa: %d weight-stationary kernels pass" % n)
