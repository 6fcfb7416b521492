#!/usr/bin/env python3
"""Hazard check for the hand-written DPP instructions of the GEMM kernels.

fmac_row_lane (ckq_gemm_common.hpp) emits v_fmac_f32_dpp from inline assembly,
which the compiler's hazard recogniser does not look into.  On gfx9 a DPP
instruction must not read a VGPR that a VALU instruction wrote in the two
wait states before it, nor follow a VALU write of EXEC (v_cmpx) by fewer than
five (writes of EXEC by scalar instructions are forwarded and need none).  This
script reads the device assembly of the given files (hipcc -S) and fails if
either distance is violated anywhere; `make check` runs it on every GEMM
translation unit, product and dump flavour.
"""
import re
import sys


def instructions(path):
    out = []
    for line in open(path):
        if not line.startswith("\t"):
            continue
        t = line.strip()
        if not t or t[0] in ".;" or t.startswith("//"):
            continue
        out.append(t.split(";")[0].strip())
    return out


def regs(operand):
    """Set of VGPR numbers an operand like v12 or v[4:7] names."""
    m = re.fullmatch(r"v(\d+)", operand)
    if m:
        return {int(m.group(1))}
    m = re.fullmatch(r"v\[(\d+):(\d+)\]", operand)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    return set()


def wait_states(ins):
    m = re.fullmatch(r"s_nop\s+(\d+)", ins)
    return int(m.group(1)) + 1 if m else 1


def check(path):
    ins = instructions(path)
    bad = 0
    count = 0
    for i, t in enumerate(ins):
        op = t.split()[0]
        if not op.endswith("_dpp"):
            continue
        count += 1
        operands = [o.strip() for o in t[len(op):].split(",")]
        src = regs(operands[1].split()[0]) if len(operands) > 1 else set()
        dist = 0
        for k in range(1, 8):
            if i - k < 0:
                break
            p = ins[i - k]
            pop = p.split()[0]
            if dist < 2 and pop.startswith("v_") and not pop.startswith("v_mfma"):
                dst = regs(p[len(pop):].split(",")[0].strip())
                if dst & src:
                    print("%s: VALU write %r within two wait states of %r" % (path, p, t))
                    bad += 1
            if dist < 5 and pop.startswith("v_") and (pop.startswith("v_cmpx") or re.search(r"\bexec(_lo|_hi)?\b", p.split(",")[0])):
                print("%s: EXEC write %r within five wait states of %r" % (path, p, t))
                bad += 1
            dist += wait_states(p)
            if dist >= 5:
                break
    return count, bad


def main(paths):
    total = bad = 0
    for p in paths:
        c, b = check(p)
        total += c
        bad += b
    print("check_dpp: %d DPP instructions in %d files, %d hazards" % (total, len(paths), bad))
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
