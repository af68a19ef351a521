"""Checks the generated code of evoattn_bwd_pw.hip and evoattn_bwd_dbias_ring.hip for hazards the compiler cannot see.

These kernels issue their MFMAs as inline assembly, so the compiler neither inserts the idle cycles gfx950
requires around them nor keeps their operands alive long enough.  This script reads the assembly text the
compiler produced (``hipcc -S``) and verifies, for every MFMA inside an ``#ASMSTART`` / ``#ASMEND`` pair:

1. no vector-ALU instruction in the two preceding issue slots writes a register the MFMA reads
   (A, B or C operand);
2. no instruction in the 13 following issue slots writes a register of the MFMA's C operand when C is not
   also its destination (the matrix pipe reads C while the product runs);
3. an MFMA whose destination is a vector register (``v[...]``) is followed by at least 12 issue slots,
   at least two of them MFMAs or idle instructions (or by 24 slots of any kind), before any other
   instruction reads that destination;
4. an MFMA whose destination is an accumulation register is followed by at least 18 issue slots before an
   instruction other than an MFMA (an LDS store, a move to a vector register) reads that destination.

It is run by ``megafold_amd.build`` after compiling; a violation fails the build.

    python check_pw_hazards.py file.s
"""
from __future__ import annotations

import re
import sys

REG = re.compile(r"\b([va])\[(\d+):(\d+)\]|\b([va])(\d+)\b")


def regs(text: str) -> set[tuple[str, int]]:
    out = set()
    for m in REG.finditer(text):
        if m.group(1):
            out.update((m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1))
        else:
            out.add((m.group(4), int(m.group(5))))
    return out


def parse(line: str):
    """(mnemonic, written registers, read registers) of one instruction line, or None."""
    line = line.split(";")[0].strip()
    if not line or line.startswith(".") or line.endswith(":"):
        return None
    parts = line.split(None, 1)
    mnem = parts[0]
    ops = [o.strip() for o in parts[1].split(",")] if len(parts) > 1 else []
    if mnem.startswith(("s_", "buffer_", "scratch_")) and not mnem.startswith("s_nop"):
        return mnem, set(), regs(" ".join(ops))
    if mnem.startswith(("ds_write", "global_store", "ds_store")):
        return mnem, set(), regs(" ".join(ops))
    if not ops:
        return mnem, set(), set()
    return mnem, regs(ops[0]), regs(" ".join(ops[1:]))


def slots(mnem: str, line: str) -> int:
    """Issue slots an instruction accounts for (s_nop N idles N + 1)."""
    if mnem == "s_nop":
        return int(line.split()[1], 0) + 1
    return 1


def check(path: str) -> list[str]:
    errors = []
    kernel = "?"
    insts = []   # (mnem, writes, reads, in_asm, text, lineno)
    in_asm = False
    for no, raw in enumerate(open(path), 1):
        m = re.match(r"^(_Z\w+):", raw)
        if m:
            if insts:
                errors += check_kernel(kernel, insts)
            kernel, insts = m.group(1), []
            continue
        if "#ASMSTART" in raw:
            in_asm = True
            continue
        if "#ASMEND" in raw:
            in_asm = False
            continue
        lab = re.match(r"^(\.LBB\w+):", raw)
        if lab:
            insts.append(("label", set(), set(), False, lab.group(1), no))
            continue
        p = parse(raw)
        if p:
            insts.append((p[0], p[1], p[2], in_asm, raw.strip(), no))
    if insts:
        errors += check_kernel(kernel, insts)
    return errors


N_CHECKED = [0]
# kernels (substrings of the mangled names) whose inline-assembly MFMAs are checked
CHECKED_KERNELS = ("dqkv_pw", "dbias_ring")


def paths(insts, i, limit):
    """Every instruction sequence that can follow position i, as lists of (instruction, issue slots that separate
    it from position i): at a conditional branch to a later label both continuations are followed.  A sequence ends
    after `limit` slots, at a backward or unconditional branch, or at the end of the program."""
    labels = {t: k for k, (m, _, _, _, t, _) in enumerate(insts) if m == "label"}
    out = []
    todo = [(i + 1, 0, [])]
    while todo:
        j, fwd, seq = todo.pop()
        seq = list(seq)
        while j < len(insts) and fwd < limit:
            m2, w2, r2, a2, t2, n2 = insts[j]
            if m2 == "label":
                j += 1
                continue
            if m2 in ("s_branch", "s_endpgm", "s_setpc_b64"):
                break
            if m2.startswith("s_cbranch"):
                target = labels.get(t2.split()[-1])
                if target is None or target <= j:
                    break
                if len(todo) < 64:
                    todo.append((target, fwd, list(seq)))
                j += 1
                continue
            seq.append((insts[j], fwd))
            fwd += slots(m2, t2)
            j += 1
        out.append(seq)
    return out


def check_kernel(kernel: str, insts) -> list[str]:
    errors = []
    if not any(name in kernel for name in CHECKED_KERNELS):
        return errors
    for i, (mnem, wr, rd, in_asm, text, no) in enumerate(insts):
        if not (in_asm and mnem.startswith("v_mfma")):
            continue
        N_CHECKED[0] += 1
        found = set()      # two paths may report the same instruction
        ops = [o.strip() for o in text.split(None, 1)[1].split(",")]
        dst, srcc = regs(ops[0]), regs(ops[3]) if len(ops) > 3 else set()
        # 1. vector-ALU writes of operands in the two preceding slots
        back, j = 0, i - 1
        while j >= 0 and back < 2:
            m2, w2, r2, a2, t2, n2 = insts[j]
            if m2 == "label":      # another path may join here: stop, the MFMA's own leading idle slots cover it
                break
            if m2.startswith("v_") and not m2.startswith("v_mfma") and (w2 & rd):
                errors.append("%s: line %d `%s` writes an operand of the MFMA at line %d within 2 slots" % (kernel, n2, t2, no))
            back += slots(m2, t2)
            j -= 1
        # 2. C operand rewritten while the product runs
        if srcc and srcc != dst:
            for seq in paths(insts, i, 13):
                for (m2, w2, r2, a2, t2, n2), fwd in seq:
                    if w2 & srcc:
                        found.add("%s: line %d `%s` rewrites the C operand of the MFMA at line %d after %d slots" % (kernel, n2, t2, no, fwd))
        # 3. vector-register result read too early (12 slots, two of them MFMAs or idle instructions; 24 slots
        #    of any kind are as good).  A register that another instruction has rewritten no longer holds the result.
        if any(k == "v" for k, _ in dst):
            for seq in paths(insts, i, 26):
                busy, live = 0, set(dst)
                for (m2, w2, r2, a2, t2, n2), fwd in seq:
                    if (fwd >= 12 and busy >= 2) or fwd >= 24 or not live:
                        break
                    if (r2 & live) and not m2.startswith("v_mfma"):
                        found.add("%s: line %d `%s` reads the result of the MFMA at line %d after %d slots" % (kernel, n2, t2, no, fwd))
                        break
                    if not m2.startswith("v_mfma"):
                        if (w2 & live) and fwd < 12:
                            found.add("%s: line %d `%s` overwrites the result of the MFMA at line %d after %d slots" % (kernel, n2, t2, no, fwd))
                            break
                        live -= w2
                    if m2.startswith("v_mfma") or m2 == "s_nop":
                        busy += 1
        # 4. accumulation-register result read by something other than an MFMA
        if any(k == "a" for k, _ in dst):
            for seq in paths(insts, i, 18):
                for (m2, w2, r2, a2, t2, n2), fwd in seq:
                    if (r2 & dst) and not m2.startswith("v_mfma"):
                        found.add("%s: line %d `%s` reads the result of the MFMA at line %d after %d slots" % (kernel, n2, t2, no, fwd))
                        break
        errors += sorted(found)
    return errors


if __name__ == "__main__":
    errs = check(sys.argv[1])
    print("%d MFMAs in inline assembly checked" % N_CHECKED[0])
    for e in errs[:40]:
        print(e)
    print("%d hazard(s)" % len(errs))
    sys.exit(1 if errs else 0)
