"""Reads the assembly hipcc writes for a kernel file (`-S`) and checks the distance the hardware wants
between an inline-assembly MFMA and the first other instruction that touches its result registers.

The kernels issue some MFMA chains through inline assembly (accumulators in vector registers where
the vector ALU reads them in place).  The compiler does not know what the assembly is and inserts no
wait states behind it, so the distance is kept by the order of the source - and checked here, on the
instruction stream the compiler actually produced, for every path through the kernel."""

import collections
import re

REG = re.compile(r"\bv(\d+)\b|\bv\[(\d+):(\d+)\]")

def vregs(text):
    out = set()
    for m in REG.finditer(text):
        if m.group(1) is not None:
            out.add(int(m.group(1)))
        else:
            out.update(range(int(m.group(2)), int(m.group(3)) + 1))
    return out

def split_functions(asm):
    """name -> list of instruction / label lines of each kernel in a -S output."""
    funcs, name, cur, in_asm = {}, None, None, False
    for line in asm.splitlines():
        mark = line.strip()
        if mark.startswith(";;#ASMSTART"):
            in_asm = True
        elif mark.startswith(";;#ASMEND"):
            in_asm = False
        s = line.split(";")[0].rstrip()
        if not s.strip():
            continue
        m = re.match(r"^(_Z\w+):", s)
        if m:
            name, cur = m.group(1), []
            funcs[name] = cur
            continue
        if cur is None:
            continue
        t = s.strip()
        if t.startswith(".") and not t.endswith(":"):
            if t.startswith(".Lfunc_end"):
                cur = None
            continue
        cur.append(("@" if in_asm else "") + t)  # "@": written by inline assembly
    return funcs

def check_function(lines, need_mfma=2, need_nops=12):
    """Every inline-assembly MFMA that leaves its result in vector registers: on every path from it, the
    first instruction other than the continuation of its own chain that touches those registers comes
    after at least `need_mfma` further MFMAs (the matrix pipe takes them one after the other, 8 passes
    each) or `need_nops` wait states (one per instruction issued, N + 1 for s_nop N; an 8-pass MFMA
    needs 11 before a vector ALU instruction may read or overwrite its result).  Returns the violations."""
    from_asm = [l.startswith("@") for l in lines]
    lines = [l.lstrip("@") for l in lines]
    labels = {l[:-1]: i for i, l in enumerate(lines) if l.endswith(":")}
    bad = []
    for i, ins in enumerate(lines):
        if not from_asm[i] or not ins.startswith("v_mfma_"):
            continue  # the compiler's own MFMAs get the compiler's own hazard handling
        ops = [o.strip() for o in ins.split(None, 1)[1].split(",")]
        dst = ops[0]
        if not dst.startswith("v"):
            continue  # accumulator registers: only MFMAs and v_accvgpr moves touch them, the compiler's domain
        R = vregs(dst)
        seen = set()
        todo = collections.deque([(i + 1, 0, 0)])
        while todo:
            pc, nm, nn = todo.popleft()
            while pc < len(lines):
                key = (pc, nm, min(nn, need_nops))
                if key in seen:
                    break
                seen.add(key)
                x = lines[pc]
                if x.endswith(":"):
                    pc += 1
                    continue
                op = x.split()[0]
                if op.startswith("v_mfma_"):
                    o2 = [o.strip() for o in x.split(None, 1)[1].split(",")]
                    if vregs(o2[1]) & R or vregs(o2[2]) & R:
                        if nm < need_mfma and nn < need_nops:
                            bad.append((i, ins, pc, x, nm, nn))
                        break
                    if vregs(o2[0]) & R:
                        break  # the chain goes on (or a new one starts in these registers): the matrix pipe orders them
                    nm += 1
                    nn += 1
                    if nm >= need_mfma or nn >= need_nops:
                        break
                    pc += 1
                    continue
                if op == "s_nop":
                    nn += int(x.split()[1], 0) + 1
                    if nn >= need_nops:
                        break
                    pc += 1
                    continue
                if vregs(x.split(None, 1)[1] if " " in x else "") & R:
                    bad.append((i, ins, pc, x, nm, nn))
                    break
                nn += 1
                if nn >= need_nops:
                    break
                if op == "s_endpgm":
                    break
                if op == "s_branch":
                    pc = labels[x.split()[1]]
                    continue
                if op.startswith("s_cbranch"):
                    todo.append((labels[x.split()[1]], nm, nn))
                pc += 1
    return bad


def check_sources(lines, need=8):
    """Every inline-assembly MFMA: none of its vector-register operands (the two factors and the addend)
    is written by a vector ALU instruction within `need` wait states before it, counted back along the
    instruction stream (labels are walked through as fall-through: a branch into the stretch can only
    come from further away).  The hardware wants a distance between such a write and a matrix
    instruction that reads the register; for its own MFMAs the compiler keeps it, behind a register that
    assembly reads it does not.  Loads (LDS, global) are not meant here: the compiler waits for them
    before the assembly statement that names their register.  Returns the violations."""
    from_asm = [l.startswith("@") for l in lines]
    lines = [l.lstrip("@") for l in lines]
    bad = []
    for i, ins in enumerate(lines):
        if not from_asm[i] or not ins.startswith("v_mfma_"):
            continue
        ops = [o.strip() for o in ins.split(None, 1)[1].split(",")]
        R = vregs(ops[1]) | vregs(ops[2]) | vregs(ops[3])
        waited, j = 0, i - 1
        while j >= 0 and waited < need:
            x = lines[j]
            j -= 1
            if x.endswith(":"):
                continue
            op = x.split()[0]
            if op == "s_nop":
                waited += int(x.split()[1], 0) + 1
                continue
            if op.startswith("v_") and not op.startswith("v_mfma_") and not op.startswith("v_cmp"):
                if vregs(x.split(None, 1)[1].split(",")[0]) & R:
                    bad.append((i, ins, j + 1, x, waited))
                    break
            waited += 1
    return bad
