#!/usr/bin/env python3
"""Build-time check of the hand-placed LDS waits in gemm_mfma.hip.

The prefill GEMM issues its LDS reads as inline asm and waits for them with hand-placed `s_waitcnt lgkmcnt(N)`, so the
compiler believes a destination register holds its value as soon as the read has been issued.  A copy, a spill or any
other use that the compiler places between a read and the wait that covers it would pick up stale data without any
diagnostic.  This script walks the device assembly of the translation unit and fails the build if, in a kernel whose
name contains the given pattern,

  * an instruction reads or overwrites a register that an LDS read has not yet delivered (LDS operations of one wave
    return in order, so `s_waitcnt lgkmcnt(N)` completes all but the youngest N of them), or
  * the kernel uses scratch memory or spills registers (from the resource remarks, when a remark file is given).

usage: check_lds_waits.py <file.s> <kernel-name-pattern> [<file with -Rpass-analysis=kernel-resource-usage remarks>]

The walk is linear in text order, through labels and branches; at a backward branch the loop body is walked once more
with the state the branch leaves.  Scalar loads count in the same counter and may return out of order: any wait with a
scalar load outstanding is taken to complete the vector reads only when it is lgkmcnt(0).
"""
import re
import sys

REG = re.compile(r"\b([va])(\d+)\b|\b([va])\[(\d+):(\d+)\]")


def regs_of(text):
    out = set()
    for m in REG.finditer(text):
        if m.group(1):
            out.add((m.group(1), int(m.group(2))))
        else:
            for i in range(int(m.group(4)), int(m.group(5)) + 1):
                out.add((m.group(3), i))
    return out


def kernel_bodies(lines, pattern):
    """(name, [instruction lines]) per function whose label contains the pattern"""
    name, body = None, []
    for ln in lines:
        m = re.match(r"^([A-Za-z_][\w$.]*):", ln)
        if m and not m.group(1).startswith((".L", "BB")):
            if name and pattern in name:
                yield name, body
            name, body = m.group(1), []
            continue
        s = ln.split(";")[0].strip()
        if name and s and s.endswith(":"):
            body.append("LABEL " + s[:-1])
        elif name and s and not s.startswith("."):
            body.append(s)
        if name and s.startswith("s_endpgm"):
            if pattern in name:
                yield name, body
            name, body = None, []


def step(name, ins, state, errors):
    """one instruction; state = [pending, scalar_out]: pending holds, in issue order, the registers of every LDS read not
    yet waited for (an empty set for LDS writes and scalar loads)"""
    op, _, rest = ins.partition(" ")
    if op == "LABEL" or op.startswith("s_cbranch") or op == "s_branch":
        return
    if op == "s_waitcnt":
        m = re.search(r"lgkmcnt\((\d+)\)", rest)
        if m:
            n = int(m.group(1))
            if n == 0:
                state[0], state[1] = [], 0
            elif state[1] == 0 and len(state[0]) > n:
                state[0] = state[0][len(state[0]) - n:]
        return
    if op.startswith("s_load") or op.startswith("s_buffer_load"):
        state[1] += 1
        state[0].append(set())
        return
    operands = [o.strip() for o in rest.split(",")] if rest else []
    busy = set().union(*state[0]) if state[0] else set()
    hit = regs_of(rest) & busy
    if hit:
        errors.append(f"{name}: `{ins}` touches {sorted(hit)[:4]} before the LDS read into it is waited for")
        for p in state[0]:  # report each register once
            p -= hit
    if op.startswith("ds_read"):
        state[0].append(regs_of(operands[0]))
    elif op.startswith("ds_"):
        state[0].append(set())


def check_body(name, body):
    errors, state, labels = [], [[], 0], {}
    for i, ins in enumerate(body):
        op, _, rest = ins.partition(" ")
        if op == "LABEL":
            labels[rest] = i
        step(name, ins, state, errors)
        if (op.startswith("s_cbranch") or op == "s_branch") and rest.strip() in labels:
            again = [[set(p) for p in state[0]], state[1]]  # a second trip through the loop, from the branch's state
            for j in range(labels[rest.strip()], i):
                step(name, body[j], again, errors)
    return sorted(set(errors), key=errors.index)


def check_resources(path, pattern):
    errors, name = [], None
    for ln in open(path, errors="replace"):
        m = re.search(r"Function Name: (\S+)", ln)
        if m:
            name = m.group(1)
            continue
        if name is None or pattern not in name:
            continue
        m = re.search(r"(ScratchSize \[bytes/lane\]|SGPRs Spill|VGPRs Spill): (\d+)", ln)
        if m and int(m.group(2)) != 0:
            errors.append(f"{name}: {m.group(1)} = {m.group(2)} (must be 0: the LDS reads of this kernel are not visible to the compiler)")
    return errors


def main(argv):
    if len(argv) < 3:
        print(__doc__)
        return 2
    lines = open(argv[1], errors="replace").read().splitlines()
    errors, n = [], 0
    for name, body in kernel_bodies(lines, argv[2]):
        n += 1
        errors += check_body(name, body)
    if n == 0:
        errors.append(f"no kernel matching '{argv[2]}' in {argv[1]}")
    if len(argv) > 3:
        errors += check_resources(argv[3], argv[2])
    for e in errors[:40]:
        print("check_lds_waits:", e, file=sys.stderr)
    if errors:
        return 1
    print(f"check_lds_waits: {n} kernels of '{argv[2]}' clean")
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
