#!/usr/bin/env python3
"""Build-time guard for kernels that issue scalar loads from inline assembly and wait for them later.

    python3 check_async_sloads.py <assembly of the library's own source, hipcc -S> <kernel name substring>...

Such a kernel (fc_grad_input_kernel) requests `s_load_dwordx4` results a loop step ahead and waits for
them with one `s_waitcnt lgkmcnt(0)` (the only count that means anything for scalar loads, which return in
no fixed order).  The compiler does not know that the destination registers are
not valid in between, so register allocation alone decides whether that is safe: an instruction that
reads such a register before the wait (a copy, or the `v_writelane_b32` of a spill) would capture
stale data without any error.  This script follows the generated code of the named kernels along its
control flow and fails if

  * any instruction between a scalar load and the next `s_waitcnt lgkmcnt(0)` reads or overwrites a
    register that load is still writing, or
  * the kernel spills vector registers (scratch memory), which the hand-written loops do not allow for.

It reads compiler output of this library only (text produced by `hipcc -S --cuda-device-only`).
"""
import re
import sys

SLOAD = re.compile(r"^\s*s_(?:buffer_)?load_dword(?:x(\d+))?\s+s(?:\[(\d+):(\d+)\]|(\d+))\s*,")
WAIT_ALL = re.compile(r"^\s*s_waitcnt\b.*lgkmcnt\(0\)")
SREG = re.compile(r"\bs(?:\[(\d+):(\d+)\]|(\d+)\b)")
LABEL = re.compile(r"^(\.LBB\w+):")
BRANCH = re.compile(r"^\s*s_c?branch\w*\s+(\.LBB\w+)")


def sregs(text):
    out = set()
    for lo, hi, one in SREG.findall(text):
        if one:
            out.add(int(one))
        else:
            out.update(range(int(lo), int(hi) + 1))
    return out


def kernel_bodies(lines, wanted):
    """{kernel symbol: its instruction lines} for symbols containing one of `wanted`."""
    out, name, body = {}, None, []
    for ln in lines:
        m = re.match(r"^(_Z\w+):\s", ln + " ")
        if m:
            name, body = m.group(1), []
            continue
        if name and ln.lstrip().startswith(".amdhsa_kernel"):
            name = None
        if name:
            body.append(ln)
            if ln.strip().startswith("s_endpgm"):
                if any(w in name for w in wanted):
                    out[name] = body
                name = None
    return out


def instructions(body):
    """[(text, from inline assembly)] of the instruction and label lines of a kernel, in program order."""
    out, in_asm = [], False
    for raw in body:
        t = raw.strip()
        if t.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if t.startswith(";;#ASMEND"):
            in_asm = False
            continue
        ln = raw.split(";")[0].rstrip()
        if not ln.strip() or ln.strip().startswith(("#", "//")):
            continue
        if ln.strip().startswith(".") and not LABEL.match(ln):
            continue                                             # assembler directives
        out.append((ln, in_asm))
    return out


def check_kernel(name, body):
    """Forward data flow over the kernel's basic blocks: the set of scalar registers that an inline-assembly
    scalar load is still writing, joined (union) over a block's predecessors; every instruction that
    names one of them before an `s_waitcnt lgkmcnt(0)` is a problem."""
    ins = instructions(body)
    # basic blocks: a label starts one, a branch or s_endpgm ends one
    starts = {0}
    for i, (ln, _) in enumerate(ins):
        if LABEL.match(ln):
            starts.add(i)
        if BRANCH.match(ln) or ln.strip().startswith(("s_endpgm", "s_setpc")):
            starts.add(i + 1)
    starts = sorted(x for x in starts if x < len(ins))
    block_of_label = {}
    blocks = []
    for bi, st in enumerate(starts):
        en = starts[bi + 1] if bi + 1 < len(starts) else len(ins)
        blocks.append((st, en))
        m = LABEL.match(ins[st][0])
        if m:
            block_of_label[m.group(1)] = bi
    succ = []
    for bi, (st, en) in enumerate(blocks):
        last = ins[en - 1][0].strip()
        out = []
        b = BRANCH.match(ins[en - 1][0])
        if b and b.group(1) in block_of_label:
            out.append(block_of_label[b.group(1)])
        unconditional = last.startswith(("s_branch", "s_endpgm", "s_setpc"))
        if not unconditional and bi + 1 < len(blocks):
            out.append(bi + 1)
        succ.append(out)

    def transfer(bi, inflight, problems):
        st, en = blocks[bi]
        for i in range(st, en):
            ln, in_asm = ins[i]
            if LABEL.match(ln):
                continue
            if WAIT_ALL.match(ln):
                inflight = set()
                continue
            if in_asm and SLOAD.match(ln):
                dst = sregs(ln.split(",")[0])
                if problems is not None and (dst | sregs(",".join(ln.split(",")[1:]))) & inflight:
                    problems.add(f"{name}: `{ln.strip()}` touches registers of a scalar load in flight")
                inflight = inflight | dst
                continue
            if problems is not None and inflight and sregs(ln) & inflight:
                problems.add(f"{name}: `{ln.strip()}` uses s{sorted(sregs(ln) & inflight)} before the s_waitcnt "
                             f"that makes them valid")
        return inflight

    state_in = [set() for _ in blocks]
    work = list(range(len(blocks)))
    while work:
        bi = work.pop(0)
        out = transfer(bi, set(state_in[bi]), None)
        for sb in succ[bi]:
            if not out <= state_in[sb]:
                state_in[sb] |= out
                if sb not in work:
                    work.append(sb)
    problems = set()
    for bi in range(len(blocks)):
        transfer(bi, set(state_in[bi]), problems)
    return sorted(problems)


def main():
    if len(sys.argv) < 3:
        sys.exit(__doc__)
    lines = open(sys.argv[1]).read().splitlines()
    wanted = sys.argv[2:]
    bodies = kernel_bodies(lines, wanted)
    missing = [w for w in wanted if not any(w in k for k in bodies)]
    if missing:
        sys.exit(f"check_async_sloads: no kernel named like {missing} in {sys.argv[1]}")
    problems = []
    for name, body in bodies.items():
        problems += check_kernel(name, body)
    text = "\n".join(lines)
    for name in bodies:
        m = re.search(re.escape(name) + r"\.private_seg_size,\s*(\d+)", text)
        if m and int(m.group(1)) > 0:
            problems.append(f"{name}: {m.group(1)} bytes of scratch per lane (vector registers spilled)")
    if problems:
        sys.exit("check_async_sloads: FAILED\n  " + "\n  ".join(problems))
    print(f"check_async_sloads: {len(bodies)} kernel(s) ok: no use of a scalar-load result before its wait, no scratch")


if __name__ == "__main__":
    main()
