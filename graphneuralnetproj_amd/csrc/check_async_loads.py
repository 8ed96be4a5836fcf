#!/usr/bin/env python3
"""Build-time check of the SpMM kernels' hand-managed asynchronous loads.

The main kernel issues its vector-memory loads from inline assembly and waits
for them with hand-placed ``s_waitcnt vmcnt(N)``.  The compiler does not know
that the destination registers of those loads are written later, so the rule
"no instruction touches a register while a load into it may still be in flight"
is the source's responsibility.  This script verifies the rule on the generated
gfx950 assembly (``hipcc -S``) by a forward dataflow analysis over each kernel's
control-flow graph, and also rejects kernels that spill registers to scratch (a
spill of a register with a load in flight would save garbage).

State: the queue of vector-memory operations that may still be outstanding,
youngest last; each entry is the set of VGPRs the operation writes (empty for
stores).  ``s_waitcnt vmcnt(N)`` keeps the N youngest entries (loads complete in
order).  Where paths merge, queues are aligned at the youngest end and entries
are united position by position, which over-approximates every path.  Any
instruction that reads or writes a VGPR held in some queue entry is reported,
except a load writing registers that an older pending load also writes.

Usage: check_async_loads.py kernels.s [name-substring]
Exit status 0 = clean, 1 = violations (listed), 2 = parse problem.
"""
import re
import sys
from collections import defaultdict

VM_LOAD = re.compile(r"^(buffer_load|global_load|flat_load|scratch_load|tbuffer_load|image_)")
VM_STORE = re.compile(r"^(buffer_store|global_store|flat_store|scratch_store|tbuffer_store|buffer_atomic|global_atomic|flat_atomic)")
VREG = re.compile(r"\bv(\d+)\b|\bv\[(\d+):(\d+)\]")
LABEL = re.compile(r"^(\.LBB\d+_\d+):")
MAXQ = 64


def vregs(text):
    out = set()
    for m in VREG.finditer(text):
        if m.group(1) is not None:
            out.add(int(m.group(1)))
        else:
            out.update(range(int(m.group(2)), int(m.group(3)) + 1))
    return out


def split_kernels(lines):
    """Yield (name, [instruction lines]) for every .amdhsa kernel body."""
    name, body = None, []
    for ln in lines:
        m = re.match(r"^(\w+):\s*(;.*)?$", ln)
        if m and not ln.startswith(".L") and name is None and m.group(1).startswith("_Z"):
            name, body = m.group(1), []
            continue
        if name is not None:
            body.append(ln)
            if ln.strip().startswith("s_endpgm"):
                # a kernel may hold several s_endpgm; stop at the .Lfunc_end marker instead
                pass
            if ln.startswith(".Lfunc_end"):
                yield name, body
                name, body = None, []


def parse_blocks(body):
    """Basic blocks (split at labels and after every branch) and the successor map."""
    blocks, cur_label, cur = [], "entry", []
    anon = 0
    for i, raw in enumerate(body):
        ln = raw.split(";")[0].strip() if not raw.strip().startswith(";;#") else ""
        if not ln:
            continue
        m = LABEL.match(ln)
        if m:
            blocks.append((cur_label, cur))
            cur_label, cur = m.group(1), []
            continue
        if ln.startswith("."):
            continue
        parts = ln.split(None, 1)
        op = parts[0]
        cur.append((i, op, parts[1] if len(parts) > 1 else ""))
        if op.startswith("s_cbranch") or op == "s_branch" or op == "s_endpgm" or op == "s_setpc_b64":
            blocks.append((cur_label, cur))
            anon += 1
            cur_label, cur = f"<after-branch-{anon}>", []
    blocks.append((cur_label, cur))
    index = {lab: k for k, (lab, _) in enumerate(blocks)}
    succ = defaultdict(list)
    for k, (lab, ins) in enumerate(blocks):
        fall = True
        if ins:
            _, op, args = ins[-1]
            if op.startswith("s_cbranch"):
                succ[k].append(index[args.strip()])
            elif op == "s_branch":
                succ[k].append(index[args.strip()])
                fall = False
            elif op in ("s_endpgm", "s_setpc_b64"):
                fall = False
        if fall and k + 1 < len(blocks):
            succ[k].append(k + 1)
    return blocks, succ


def merge(a, b):
    """Union of two queues aligned at the youngest end."""
    if a is None:
        return b
    n = max(len(a), len(b))
    out = []
    for i in range(1, n + 1):
        sa = a[-i] if i <= len(a) else frozenset()
        sb = b[-i] if i <= len(b) else frozenset()
        out.append(sa | sb)
    out.reverse()
    return tuple(out)


def transfer(queue, ins, report):
    q = list(queue)
    for (lineno, op, args) in ins:
        if op == "s_waitcnt":
            m = re.search(r"vmcnt\((\d+)\)", args)
            if m:
                n = int(m.group(1))
                q = q[len(q) - n:] if n < len(q) else q
            continue
        regs = vregs(args)
        pending = set().union(*q) if q else set()
        if VM_LOAD.match(op):
            dest = vregs(args.split(",")[0])
            srcs = regs - dest if not (dest & vregs(",".join(args.split(",")[1:]))) else vregs(",".join(args.split(",")[1:]))
            bad = srcs & pending
            if bad and report is not None:
                report.append((lineno, op, args, sorted(bad)))
            q.append(frozenset(dest))
        elif VM_STORE.match(op):
            bad = regs & pending
            if bad and report is not None:
                report.append((lineno, op, args, sorted(bad)))
            q.append(frozenset())
        else:
            bad = regs & pending
            if bad and report is not None:
                report.append((lineno, op, args, sorted(bad)))
        if len(q) > MAXQ:
            q = q[-MAXQ:]
    return tuple(q)


def check_kernel(name, body):
    blocks, succ = parse_blocks(body)
    state_in = [None] * len(blocks)
    state_in[0] = tuple()
    work = [0]
    rounds = 0
    while work:
        k = work.pop()
        rounds += 1
        if rounds > 200000:
            return None
        out = transfer(state_in[k], blocks[k][1], None)
        for s in succ[k]:
            new = merge(state_in[s], out)
            if new != state_in[s]:
                state_in[s] = new
                work.append(s)
    report = []
    for k, (lab, ins) in enumerate(blocks):
        if state_in[k] is not None:
            transfer(state_in[k], ins, report)
    return report


def main():
    path = sys.argv[1]
    want = sys.argv[2] if len(sys.argv) > 2 else "tcsl_spmm_kernel"
    lines = open(path).read().splitlines()
    status = 0
    checked = 0
    # scratch usage from the kernel descriptors
    for m in re.finditer(r"\.amdhsa_kernel (\S+)(.*?)\.end_amdhsa_kernel", "\n".join(lines), re.S):
        if want in m.group(1):
            ps = re.search(r"\.amdhsa_private_segment_fixed_size (\d+)", m.group(2))
            if ps and int(ps.group(1)) != 0:
                print(f"FAIL {m.group(1)}: {ps.group(1)} bytes of scratch per lane (register spills)")
                status = 1
    for name, body in split_kernels(lines):
        if want not in name:
            continue
        checked += 1
        rep = check_kernel(name, body)
        if rep is None:
            print(f"FAIL {name}: analysis did not converge")
            status = 2
            continue
        if rep:
            status = 1
            print(f"FAIL {name}: {len(rep)} accesses to registers with a load possibly in flight")
            for (lineno, op, args, bad) in rep[:20]:
                print(f"   body line {lineno}: {op} {args}   <- v{bad}")
        else:
            print(f"ok   {name}")
    if checked == 0:
        print("no kernel matched", want)
        status = 2
    sys.exit(status)


if __name__ == "__main__":
    main()
