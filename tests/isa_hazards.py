"""Static check of generated gfx950 assembly for the hand-waited load pipelines.

The GEMM kernels request global loads with inline assembly and wait for them with hand-placed
`s_waitcnt vmcnt(N)`.  The compiler does not know that those registers are filled asynchronously,
so a register copy, spill or reuse it decides to place between a request and its wait would read or
overwrite data that has not arrived - silently.  This walks each kernel's control-flow graph,
carries the in-order queue of outstanding loads along every path (loads retire oldest-first at
`s_waitcnt vmcnt(N)`), and reports any instruction that touches a register of a load still in
flight, plus any kernel that uses scratch memory (spills also travel through the same counter).
"""
import re


def _regs(tok):
    """Vector registers named in an operand string: v0.. as 0.., accumulation registers a0.. as 1000.. ."""
    out = set()
    for file, base in (("v", 0), ("a", 1000)):
        for m in re.finditer(r"(?<![\w])%s\[(\d+):(\d+)\]" % file, tok):
            out |= set(range(base + int(m.group(1)), base + int(m.group(2)) + 1))
        for m in re.finditer(r"(?<![\w\[:])%s(\d+)\b" % file, tok):
            out.add(base + int(m.group(1)))
    return frozenset(out)


def kernels(asm):
    for fm in re.finditer(r"^(_Z\w+):.*\n", asm, re.M):
        end = asm.find(".Lfunc_end", fm.end())
        if end > 0:
            yield fm.group(1), asm[fm.end():end]


def scratch_bytes(asm):
    """kernel symbol -> private segment size from the metadata."""
    out = {}
    for blk in asm.split("  - .agpr_count:")[1:]:
        name = re.search(r"\.name:\s+(\S+)", blk)
        size = re.search(r"\.private_segment_fixed_size:\s+(\d+)", blk)
        if name and size:
            out[name.group(1)] = int(size.group(1))
    return out


def hazards(body, max_states=24):
    blocks, order, cur = {"ENTRY": []}, ["ENTRY"], "ENTRY"
    for raw in body.split("\n"):
        l = raw.strip()
        if not l or l.startswith(";"):
            continue
        m = re.match(r"^(\.LBB\w+):", l)
        if m:
            cur = m.group(1)
            blocks[cur] = []
            order.append(cur)
            continue
        if l.startswith("."):
            continue
        blocks[cur].append(l.split(";")[0].strip())
        if l.startswith(("s_cbranch", "s_branch", "s_endpgm")):     # unlabelled fall-through block
            cur = f"{cur}+"
            blocks[cur] = []
            order.append(cur)
    succ = {}
    for n, b in enumerate(order):
        out, fall = [], True
        for l in blocks[b]:
            op = l.split()[0] if l else ""
            if op.startswith("s_cbranch"):
                out.append(l.split()[-1])
            elif op == "s_branch":
                out.append(l.split()[-1])
                fall = False
            elif op == "s_endpgm":
                fall = False
        if fall and n + 1 < len(order):
            out.append(order[n + 1])
        succ[b] = out
    seen = {b: set() for b in order}
    work, bad = [("ENTRY", ())], set()
    while work:
        b, q = work.pop()
        if q in seen[b] or len(seen[b]) > max_states:
            continue
        seen[b].add(q)
        q = list(q)
        for l in blocks[b]:
            op = l.split()[0]
            m = re.match(r"s_waitcnt.*vmcnt\((\d+)\)", l)
            if m:
                while len(q) > int(m.group(1)):
                    q.pop(0)
                continue
            rest = l[len(op):]
            ops = rest.split(",")
            if op.startswith(("global_load", "scratch_load", "buffer_load", "flat_load")):
                if "_lds_" in op:
                    dst, used = frozenset(), _regs(rest)
                else:
                    dst, used = _regs(ops[0]), _regs(",".join(ops[1:]))
                if any(d & used for d in q) or any(d & dst for d in q):
                    bad.add((b, l))
                q.append(dst)
                continue
            used = _regs(rest)
            if any(d & used for d in q):
                bad.add((b, l))
        for t in succ[b]:
            if t in blocks:
                work.append((t, tuple(q)))
    return sorted(bad)
