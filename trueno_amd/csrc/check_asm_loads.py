#!/usr/bin/env python3
"""Build-time check of the gfx950 assembly of the kernels (run by the Makefile on `hipcc -S` output).

The matrix-core GEMM issues some global loads in inline asm and waits for them with hand-counted `s_waitcnt vmcnt(N)`, also
in inline asm.  Between the two the compiler does not know that the destination registers are not valid yet: if it decides
to copy or otherwise touch one of them there, the kernel computes with stale data.

The check models the counter the hardware keeps.  Vector-memory operations complete in the order they were issued, and
`s_waitcnt vmcnt(N)` returns when at most N of them are outstanding: a load is known to have landed once a wait with
N <= (operations issued after the load) has been passed.  For every kernel the script builds the control-flow graph
(labels, s_branch / s_cbranch_*, s_endpgm) and computes, for every load written in an asm block, the least number of
operations issued after it over all paths to each point (a forward data-flow analysis: at a join the minimum, around a
loop until nothing changes), so a load that is still in flight at the end of a loop body is still in flight at the top of
the next iteration.  It fails when an instruction outside an asm block names a register of a load that is not known to
have landed there.

usage: check_asm_loads.py kernels.s
"""
import re
import sys

LOAD = re.compile(r"^\s*(global_load_\w+|buffer_load_\w+|flat_load_\w+|scratch_load_\w+)\s+(v\[\d+:\d+\]|v\d+)(?=[,\s])")
# what the counter counts on this target: every vector-memory load, store and atomic (cache maintenance is left out,
# which can only make a load look outstanding for longer)
VMOP = re.compile(r"^\s*(global_|buffer_|flat_|scratch_|tbuffer_|image_)(load|store|atomic)")
REG = re.compile(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b")
VMCNT = re.compile(r"vmcnt\((\d+)\)")
LABEL = re.compile(r"^([.A-Za-z_$][\w.$]*):")
BRANCH = re.compile(r"^\s*(s_branch|s_cbranch_\w+)\s+([.A-Za-z_$][\w.$]*)")
CAP = 63          # the counter's field is six bits wide; nothing waits for more


def regs(text):
    out = set()
    for m in REG.finditer(text):
        if m.group(3) is not None:
            out.add(int(m.group(3)))
        else:
            out.update(range(int(m.group(1)), int(m.group(2)) + 1))
    return out


class Ins:
    __slots__ = ("no", "text", "asm")

    def __init__(self, no, text, asm):
        self.no, self.text, self.asm = no, text, asm


def kernels_of(path):
    """[(name, [Ins or ('label', name)])] for every function of the file"""
    out, cur, in_asm = [], None, False
    for no, raw in enumerate(open(path), 1):
        if ";;#ASMSTART" in raw:
            in_asm = True
            continue
        if ";;#ASMEND" in raw:
            in_asm = False
            continue
        line = raw.split(";")[0].rstrip()
        if not line.strip():
            continue
        m = LABEL.match(line.strip())
        if m and not in_asm:
            name = m.group(1)
            if name.startswith(".Lfunc_end"):
                cur = None
            elif name.startswith("."):
                if cur is not None:
                    cur.append(("label", name))
            else:
                cur = []
                out.append((name, cur))
            continue
        if line.lstrip().startswith(".") or cur is None:
            continue
        cur.append(Ins(no, line.strip(), in_asm))
    return out


def blocks_of(items):
    """basic blocks: [{'ins': [...], 'succ': [block index, ...]}]"""
    blocks, label_at, cur = [], {}, None
    for it in items:
        if isinstance(it, tuple):
            cur = {"ins": [], "succ": [], "fall": True}
            blocks.append(cur)
            label_at[it[1]] = len(blocks) - 1
            continue
        if cur is None:
            cur = {"ins": [], "succ": [], "fall": True}
            blocks.append(cur)
        cur["ins"].append(it)
        if BRANCH.match(it.text) or it.text.startswith("s_endpgm") or it.text.startswith("s_setpc") or it.text.startswith("s_swappc"):
            cur = None
    for i, b in enumerate(blocks):
        last = b["ins"][-1].text if b["ins"] else ""
        m = BRANCH.match(last)
        if m:
            if m.group(2) in label_at:
                b["succ"].append(label_at[m.group(2)])
            if m.group(1) != "s_branch" and i + 1 < len(blocks):
                b["succ"].append(i + 1)
        elif last.startswith("s_endpgm"):
            pass
        elif i + 1 < len(blocks):
            b["succ"].append(i + 1)
    return blocks


def step(state, ins, report=None):
    """state: {load line: (ops issued after it, frozenset of its registers)}; returns the state behind `ins`"""
    text = ins.text
    if "s_waitcnt" in text:
        m = VMCNT.search(text)
        if m:
            n = int(m.group(1))
            state = {k: v for k, v in state.items() if v[0] < n}
        return state
    if not ins.asm and state and report is not None:
        named = regs(text)
        for line, (_, rs) in sorted(state.items()):
            hit = named & rs
            if hit:
                report(ins, min(hit), line)
    if VMOP.match(text):
        state = {k: (min(v[0] + 1, CAP), v[1]) for k, v in state.items()}
        m = LOAD.match(text)
        if ins.asm and m and "lds" not in m.group(1):
            state[ins.no] = (0, frozenset(regs(m.group(2))))
    return state


def join(a, b):
    if a is None:
        return dict(b)
    out = dict(a)
    for k, v in b.items():
        out[k] = v if k not in out else (min(out[k][0], v[0]), v[1])
    return out


def check_kernel(path, name, items):
    if not any(isinstance(it, Ins) and it.asm and LOAD.match(it.text) for it in items):
        return []
    errors = []
    for it in items:
        if isinstance(it, Ins) and (it.text.startswith("s_setpc") or it.text.startswith("s_swappc")):
            errors.append(f"{path}:{it.no}: {name}: `{it.text}`: an indirect jump in a kernel with loads written in asm cannot be followed")
    blocks = blocks_of(items)
    if not blocks:
        return errors
    state_in = [None] * len(blocks)
    state_in[0] = {}
    work = [0]
    while work:
        i = work.pop()
        st = state_in[i]
        for ins in blocks[i]["ins"]:
            st = step(st, ins)
        for s in blocks[i]["succ"]:
            merged = join(state_in[s], st)
            if merged != state_in[s]:
                state_in[s] = merged
                work.append(s)
    seen = set()

    def report(ins, reg, line):
        if (ins.no, line) not in seen:
            seen.add((ins.no, line))
            errors.append(f"{path}:{ins.no}: {name}: `{ins.text}` names v{reg}, written by the asm load at line {line} "
                          f"whose wait has not come yet")

    for i, b in enumerate(blocks):
        st = state_in[i]
        if st is None:
            continue
        for ins in b["ins"]:
            st = step(st, ins, report)
    return errors


def check(path):
    errors = []
    for name, items in kernels_of(path):
        errors += check_kernel(path, name, items)
    return errors


def main():
    if len(sys.argv) != 2:
        print(__doc__)
        return 2
    errors = check(sys.argv[1])
    for e in errors:
        print(e, file=sys.stderr)
    if errors:
        print(f"check_asm_loads: {len(errors)} use(s) of registers of loads in flight by the compiler", file=sys.stderr)
        return 1
    print("check_asm_loads: ok")
    return 0


if __name__ == "__main__":
    sys.exit(main())
