#!/usr/bin/env python3
"""Build-time check of the gfx950 assembly of the kernels (run by the Makefile on `hipcc -S` output).

The matrix-core GEMM issues some global loads in inline asm and waits for them with hand-counted `s_waitcnt vmcnt(N)`, also
in inline asm.  Between the two the compiler does not know that the destination registers are not valid yet: if it decides
to copy or otherwise touch one of them there, the kernel computes with stale data.  This script walks every kernel in
program order and fails when an instruction outside an asm block names a register that an asm-block load has written
and no asm-block `s_waitcnt vmcnt` (or a compiler-placed `vmcnt(0)`) has followed yet.

usage: check_asm_loads.py kernels.s
"""
import re
import sys

LOAD = re.compile(r"^\s*(global_load_\w+|buffer_load_\w+)\s+(v\[\d+:\d+\]|v\d+)(?=[,\s])")
REG = re.compile(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b")


def regs(text):
    out = set()
    for m in REG.finditer(text):
        if m.group(3) is not None:
            out.add(int(m.group(3)))
        else:
            out.update(range(int(m.group(1)), int(m.group(2)) + 1))
    return out


def check(path):
    errors, kernel, in_asm, pending = [], None, False, {}
    for no, raw in enumerate(open(path), 1):
        line = raw.split(";")[0].rstrip() if ";;#ASM" not in raw else raw.strip()
        if re.match(r"^[A-Za-z_]\w*:\s*$", raw) and not raw.startswith(".L"):
            kernel, in_asm, pending = raw.strip().rstrip(":"), False, {}
            continue
        if ";;#ASMSTART" in raw:
            in_asm = True
            continue
        if ";;#ASMEND" in raw:
            in_asm = False
            continue
        if not line.strip() or line.lstrip().startswith("."):
            continue
        if "s_endpgm" in line:
            pending = {}
            continue
        if in_asm:
            m = LOAD.match(line)
            if m and "lds" not in m.group(1):
                for r in regs(m.group(2)):
                    pending[r] = no
            elif "s_waitcnt" in line and "vmcnt" in line:
                pending = {}
            continue
        if "s_waitcnt" in line and "vmcnt(0)" in line:
            pending = {}
            continue
        touched = regs(line) & set(pending)
        if touched:
            r = min(touched)
            errors.append(f"{path}:{no}: {kernel}: `{line.strip()}` names v{r}, written by the asm load at line {pending[r]} "
                          f"whose wait has not come yet")
            for t in touched:
                del pending[t]
    return errors


def main():
    if len(sys.argv) != 2:
        print(__doc__)
        return 2
    errors = check(sys.argv[1])
    for e in errors:
        print(e, file=sys.stderr)
    if errors:
        print(f"check_asm_loads: {len(errors)} register(s) of loads in flight touched by the compiler", file=sys.stderr)
        return 1
    print("check_asm_loads: ok")
    return 0


if __name__ == "__main__":
    sys.exit(main())
