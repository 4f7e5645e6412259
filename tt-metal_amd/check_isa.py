"""Build-time check of the hand-scheduled loads in the streaming GEMM kernel.

bfp_matmul.hip issues some global loads as inline assembly and waits for them with its own s_waitcnt, because the
compiler's waits would drain the prefetch pipeline.  The compiler therefore believes that a loaded register holds its
value as soon as the load has issued.  That is only safe if it never copies, moves or reuses such a register between
the load and the wait.  This script reads the device assembly of the file and fails the build if that ever happens:

  ring loads   (global_load_dwordx4 without sc1, activations in flight across loop iterations): from the first of
               them to the last inline v_mov_b32 that hands a loaded register on (the pipelined loop and its tails),
               their destination registers may be mentioned only inside inline-assembly blocks
  slot loads   (global_load_dwordx4 ... sc1, partial sums of other workgroups): between the load and the inline
               s_waitcnt vmcnt(0) that follows it, no compiler-generated instruction may mention the destination

    python tt-metal_amd/check_isa.py file.s
"""
from __future__ import annotations

import re
import sys

_REG = re.compile(r"\bv(\d+)\b|\bv\[(\d+):(\d+)\]")


def _regs(text: str) -> set:
    out = set()
    for m in _REG.finditer(text):
        if m.group(1) is not None:
            out.add(int(m.group(1)))
        else:
            out.update(range(int(m.group(2)), int(m.group(3)) + 1))
    return out


def _kernels(lines):
    name, body = None, []
    for line in lines:
        m = re.match(r"^(_Z\w+):", line)
        if m:
            name, body = m.group(1), []
            continue
        if name is not None:
            body.append(line)
            if line.strip().startswith("s_endpgm"):
                yield name, body
                name = None


def check(path: str, kernel_substring: str = "matmul_stream_kernel") -> int:
    problems, checked = [], 0
    with open(path) as f:
        lines = f.read().split("\n")
    for name, body in _kernels(lines):
        if kernel_substring not in name:
            continue
        checked += 1
        # classify instructions: (index, text, inside inline assembly?)
        instrs, in_asm = [], False
        for line in body:
            s = line.strip()
            if s.startswith(";;#ASMSTART"):
                in_asm = True
                continue
            if s.startswith(";;#ASMEND"):
                in_asm = False
                continue
            if not s or s.startswith(";") or s.startswith("."):
                if re.match(r"^\.LBB", s):
                    instrs.append((s, in_asm, True))
                continue
            instrs.append((s.split(";")[0].strip(), in_asm, False))
        ring = set()
        for text, asm, _ in instrs:
            if asm and text.startswith("global_load_dwordx4") and "sc1" not in text:
                ring |= _regs(text.split(",")[0])
        if not ring:
            problems.append(f"{name}: no hand-written activation loads found (has the kernel changed?)")
        # the stretch of code from the first request to the last hand-over (loop and tails as laid out in the file)
        first = min((i for i, (t, a, _) in enumerate(instrs) if a and t.startswith("global_load_dwordx4") and "sc1" not in t), default=0)
        last = max((i for i, (t, a, _) in enumerate(instrs) if a and t.startswith("v_mov_b32") and _regs(t.split(",")[-1]) & ring), default=0)
        for text, asm, label in instrs[first:last + 1]:
            if label or asm:
                continue
            hit = _regs(text) & ring
            if hit:
                problems.append(f"{name}: compiler instruction touches activation ring registers {sorted(hit)}: {text}")
        for i, (text, asm, _) in enumerate(instrs):
            if not (asm and text.startswith("global_load_dwordx4") and "sc1" in text):
                continue
            dest = _regs(text.split(",")[0])
            for later, later_asm, later_label in instrs[i + 1:]:
                if later_asm and later.startswith("s_waitcnt vmcnt(0)"):
                    break
                if later_label:
                    problems.append(f"{name}: branch target between a slot load and its wait: {later}")
                    break
                if not later_asm and _regs(later) & dest:
                    problems.append(f"{name}: compiler instruction touches a slot load's destination before the wait: {later}")
                    break
            else:
                problems.append(f"{name}: slot load without a following inline wait: {text}")
    if not checked:
        problems.append(f"no kernel matching '{kernel_substring}' in {path}")
    for p in problems:
        print("check_isa:", p, file=sys.stderr)
    return len(problems)


if __name__ == "__main__":
    sys.exit(1 if check(sys.argv[1]) else 0)
