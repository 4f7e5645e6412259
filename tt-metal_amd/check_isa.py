"""Build-time check of the hand-scheduled loads in the streaming GEMM kernel.

bfp_matmul.hip issues some global loads as inline assembly and waits for them with its own s_waitcnt, because the
compiler's waits would drain the prefetch pipeline.  The compiler therefore believes that a loaded register holds its
value as soon as the load has issued.  That is only safe if it never copies, moves, reads or reuses such a register
between the load and the point where the data is taken over.  This script reads the device assembly of the file,
builds the control-flow graph of each streaming kernel (64- and 128-column) and propagates the set of registers with a load in flight:

  ring loads   (inline global_load_dwordx4 / global_load_ubyte without sc1: activations, and the exponent bytes of block-float
               ones, in flight across loop iterations) are in flight
               until an inline `v_mov_b32 vX, vN` reads register N
  slot loads   (inline global_load_dwordx4 ... sc1: partial sums of other workgroups) are in flight until the next
               `s_waitcnt vmcnt(0)`
  any `s_waitcnt vmcnt(0)` ends every flight (the kernel drains the ring that way when its k range is done)
  LDS reads    (inline ds_read*: staged tiles, read behind the compiler's back for the same reason) are in flight until
               the next `s_waitcnt` with lgkmcnt(0), the kernel's own or the compiler's

and fails the build if any compiler-generated instruction mentions a register while it is in flight, or if a register is
still in flight when the kernel ends.

    python tt-metal_amd/check_isa.py file.s

A second, simpler check (check_ring_operands, `--ring-operands file.s`) covers the 384-row kernel of bfp_matmul_tile.hip,
whose inline loads of A land in registers that the MFMAs read directly; it is described at the function.
"""
from __future__ import annotations

import re
import sys

_REG = re.compile(r"\bv(\d+)\b|\bv\[(\d+):(\d+)\]")
_BRANCH = re.compile(r"^s_(cbranch_\w+|branch)\s+(\.LBB\w+)")


def _regs(text: str) -> frozenset:
    out = set()
    for m in _REG.finditer(text):
        if m.group(1) is not None:
            out.add(int(m.group(1)))
        else:
            out.update(range(int(m.group(2)), int(m.group(3)) + 1))
    return frozenset(out)


def _kernels(lines):
    """(name, lines) of every function: from its label to the .Lfunc_end label (blocks may follow an s_endpgm)."""
    name, body = None, []
    for line in lines:
        m = re.match(r"^(_Z\w+):", line)
        if m:
            name, body = m.group(1), []
            continue
        if name is not None:
            if line.startswith(".Lfunc_end"):
                yield name, body
                name = None
            else:
                body.append(line)


def _blocks(body):
    """Basic blocks: list of dicts {label, instrs: [(text, inline_asm)], succ: [labels or '+1' or 'end']}."""
    blocks, cur, in_asm = [], {"label": None, "instrs": [], "succ": None}, False

    def close(succ):
        nonlocal cur
        cur["succ"] = succ
        blocks.append(cur)
        cur = {"label": None, "instrs": [], "succ": None}

    for line in body:
        s = line.strip()
        if s.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if s.startswith(";;#ASMEND"):
            in_asm = False
            continue
        m = re.match(r"^(\.LBB\w+):", s)
        if m:
            if cur["instrs"] or cur["label"] is not None:
                close(["+1"])
            cur["label"] = m.group(1)
            continue
        if not s or s.startswith(";") or s.startswith("."):
            continue
        text = s.split(";")[0].strip()
        cur["instrs"].append((text, in_asm))
        b = _BRANCH.match(text)
        if b:
            close([b.group(2)] if b.group(1) == "branch" else [b.group(2), "+1"])
        elif text.startswith("s_endpgm"):
            close(["end"])
    if cur["instrs"]:
        close(["end"])
    return blocks


def _check_kernel(name, body, problems, release_on_mfma=False):
    blocks = _blocks(body)
    index = {b["label"]: i for i, b in enumerate(blocks) if b["label"] is not None}
    succs = []
    for i, b in enumerate(blocks):
        out = []
        for t in b["succ"]:
            if t == "+1":
                if i + 1 < len(blocks):
                    out.append(i + 1)
            elif t != "end":
                if t not in index:
                    problems.append(f"{name}: branch to unknown label {t}")
                else:
                    out.append(index[t])
        succs.append(out)
    n_ring = sum(1 for b in blocks for t, a in b["instrs"] if a and t.startswith("global_load_dwordx4") and "sc1" not in t)
    if not n_ring:
        problems.append(f"{name}: no hand-written activation loads found (has the kernel changed?)")

    def run(block, state, report):
        ring, slot, lds = set(state[0]), set(state[1]), set(state[2])
        for text, asm in block["instrs"]:
            if text.startswith("s_waitcnt") and "lgkmcnt(0)" in text:           # every LDS read has returned
                lds.clear()
            if asm:
                if text.startswith(("global_load_dwordx4", "global_load_ubyte")):
                    dest = _regs(text.split(",")[0])
                    (slot if "sc1" in text else ring).update(dest)
                elif text.startswith("ds_read"):
                    lds.update(_regs(text.split(",")[0]))
                elif text.startswith("v_mov_b32"):
                    ring -= _regs(text.split(",")[-1])
                elif text.startswith("s_waitcnt vmcnt(0)"):
                    ring.clear()
                    slot.clear()
                continue
            if text.startswith("s_waitcnt") and "vmcnt(0)" in text:      # every vector-memory operation has landed
                ring.clear()
                slot.clear()
                continue
            if release_on_mfma and text.startswith("v_mfma"):
                operands = text.split(None, 1)[1].split(",")
                written = _regs(operands[0]) & ring
                if written and report is not None:
                    report.append(f"{name}: an MFMA writes registers {sorted(written)} while a hand-scheduled load into them is in flight: {text}")
                ring -= _regs(",".join(operands[1:]))
                continue
            if report is not None:
                hit = _regs(text) & (ring | slot | lds)
                if hit:
                    report.append(f"{name}: compiler instruction touches registers {sorted(hit)} while a hand-scheduled load into them is in flight: {text}")
            if text.startswith("s_endpgm") and report is not None and (ring or slot or lds):
                report.append(f"{name}: registers {sorted(ring | slot | lds)} still have a load in flight at s_endpgm")
        return frozenset(ring), frozenset(slot), frozenset(lds)

    empty = (frozenset(), frozenset(), frozenset())
    state_in = [None] * len(blocks)
    state_in[0] = empty
    work = [0]
    while work:
        i = work.pop()
        out = run(blocks[i], state_in[i], None)
        for j in succs[i]:
            merged = out if state_in[j] is None else tuple(a | b for a, b in zip(state_in[j], out))
            if merged != state_in[j]:
                state_in[j] = merged
                work.append(j)
    found = []
    for i, b in enumerate(blocks):
        if state_in[i] is not None:
            run(b, state_in[i], found)
    seen = set()
    for f in found:
        if f not in seen:
            seen.add(f)
            problems.append(f)


def check(path: str, kernel_substrings=("matmul_stream_kernel", "matmul_wide_kernel")) -> int:
    problems, checked = [], 0
    with open(path) as f:
        lines = f.read().split("\n")
    for name, body in _kernels(lines):
        if any(k in name for k in kernel_substrings):
            checked += 1
            _check_kernel(name, body, problems)
    if not checked:
        problems.append(f"no kernel matching {kernel_substrings} in {path}")
    for p in problems[:40]:
        print("check_isa:", p, file=sys.stderr)
    if len(problems) > 40:
        print(f"check_isa: ... and {len(problems) - 40} more", file=sys.stderr)
    return len(problems)


def check_ring_operands(path: str, kernel_substrings=("matmul_tall_kernel",)) -> int:
    """The 384-row GEMM of bfp_matmul_tile.hip loads its A operands with inline `global_load_dwordx4 vDST, vOFF, s[..]` into
    a ring of registers that the MFMAs read directly, behind the kernel's own partial waits.  Here a register is in flight
    from its inline load until the first compiler-generated v_mfma that reads it (the kernel puts that behind its wait);
    any other compiler-generated instruction naming it meanwhile (a copy, a spill, a reuse) fails the build, as does an
    MFMA that writes it."""
    problems, checked = [], 0
    with open(path) as f:
        lines = f.read().split("\n")
    for name, body in _kernels(lines):
        if any(k in name for k in kernel_substrings):
            checked += 1
            _check_kernel(name, body, problems, release_on_mfma=True)
    if not checked:
        problems.append(f"no kernel matching {kernel_substrings} in {path}")
    for p in problems[:40]:
        print("check_isa:", p, file=sys.stderr)
    return len(problems)


if __name__ == "__main__":
    sys.exit(1 if (check_ring_operands(sys.argv[2]) if sys.argv[1] == "--ring-operands" else check(sys.argv[1])) else 0)
