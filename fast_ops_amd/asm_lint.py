"""Checks the gfx950 assembly of kernels that issue MFMAs as inline assembly for the two data hazards that the
compiler's hazard recognizer handles for its own MFMA instructions but cannot see inside an asm statement:

  1. an MFMA source register (A, B or C, VGPR or AGPR) written by a VALU instruction needs 2 wait states before the
     MFMA reads it (measured on MI355X: back-to-back gives wrong products; v_accvgpr_read counts as VALU);
  2. a register written by an 8-pass MFMA (32x32x16 f16/bf16) needs 11 wait states before any other instruction than
     an MFMA touches it.

A third rule concerns the direct-to-LDS copies, which the kernels also issue as inline assembly:

  3. an LDS-DMA instruction (global_load_lds_*, buffer_load_* ... lds) reads M0 and needs 1 wait state after a scalar
     instruction that wrote M0 (checked by lint_m0_* for every function of a file).

A wait state is one issued instruction (s_nop N counts N+1). For rule 2 time is modelled in wait states; an MFMA is
taken to issue no earlier than 8 wait states after the previous one (the matrix pipe is busy for its 8 passes), every
other instruction advances time by one. Control flow is treated conservatively for rule 1 (an MFMA within two
instructions after a label fails) and in layout order for rule 2 (the kernels fence every out-of-line reader
explicitly).

Used by build.py: the attention kernels are first compiled without wait states in front of their MFMAs; if this
check reports anything, they are compiled again with them.
"""
from __future__ import annotations

import re
from typing import Iterable, List, Set, Tuple

_REG = re.compile(r"\b([va])(\d+)\b|\b([va])\[(\d+):(\d+)\]")


def _regs(operand: str) -> Set[Tuple[str, int]]:
    out = set()
    for m in _REG.finditer(operand):
        if m.group(1):
            out.add((m.group(1), int(m.group(2))))
        else:
            out.update((m.group(3), i) for i in range(int(m.group(4)), int(m.group(5)) + 1))
    return out


def _split_operands(rest: str) -> List[str]:
    ops, depth, cur = [], 0, ""
    for ch in rest:
        if ch == "[":
            depth += 1
        elif ch == "]":
            depth -= 1
        if ch == "," and depth == 0:
            ops.append(cur.strip())
            cur = ""
        else:
            cur += ch
    if cur.strip():
        ops.append(cur.strip())
    return ops


# VALU instructions that write more than their first operand
_SWAPS = ("v_permlane32_swap", "v_permlane16_swap", "v_swap_b32")
MFMA_PASSES = 8
VALU_TO_MFMA = 2          # wait states between a VALU write and an MFMA read
MFMA_TO_OTHER = 11        # wait states between an 8-pass MFMA write and any non-MFMA access


def lint_function(lines: Iterable[str], name: str) -> List[str]:
    problems: List[str] = []
    recent: List[Set[Tuple[str, int]]] = []     # registers written by VALU in each of the last instructions (newest last)
    since_label = 10**9
    t = 0                                         # time in wait states
    last_mfma_issue = -10**9
    ready = {}                                    # register -> time from which a non-MFMA instruction may touch it
    for ln, raw in enumerate(lines, 1):
        line = raw.split(";")[0].strip()
        if not line or line.startswith("."):
            if line.startswith(".LBB") or (line.endswith(":") and not line.startswith(".")):
                since_label = 0
                recent = []
            continue
        if line.endswith(":"):
            since_label = 0
            recent = []
            continue
        parts = line.split(None, 1)
        op = parts[0]
        ops = _split_operands(parts[1]) if len(parts) > 1 else []
        if op.startswith("v_mfma") or op.startswith("v_smfmac"):
            srcs = set()
            for o in ops[1:]:
                srcs |= _regs(o)
            if since_label < VALU_TO_MFMA:
                problems.append(f"{name}:{ln}: MFMA {since_label} instruction(s) after a label: {line}")
            for age, written in enumerate(reversed(recent[-VALU_TO_MFMA:])):
                hit = srcs & written
                if hit:
                    problems.append(f"{name}:{ln}: MFMA reads {sorted(hit)[:4]} written by a VALU instruction {age} wait state(s) earlier: {line}")
            issue = max(t, last_mfma_issue + MFMA_PASSES)
            last_mfma_issue = issue
            for r in _regs(ops[0]):
                ready[r] = issue + MFMA_TO_OTHER + 1
            t = issue + 1
            recent.append(set())
            since_label += 1
            continue
        # any other instruction: rule 2 on every register it names
        touched = set()
        for o in ops:
            touched |= _regs(o)
        for r in touched:
            if ready.get(r, -1) > t:
                problems.append(f"{name}:{ln}: {r[0]}{r[1]} touched {ready[r] - t} wait state(s) too early after an MFMA wrote it: {line}")
                break
        for r in touched:
            ready.pop(r, None)
        written = set()
        if op.startswith("v_") and ops:
            written |= _regs(ops[0])
            if op.startswith(_SWAPS) and len(ops) > 1:
                written |= _regs(ops[1])
        states = 1
        if op == "s_nop" and ops:
            try:
                states = int(ops[0], 0) + 1
            except ValueError:
                states = 1
        for _ in range(states):
            recent.append(set())
        recent[-1] = written
        if len(recent) > 8:
            recent = recent[-8:]
        t += states
        since_label += states
    return problems


def lint_file(path: str, name_filter: str) -> List[str]:
    """Lints every function of the assembly file whose symbol matches the regular expression `name_filter`. A filter
    that matches no function is reported as a problem: a check that looked at nothing must not read as a pass."""
    pat = re.compile(name_filter)
    problems: List[str] = []
    matched = 0
    cur_name, cur_lines = None, []
    with open(path) as f:
        for raw in f:
            s = raw.rstrip("\n")
            if cur_name is None:
                head = s.split(";")[0].rstrip()
                if head.endswith(":") and not head.startswith((".", " ", "\t")) and pat.search(head):
                    cur_name, cur_lines = head[:-1], []
                    matched += 1
            else:
                if s.startswith(".Lfunc_end"):
                    problems += lint_function(cur_lines, cur_name)
                    cur_name = None
                else:
                    cur_lines.append(s)
    if matched == 0:
        problems.append(f"{path}: no function matches {name_filter!r}")
    return problems


_M0_WRITE = re.compile(r"^s_\w+\s+m0\s*,")


def _is_lds_dma(op: str, rest: str) -> bool:
    if op.startswith("global_load_lds_") or op.startswith("scratch_load_lds_"):
        return True
    return op.startswith("buffer_load_") and re.search(r"\blds\b", rest) is not None


def lint_m0_function(lines: Iterable[str], name: str) -> List[str]:
    """Rule 3: no LDS-DMA instruction directly after a scalar write of M0 (or directly after a label, where the
    predecessor is unknown, if the instruction before the label wrote M0)."""
    problems: List[str] = []
    m0_age = 10**9           # wait states since the last scalar write of M0
    for ln, raw in enumerate(lines, 1):
        line = raw.split(";")[0].strip()
        if not line or line.startswith(".") or line.endswith(":"):
            continue            # labels do not reset the age: a fall-through predecessor counts
        parts = line.split(None, 1)
        op, rest = parts[0], (parts[1] if len(parts) > 1 else "")
        if _is_lds_dma(op, rest) and m0_age < 1:
            problems.append(f"{name}:{ln}: LDS-DMA reads M0 directly after it was written: {line}")
        if _M0_WRITE.match(line):
            m0_age = 0
            continue
        states = 1
        if op == "s_nop":
            try:
                states = int(rest.strip(), 0) + 1
            except ValueError:
                states = 1
        m0_age += states
    return problems


def lint_m0_file(path: str) -> List[str]:
    """Rule 3 over every function of the assembly file."""
    problems: List[str] = []
    cur_name, cur_lines = None, []
    with open(path) as f:
        for raw in f:
            s = raw.rstrip("\n")
            if cur_name is None:
                head = s.split(";")[0].rstrip()
                if head.endswith(":") and not head.startswith((".", " ", "\t")):
                    cur_name, cur_lines = head[:-1], []
            else:
                if s.startswith(".Lfunc_end"):
                    problems += lint_m0_function(cur_lines, cur_name)
                    cur_name = None
                else:
                    cur_lines.append(s)
    return problems


if __name__ == "__main__":
    import sys
    found = lint_file(sys.argv[1], sys.argv[2] if len(sys.argv) > 2 else "attn_fwd_wide_kernel") + lint_m0_file(sys.argv[1])
    for p in found[:50]:
        print(p)
    print(f"{len(found)} problem(s)")
