"""Static check of the compiled gfx950 assembly for a matrix-instruction hazard that hipcc (ROCm 7.2) does not guard.

Measured on MI355X: a v_mfma whose accumulator input (SrcC) is the result of an immediately preceding v_mfma of a
DIFFERENT opcode (seen with v_mfma_f32_16x16x32_bf16 followed by v_mfma_f32_16x16x16_bf16 and the reverse) returns
wrong sums unless at least five wait states separate the two -- whether it writes its own result over that
accumulator (in place) or into other registers; the same pair with the same opcode is forwarded correctly back to
back.  The compiler emits no wait states for the mixed pair (with or without -amdgpu-mfma-vgpr-form), and a memory
wait that happens to fall between the two hides the error on some runs and not on others.  Measured boundary for
the two bf16 shapes (4 passes each): four wait states wrong, five right, i.e. passes + 1, which is what a dependent
read that is not forwarded needs.  This scan fails the build when the generated code contains such a pair closer
than passes + 1 wait states of the first instruction (8 passes for v_mfma_f32_16x16x4_f32, 16 assumed for any opcode
not listed), counting every instruction in between as one wait state and `s_nop n` as n + 1.  Code is read in
text order and, from every branch, on into the branch target while an earlier matrix instruction can still matter
(loop back edges included).

Functions whose name contains "selftest" are skipped: the library's own test of this fact places such pairs on
purpose, in inline assembly.

Usage: python isa_check.py file.s      (exit status 1 and a listing if a hazard is found)
"""
from __future__ import annotations

import re
import sys

PASSES = {"v_mfma_f32_16x16x16_bf16": 4, "v_mfma_f32_16x16x32_bf16": 4, "v_mfma_f32_16x16x4_f32": 8}
DEFAULT_PASSES = 16


def min_wait_states(first_opcode: str) -> int:
    return PASSES.get(first_opcode, DEFAULT_PASSES) + 1


MAX_WINDOW = DEFAULT_PASSES + 1
_MFMA = re.compile(r"^\s*(v_mfma_\w+)\s+([av])\[(\d+):(\d+)\],\s*(.*)$")
_REG = re.compile(r"([av])\[(\d+):(\d+)\]")
_FUNC = re.compile(r"^([A-Za-z_][\w.$]*):")


def _srcc(rest: str):
    """Register range of the last operand (SrcC) of an MFMA, or None for a constant."""
    ops = [o.strip() for o in rest.split(",")]
    # operands after vDst: SrcA, SrcB, SrcC [, modifiers like cbsz:.. abid:.. blgp:..]
    ops = [o for o in ops if ":" not in o or _REG.fullmatch(o.split()[0])]
    if len(ops) < 3:
        return None
    m = _REG.fullmatch(ops[2].split()[0])
    return (m.group(1), int(m.group(2)), int(m.group(3))) if m else None


def _overlap(a, b):
    return a[0] == b[0] and not (a[2] < b[1] or b[2] < a[1])


_BRANCH = re.compile(r"^s_c?branch\w*\s+(\.L\w+)")


def _states(s: str) -> int:
    n = re.match(r"s_nop\s+(\d+)", s)
    return int(n.group(1)) + 1 if n else 1


def _step(window, s, m, func, no):
    """Advances the window of recent MFMAs over instruction `s` (m: its MFMA match or None); returns the new window
    and the hazards this instruction completes."""
    found = []
    if m:
        op, dst = m.group(1), (m.group(2), int(m.group(3)), int(m.group(4)))
        c = _srcc(m.group(5))
        if c is not None and "selftest" not in func:
            for w in window:
                if _overlap(w[1], c) and w[0] != op and w[2] < min_wait_states(w[0]):
                    found.append((func, no, w[3], s, w[2]))
    states = _states(s)
    # a write to the same registers by anything else ends the dependence; keeping the entry is conservative
    window = [[w[0], w[1], w[2] + states, w[3], w[4]] for w in window if w[2] + states < MAX_WINDOW]
    if m:
        # the new instruction supersedes older writers of the same registers
        window = [w for w in window if not _overlap(w[1], dst)]
        window.append([op, dst, 0, s, no])
    return window, found


def _instructions(lines):
    """(line number, function, text, label or None) for every label and instruction line."""
    func = "?"
    for no, raw in enumerate(lines, 1):
        line = raw.split(";")[0].rstrip()
        if not line.strip():
            continue
        f = _FUNC.match(line)
        if f and not line.startswith(".L") and not line.startswith("\t"):
            func = f.group(1)
            yield no, func, None, "<function>"
            continue
        s = line.strip()
        if s.endswith(":"):
            yield no, func, None, s[:-1]
            continue
        if s.startswith("."):
            continue  # directives take no issue slot
        yield no, func, s, None


def scan(lines):
    """Yields (function, line number, first instruction, second instruction, wait states between).  Code is followed
    in text order and, from every branch, into its target for as long as an earlier MFMA can still matter."""
    items = list(_instructions(lines))
    labels = {}
    for i, (no, func, s, label) in enumerate(items):
        if label is not None and label != "<function>":
            labels[(func, label)] = i
    seen = set()
    window = []
    for i, (no, func, s, label) in enumerate(items):
        if label == "<function>":
            window = []
            continue
        if s is None:
            continue
        window, found = _step(window, s, _MFMA.match("\t" + s), func, no)
        for h in found:
            if (h[1], h[2]) not in seen:
                seen.add((h[1], h[2]))
                yield h
        br = _BRANCH.match(s)
        if br and window and (func, br.group(1)) in labels:
            w2 = [list(w) for w in window]
            for no2, func2, s2, label2 in items[labels[(func, br.group(1))]:]:
                if label2 == "<function>" or not w2:
                    break
                if s2 is None:
                    continue
                w2, found = _step(w2, s2, _MFMA.match("\t" + s2), func, no2)
                # only what was in flight at the branch matters here: later instructions are met in text order
                w2 = [w for w in w2 if w[4] <= no or w[4] > no2]
                for h in found:
                    if (h[1], h[2]) not in seen:
                        seen.add((h[1], h[2]))
                        yield h
                if s2.startswith("s_endpgm") or s2.startswith("s_branch"):
                    break


def check_file(path: str):
    with open(path) as fh:
        return list(scan(fh))


if __name__ == "__main__":
    bad = check_file(sys.argv[1])
    for func, no, a, b, ws in bad:
        print(f"{sys.argv[1]}:{no}: in {func}: {ws} wait state(s) between\n    {a}\n    {b}")
    print(f"{len(bad)} MFMA pair(s) of different shapes, the second accumulating from the first, closer than the first's passes + 1 wait states")
    sys.exit(1 if bad else 0)
