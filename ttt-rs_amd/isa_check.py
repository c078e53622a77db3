"""Static check of the compiled gfx950 assembly for a matrix-instruction hazard that hipcc (ROCm 7.2) does not guard.

Measured on MI355X: a v_mfma that accumulates in place (SrcC == vDst) onto the result of an immediately preceding
v_mfma of a DIFFERENT opcode (seen with v_mfma_f32_16x16x32_bf16 followed by v_mfma_f32_16x16x16_bf16 and the
reverse) returns wrong sums unless at least five wait states separate the two; the same pair with the same opcode is
forwarded correctly back to back, and so is a pair whose second instruction writes other registers than it
accumulates from.  The compiler emits no wait states for the in-place mixed pair (with or without
-amdgpu-mfma-vgpr-form), and a memory wait that happens to fall between the two hides the error on some runs and
not on others.  Measured boundary for the two bf16 shapes (4 passes each): four wait states wrong, five right, i.e.
passes + 1, which is what a dependent read that is not forwarded needs.  This scan fails the build when the
generated code contains such a pair closer than passes + 1 wait states of the first instruction (8 passes for
v_mfma_f32_16x16x4_f32, 16 assumed for any opcode not listed), counting every instruction in between as one wait
state and `s_nop n` as n + 1.

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


def scan(lines):
    """Yields (function, line number, first instruction, second instruction, wait states between)."""
    func = "?"
    window = []  # recent MFMAs: [opcode, dst, wait states since, text, line]
    for no, raw in enumerate(lines, 1):
        line = raw.split(";")[0].rstrip()
        if not line.strip():
            continue
        f = _FUNC.match(line)
        if f and not line.startswith(".L") and not line.startswith("\t"):
            func, window = f.group(1), []
            continue
        s = line.strip()
        if s.startswith(".") or s.endswith(":"):
            continue  # directives and local labels take no issue slot
        m = _MFMA.match(line)
        if m:
            op, dst = m.group(1), (m.group(2), int(m.group(3)), int(m.group(4)))
            c = _srcc(m.group(5))
            if c is not None and c == dst and "selftest" not in func:
                for w in window:
                    if w[1] == dst and w[0] != op and w[2] < min_wait_states(w[0]):
                        yield func, no, w[3], s, w[2]
        states = 1
        n = re.match(r"s_nop\s+(\d+)", s)
        if n:
            states = int(n.group(1)) + 1
        # a write to the same registers by anything else ends the dependence; keeping the entry is conservative
        window = [[w[0], w[1], w[2] + states, w[3], w[4]] for w in window if w[2] + states < MAX_WINDOW]
        if m:
            # the new instruction supersedes older writers of the same registers
            window = [w for w in window if w[1] != dst]
            window.append([op, dst, 0, s, no])


def check_file(path: str):
    with open(path) as fh:
        return list(scan(fh))


if __name__ == "__main__":
    bad = check_file(sys.argv[1])
    for func, no, a, b, ws in bad:
        print(f"{sys.argv[1]}:{no}: in {func}: {ws} wait state(s) between\n    {a}\n    {b}")
    print(f"{len(bad)} mixed in-place MFMA pair(s) closer than the first instruction's passes + 1 wait states")
    sys.exit(1 if bad else 0)
