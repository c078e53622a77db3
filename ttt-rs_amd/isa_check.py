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

A second rule, described where it is implemented below (scan_scc_select), reports a scalar select that reads a
condition code which the vector comparison in front of it does not set.

Usage: python isa_check.py file.s      (exit status 1 and a listing if either rule finds something)
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


# ---- second rule: a scalar select on a vector comparison ---------------------------------------------------------
# hipcc (ROCm 7.2) takes a value loaded from a wave-uniform LDS address for uniform.  Seen in this library's code: the
# loaded word is compared on the vector unit (v_cmp ... vcc) and the result is then selected with s_cselect, which
# reads the SCALAR condition code -- set by whatever scalar instruction came last (an address addition), not by that
# comparison.  The kernel ran, and a status word read "given up" after a clean run.  Signature looked for, inside one
# basic block: [scalar ARITHMETIC that writes SCC as a by-product: s_add, s_sub, a shift, s_and_saveexec ...] ...
# v_cmp ... s_cselect, with nothing that writes SCC between the vector comparison and the select.  A scalar comparison
# or a logical operation on a mask (s_cmp*, s_bitcmp*, s_and_b64 ... whose SCC is what a select is meant to read) in
# that place is the ordinary, correct form and is not reported.  (The cure in source is to move the loaded word to a
# scalar register by hand, __builtin_amdgcn_readfirstlane, before it is compared.)
_SCC_ON_PURPOSE = ("s_cmp", "s_bitcmp", "s_and_b", "s_or_b", "s_xor_b", "s_andn2_b", "s_orn2_b", "s_not_b", "s_nand_b",
                   "s_nor_b", "s_xnor_b")
_NO_SCC = ("s_mov", "s_cmov", "s_load", "s_buffer_load", "s_waitcnt", "s_nop", "s_barrier", "s_branch", "s_cbranch",
           "s_cselect", "s_getreg", "s_setreg", "s_mul_i32", "s_mul_hi", "s_bfm", "s_movk", "s_sext", "s_ff1", "s_ff0",
           "s_flbit", "s_bitset", "s_getpc", "s_setpc", "s_swappc", "s_sleep", "s_sendmsg", "s_endpgm", "s_memtime",
           "s_memrealtime", "s_dcache", "s_icache", "s_setprio", "s_sethalt", "s_trap", "s_setvskip", "s_set_gpr",
           "s_brev", "s_bcnt0", "s_pack", "s_cmovk", "s_version", "s_code_end", "s_inst_prefetch", "s_clause",
           "s_incperflevel", "s_decperflevel", "s_ttrace", "s_rfe", "s_wakeup")


def scan_scc_select(lines):
    """[(function, line number, vector comparison, select)] for every s_cselect whose nearest SCC-writing
    predecessor in its basic block lies in front of a v_cmp that lies in front of the select."""
    bad = []
    func = "?"
    scc_seen = False   # the last SCC writer of this block wrote SCC as a by-product of arithmetic
    vcmp = None        # a vector comparison issued since that writer
    for no, raw in enumerate(lines, 1):
        line = raw.split(";")[0].strip()
        m = _FUNC.match(line)
        if m:
            func = m.group(1)
            scc_seen, vcmp = False, None
            continue
        if re.match(r"^\.L[\w.$]*:", line):  # a local label: a new basic block
            scc_seen, vcmp = False, None
            continue
        if not line or line.startswith(".") or line.startswith("//"):
            continue
        op = line.split()[0]
        if op.startswith("v_cmp"):
            if scc_seen:
                vcmp = (no, line)
            continue
        if op.startswith("s_cselect"):
            if vcmp is not None and "selftest" not in func:
                bad.append((func, no, vcmp[1], line))
            continue
        if op.startswith("s_") and not op.startswith(_NO_SCC):
            scc_seen, vcmp = not op.startswith(_SCC_ON_PURPOSE), None
    return bad


def check_scc_select_file(path: str):
    with open(path) as f:
        return scan_scc_select(f.readlines())


if __name__ == "__main__":
    bad = check_file(sys.argv[1])
    for func, no, a, b, ws in bad:
        print(f"{sys.argv[1]}:{no}: in {func}: {ws} wait state(s) between\n    {a}\n    {b}")
    print(f"{len(bad)} MFMA pair(s) of different shapes, the second accumulating from the first, closer than the first's passes + 1 wait states")
    sel = check_scc_select_file(sys.argv[1])
    for func, no, a, b in sel:
        print(f"{sys.argv[1]}:{no}: in {func}: scalar select on a vector comparison\n    {a}\n    {b}")
    print(f"{len(sel)} s_cselect instruction(s) behind a vector comparison with no scalar comparison between")
    sys.exit(1 if bad or sel else 0)
