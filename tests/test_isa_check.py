"""The build's assembly scan (ttt-rs_amd/isa_check.py) and the hardware fact behind it.

CPU: the scanner flags a matrix instruction that takes its accumulator from one of another shape too closely behind
it (in place or into other registers, in text order or across a branch), and nothing else.  GPU: the library's self-test entry point runs such pairs at chosen distances; at the distance
the scanner demands the result is exact, and what the hardware does with closer pairs is printed for the record
(MI355X returns wrong sums; nothing is asserted about them, a later part may forward them correctly)."""
import ctypes as C
import importlib
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "ttt-rs_amd"))
import isa_check  # noqa: E402

sys.path.pop(0)

K32 = "\tv_mfma_f32_16x16x32_bf16 v[0:3], v[4:7], v[8:11], {c}"
K16 = "\tv_mfma_f32_16x16x16_bf16 {d}, v[20:21], v[22:23], {c}"
F32 = "\tv_mfma_f32_16x16x4_f32 v[0:3], v30, v31, v[0:3]"


def flagged(lines):
    return list(isa_check.scan(["kern:"] + lines))


def test_scanner_flags_a_scalar_select_on_a_vector_comparison():
    """The second rule of the scan: s_cselect reads SCC; a comparison on the vector unit sets VCC.  The sequence the
    compiler once produced for `lds_word != 0 ? a : b` (the word loaded from a wave-uniform LDS address) is reported,
    the repaired form (v_readfirstlane + s_cmp) and the ordinary mask idiom (v_cmp, s_and_b64, s_cselect_b64) are not."""
    wrong = ["kern:", "\ts_add_i32 s0, s23, 0", "\tv_mov_b32_e32 v0, s0", "\tds_read_b32 v0, v0", "\ts_waitcnt lgkmcnt(0)",
             "\tv_cmp_eq_u32_e32 vcc, 0, v0", "\ts_cselect_b32 s0, s22, -1"]
    bad = isa_check.scan_scc_select(wrong)
    assert len(bad) == 1 and bad[0][0] == "kern" and bad[0][1] == 7
    right = ["kern:", "\ts_add_i32 s0, s23, 0", "\tds_read_b32 v0, v0", "\ts_waitcnt lgkmcnt(0)", "\tv_readfirstlane_b32 s0, v0",
             "\ts_cmp_eq_u32 s0, 0", "\tv_cmp_eq_u32_e32 vcc, 0, v0", "\ts_cselect_b32 s0, s22, -1"]
    assert isa_check.scan_scc_select(right) == []
    mask = ["kern:", "\ts_lshl_b32 s4, s5, 2", "\tv_cmp_gt_i32_e32 vcc, 4, v1", "\ts_and_b64 s[6:7], vcc, exec",
            "\ts_cselect_b64 s[8:9], -1, 0"]
    assert isa_check.scan_scc_select(mask) == []
    # a label starts a new basic block: what set SCC in front of it is not known, nothing is reported
    assert isa_check.scan_scc_select(["kern:", "\ts_add_i32 s0, s1, 4", ".LBB0_2:", "\tv_cmp_eq_u32_e32 vcc, 0, v0",
                                      "\ts_cselect_b32 s0, s2, -1"]) == []
    # the library's own self-test functions are skipped, as in the first rule
    assert isa_check.scan_scc_select(["ttt_selftest_x:"] + wrong[1:]) == []


def test_scanner_flags_a_close_mixed_pair_in_place():
    assert len(flagged([K32.format(c="0"), K16.format(d="v[0:3]", c="v[0:3]")])) == 1
    assert len(flagged([K16.format(d="v[0:3]", c="0"), K32.format(c="v[0:3]")])) == 1
    # four wait states are too few, five are enough (s_nop n = n + 1; any instruction = 1)
    assert len(flagged([K32.format(c="0"), "\ts_nop 3", K16.format(d="v[0:3]", c="v[0:3]")])) == 1
    assert flagged([K32.format(c="0"), "\ts_nop 4", K16.format(d="v[0:3]", c="v[0:3]")]) == []
    four = ["\tv_add_f32_e32 v40, v41, v42"] * 4
    assert len(flagged([K32.format(c="0")] + four + [K16.format(d="v[0:3]", c="v[0:3]")])) == 1
    assert flagged([K32.format(c="0")] + four + ["\ts_waitcnt vmcnt(0)"] + [K16.format(d="v[0:3]", c="v[0:3]")]) == []
    # comments, directives and labels take no issue slot
    assert len(flagged([K32.format(c="0"), "; a comment", ".LBB0_1:", "\t.p2align 4", K16.format(d="v[0:3]", c="v[0:3]")])) == 1
    # an eight-pass first instruction needs nine
    assert len(flagged([F32, "\ts_nop 7", K16.format(d="v[0:3]", c="v[0:3]")])) == 1
    assert flagged([F32, "\ts_nop 7", "\ts_nop 0", K16.format(d="v[0:3]", c="v[0:3]")]) == []


def test_scanner_accepts_what_the_hardware_forwards():
    # the same shape back to back, in place
    assert flagged([K32.format(c="0"), K32.format(c="v[0:3]")]) == []
    assert flagged([K16.format(d="v[0:3]", c="0"), K16.format(d="v[0:3]", c="v[0:3]")]) == []
    # another shape reading the first's result as an A or B operand (interlocked by the hardware)
    assert flagged([K32.format(c="0"), "\tv_mfma_f32_16x16x16_bf16 v[12:15], v[0:1], v[2:3], 0"]) == []
    # another shape accumulating onto registers the first did not write
    assert flagged([K32.format(c="0"), K16.format(d="v[12:15]", c="v[12:15]")]) == []
    # the self-test kernel places such pairs on purpose
    assert list(isa_check.scan(["ttt_selftest_kernel:", K32.format(c="0"), K16.format(d="v[0:3]", c="v[0:3]")])) == []


def test_scanner_flags_a_mixed_pair_that_writes_elsewhere():
    """The accumulator input is what matters, not where the result goes: found in a forward kernel whose bias update
    (k = 16) the compiler had placed right in front of the next mini-batch's k = 32 product that starts from the bias."""
    assert len(flagged([K32.format(c="0"), K16.format(d="v[12:15]", c="v[0:3]")])) == 1
    assert len(flagged([K16.format(d="v[52:55]", c="v[52:55]"),
                        "\tv_mfma_f32_16x16x32_bf16 v[100:103], v[132:135], a[4:7], v[52:55]"])) == 1
    # partial overlap of the register ranges counts
    assert len(flagged([K32.format(c="0"), K16.format(d="v[12:15]", c="v[2:5]")])) == 1
    assert flagged([K32.format(c="0"), "\ts_nop 4", K16.format(d="v[12:15]", c="v[0:3]")]) == []


def test_scanner_follows_branches():
    loop = [".LBB0_1:", K32.format(c="v[12:15]"), "\tv_add_f32_e32 v40, v41, v42",
            K16.format(d="v[12:15]", c="v[12:15]"), "\ts_cbranch_scc1 .LBB0_1", "\ts_endpgm"]
    assert len(flagged(loop)) == 1          # the pair meets only across the back edge
    assert flagged([loop[0], "\ts_nop 4"] + loop[1:]) == []
    fwd = [K32.format(c="0"), "\ts_branch .LBB0_2", "\ts_nop 7", ".LBB0_2:", K16.format(d="v[0:3]", c="v[0:3]")]
    assert len(flagged(fwd)) == 1           # the s_nop is jumped over


def expected(order):
    a = lambda p, i, k: float((i * 7 + k * 3 + p * 5) % 7 - 3)
    b = lambda p, k, j: float((j * 5 + k * 11 + p * 3) % 7 - 3)
    ks = (32, 16) if order % 2 == 0 else (16, 32)
    D = np.zeros((16, 16))
    for p, kk in enumerate(ks):
        A = np.array([[a(p, i, k) for k in range(kk)] for i in range(16)])
        B = np.array([[b(p, k, j) for j in range(16)] for k in range(kk)])
        D += A @ B
    return D


@pytest.mark.gpu
def test_mixed_shapes_five_wait_states_apart_are_exact():
    import torch
    P = importlib.import_module("ttt-rs_amd")
    out = torch.empty(256, device="cuda:0")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    for order in (0, 1, 2, 3):  # 0, 1: the second instruction writes over its accumulator; 2, 3: into other registers
        want = expected(order)
        for gap in (5, 4, 0):
            print(f"case mfma mixed shapes order {order} gap {gap}", flush=True)
            out.fill_(float("nan"))
            P.check(P.lib().ttt_selftest_mfma_mixed(order, gap, C.c_void_p(out.data_ptr()), stream))
            torch.cuda.synchronize()
            got = out.cpu().double().numpy().reshape(16, 16)
            exact = np.array_equal(got, want)
            print(f"  order {order}, {gap} wait states: {'exact' if exact else 'WRONG (max abs error %.3g)' % np.nanmax(np.abs(got - want))}", flush=True)
            if gap == 5:
                assert exact, f"order {order}: five wait states between the two shapes no longer suffice"
    assert P.lib().ttt_selftest_mfma_mixed(4, 5, C.c_void_p(out.data_ptr()), stream) == P.TTT_ERR_SHAPE
