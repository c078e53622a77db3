"""GPU parity: ttt_linear_bwd_ws on two workgroups per unit (f32 I/O, head_dim 32 / 64, one checkpoint per
mini-batch) against the float64 oracle backward and against ttt_linear_bwd on one workgroup per unit.

The two kernels evaluate the same expressions; the compiler is free to fuse multiply-adds differently in each, so they
are compared to a few ulps of f32 (1e-5 of the tensor's largest magnitude), not bit for bit; every gradient of both
is held to the oracle at the f32 bar (reference tolerance, rust/core/src/test_utils.rs:473-607).
"""
import importlib

import numpy as np
import pytest
import torch

from helpers import TOL, assert_close, np_inputs, to_dev
from oracle import ttt_oracle as orc

pytestmark = pytest.mark.gpu

NAMES = [("grad_xq", "d_xq"), ("grad_xk", "d_xk"), ("grad_xv", "d_xv"), ("grad_weight", "d_W0"),
         ("grad_bias", "d_b0"), ("grad_ttt_lr_eta", "d_lr"), ("grad_token_eta", "d_token_eta"),
         ("grad_ln_weight", "d_gamma"), ("grad_ln_bias", "d_beta")]


@pytest.fixture(scope="module")
def P():
    return importlib.import_module("ttt-rs_amd")


def fwd_bwd(P, c, dO, K, packed, workspace, hint=0, state_grads=None):
    d = to_dev(c)
    out, W, b, Wc, bc = P.ttt_linear_forward_raw(d["xq"], d["xk"], d["xv"], d["W0"], d["b0"], d["token_eta"],
                                                 d["lr"], d["gamma"], d["beta"], K, 1e-6, 1,
                                                 want_checkpoints=True, packed_checkpoints=packed)
    gw = gb = None
    if state_grads is not None:
        gw, gb = (x.to("cuda:0") for x in state_grads)
    g = P.ttt_linear_backward_raw(d["xq"], d["xk"], d["xv"], d["W0"], d["b0"], d["token_eta"], d["lr"],
                                  d["gamma"], d["beta"], Wc, bc, dO.to("cuda:0"), K, 1e-6, 1, gw, gb,
                                  packed_checkpoints=packed, kernel_hint=hint, workspace=workspace)
    torch.cuda.synchronize()
    return g


def oracle_bwd(c, dO, K, state_grads=None):
    n = np_inputs(c)
    kw = {}
    if state_grads is not None:
        kw = dict(d_W_out=state_grads[0].double().numpy(), d_b_out=state_grads[1].double().numpy())
    return orc.linear_backward(n["W0"], n["b0"], n["xq"], n["xk"], n["xv"], n["token_eta"], n["lr"],
                               n["gamma"], n["beta"], dO.double().numpy(), K=K, **kw)


def close_to_each_other(a, b, what):
    for gn, _ in NAMES:
        x, y = a[gn].double().cpu(), b[gn].double().cpu()
        scale = float(y.abs().max()) + 1e-30
        err = float((x - y).abs().max()) / scale
        assert err <= 1e-5, f"{what}: {gn} differs by {err:.2e} of its largest magnitude"


def workspace_bytes(P, B, H, seq, d, K, packed, hint=0):
    import ctypes as C
    desc = P.TttDesc(B, H, seq, d, K, 1e-6, 1, P._lib.TTT_F32, 0, 0, int(packed), hint)
    return P.lib().ttt_linear_bwd_workspace_bytes(C.byref(desc))


# (B, H, d, K, mini-batches)
CASES = [(2, 2, 32, 8, 2), (2, 2, 32, 8, 4), (1, 2, 64, 16, 3), (2, 3, 64, 16, 8), (1, 2, 64, 5, 3),
         (1, 1, 64, 16, 2), (3, 5, 64, 16, 7), (1, 17, 32, 16, 9), (2, 4, 64, 11, 6)]


@pytest.mark.parametrize("packed", [False, True], ids=["rowmajor", "packed"])
@pytest.mark.parametrize("B,H,d,K,N", CASES)
def test_two_workgroups_match_oracle_and_one_workgroup(P, B, H, d, K, N, packed):
    print(f"case linear bwd pair B{B} H{H} d{d} K{K} N{N} packed{packed}", flush=True)
    assert workspace_bytes(P, B, H, N * K, d, K, packed) > 0
    c = P.synthetic.reference_test_inputs(300 + B + H + d + K + N, B, H, N * K, d, K)
    dO = torch.randn(B, H, N * K, d, generator=torch.Generator().manual_seed(11))
    before = P.mlp_fwd_lost_workgroups()
    two = fwd_bwd(P, c, dO, K, packed, None)
    one = fwd_bwd(P, c, dO, K, packed, False)
    assert P.mlp_fwd_lost_workgroups() == before
    ref = oracle_bwd(c, dO, K)
    for gn, rn in NAMES:
        assert_close(two[gn], ref[rn], TOL[torch.float32], "two workgroups " + gn)
        assert_close(one[gn], ref[rn], TOL[torch.float32], "one workgroup " + gn)
    close_to_each_other(two, one, "two against one workgroup")


def test_two_workgroups_baseline_style_inputs_and_state_gradients(P):
    """N(0,1) activations, sigmoid lr / d (benchmark config 2 style), upstream gradients of the final state."""
    print("case linear bwd pair baseline-style + state grads", flush=True)
    B, H, d, K, N = 2, 3, 64, 16, 8
    c = P.synthetic.baseline_inputs(2, B, H, N * K, d, K, io_dtype=torch.float32, with_dout=True)
    dO = c.pop("d_out")
    g = torch.Generator().manual_seed(6)
    sg = (torch.randn(B, H, d, d, generator=g), torch.randn(B, H, d, generator=g))
    for packed in (False, True):
        two = fwd_bwd(P, c, dO, K, packed, None, state_grads=sg)
        ref = oracle_bwd(c, dO, K, sg)
        for gn, rn in NAMES:
            assert_close(two[gn], ref[rn], TOL[torch.float32], f"packed{packed} " + gn)


def test_two_workgroups_repeat_and_caller_workspace(P):
    """A caller-owned workspace reused across calls (nothing in it has to be kept or cleared): the same bits every
    time, apart from the three outputs summed over units by atomic additions."""
    print("case linear bwd pair repeat", flush=True)
    B, H, d, K, N = 2, 4, 64, 16, 6
    c = P.synthetic.reference_test_inputs(41, B, H, N * K, d, K)
    dO = torch.randn(B, H, N * K, d, generator=torch.Generator().manual_seed(12))
    nbytes = workspace_bytes(P, B, H, N * K, d, K, True)
    ws = torch.full((nbytes,), 0xA5, dtype=torch.uint8, device="cuda:0")
    runs = [fwd_bwd(P, c, dO, K, True, ws) for _ in range(3)]
    for r in runs[1:]:
        for gn in ("grad_xq", "grad_xk", "grad_xv", "grad_weight", "grad_bias", "grad_ttt_lr_eta"):
            assert torch.equal(r[gn], runs[0][gn]), gn
    # a smaller problem in the same workspace afterwards
    c2 = P.synthetic.reference_test_inputs(42, 1, 3, 3 * K, d, K)
    dO2 = torch.randn(1, 3, 3 * K, d, generator=torch.Generator().manual_seed(13))
    small = fwd_bwd(P, c2, dO2, K, True, ws)
    ref = oracle_bwd(c2, dO2, K)
    for gn, rn in NAMES:
        assert_close(small[gn], ref[rn], TOL[torch.float32], "smaller problem " + gn)


def test_pair_on_two_xcds_takes_device_scope_release(P):
    """TTT_HINT_TEST_OTHER_XCD keeps the producer on the path of a pair that does not share an L2."""
    print("case linear bwd pair other xcd", flush=True)
    B, H, d, K, N = 2, 3, 64, 16, 5
    c = P.synthetic.reference_test_inputs(43, B, H, N * K, d, K)
    dO = torch.randn(B, H, N * K, d, generator=torch.Generator().manual_seed(14))
    fast = fwd_bwd(P, c, dO, K, True, None)
    wide = fwd_bwd(P, c, dO, K, True, None, hint=P.TTT_HINT_TEST_OTHER_XCD)
    for gn in ("grad_xq", "grad_xk", "grad_xv", "grad_weight", "grad_bias", "grad_ttt_lr_eta"):
        assert torch.equal(fast[gn], wide[gn]), gn


def test_lost_partner_is_loud(P):
    """Both workgroups of every unit give up waiting at once (TTT_HINT_TEST_LOST_PARTNER): the kernel runs to its end,
    every unit's grad_bias is NaN and the status word counts the workgroups."""
    print("case linear bwd pair lost partner", flush=True)
    B, H, d, K, N = 2, 3, 64, 16, 4
    c = P.synthetic.reference_test_inputs(44, B, H, N * K, d, K)
    dO = torch.randn(B, H, N * K, d, generator=torch.Generator().manual_seed(15))
    before = P.mlp_fwd_lost_workgroups()
    got = fwd_bwd(P, c, dO, K, True, None, hint=P.TTT_HINT_TEST_LOST_PARTNER)
    assert bool(torch.isnan(got["grad_bias"]).all()), "grad_bias of every unit must be NaN"
    assert P.mlp_fwd_lost_workgroups() - before == 2 * B * H
    ok = fwd_bwd(P, c, dO, K, True, None)
    ref = oracle_bwd(c, dO, K)
    for gn, rn in NAMES:
        assert_close(ok[gn], ref[rn], TOL[torch.float32], "call after a lost partner " + gn)
    assert P.mlp_fwd_lost_workgroups() - before == 2 * B * H


def test_no_workspace_where_the_pair_does_not_apply(P):
    """bf16 I/O, more than 128 units, coarser checkpoints, TTT_HINT_ONE_WORKGROUP: size zero, and ttt_linear_bwd_ws is
    ttt_linear_bwd."""
    print("case linear bwd pair not applicable", flush=True)
    assert workspace_bytes(P, 2, 2, 64, 64, 16, False, P.TTT_HINT_ONE_WORKGROUP) == 0
    assert workspace_bytes(P, 16, 12, 64, 64, 16, False) == 0
    assert workspace_bytes(P, 2, 2, 16, 64, 16, False) == 0  # a single mini-batch
    B, H, d, K, N = 1, 2, 64, 16, 3
    c = P.synthetic.reference_test_inputs(45, B, H, N * K, d, K)
    dO = torch.randn(B, H, N * K, d, generator=torch.Generator().manual_seed(16))
    a = fwd_bwd(P, c, dO, K, False, None, hint=P.TTT_HINT_ONE_WORKGROUP)
    b = fwd_bwd(P, c, dO, K, False, False)
    for gn in ("grad_xq", "grad_xk", "grad_xv", "grad_weight", "grad_bias", "grad_ttt_lr_eta"):
        assert torch.equal(a[gn], b[gn]), gn
