"""GPU tests of the TTT-MLP reverse scan on two workgroups per (batch, head) unit (the library's choice up to 128
units: a producer workgroup walks the state back and recomputes the forward's intermediates one mini-batch ahead of
the consumer workgroup that carries the gradient).  The arithmetic is that of the one-workgroup kernel in the same
order, so the two are compared bit for bit (d_token_eta, summed over the units with atomic additions, to rounding);
the comparison with the oracle is test_mlp_bwd_gpu.py's, which runs on two workgroups wherever the units allow."""
import importlib

import numpy as np
import pytest
import torch

from helpers import TOL, assert_close, np_inputs, to_dev
from oracle import ttt_oracle as orc
from test_mlp_bwd_gpu import GRADS, run_case
from test_mlp_fwd_gpu import mlp_case

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def P():
    return importlib.import_module("ttt-rs_amd")


def call(P, c, d_out, K, hint, dst=None):
    dv = to_dev(c)
    got = P.ttt_mlp_backward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W1"], dv["b1"], dv["W2"], dv["b2"],
                                 dv["token_eta"], dv["lr"], dv["gamma"], dv["beta"], d_out.to("cuda:0"), K,
                                 d_state_out=None if dst is None else [x.to("cuda:0") for x in dst], kernel_hint=hint)
    torch.cuda.synchronize()
    return got


def same_bits(a, b, what):
    for k in GRADS:
        x, y = a[k].float().cpu().numpy(), b[k].float().cpu().numpy()
        if k in ("d_token_eta", "d_gamma", "d_beta"):  # atomic additions over units: their order is not fixed
            np.testing.assert_allclose(x, y, rtol=1e-5, atol=1e-6 * max(1.0, float(np.abs(y).max())), err_msg=f"{what}: {k}")
        else:
            assert np.array_equal(x, y, equal_nan=False), f"{what}: {k} differs, max |diff| {np.abs(x - y).max():.3e}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("B,H,d,K,N,sg", [(1, 1, 32, 16, 1, False), (2, 2, 32, 8, 2, True), (1, 3, 64, 16, 5, False),
                                          (3, 3, 96, 16, 4, True), (1, 2, 128, 16, 3, False), (2, 5, 64, 5, 6, False),
                                          (1, 8, 96, 16, 7, False), (1, 17, 32, 16, 3, False)])
def test_two_workgroups_match_one_bit_for_bit(P, B, H, d, K, N, sg, dtype):
    print(f"case mlp bwd pipe B{B} H{H} d{d} K{K} N{N} sg={sg} {dtype}", flush=True)
    seq = N * K
    c = mlp_case(P, 900 + d + K + N, B, H, seq, d, K, dtype, "baseline" if d == 96 else "ref")
    g = torch.Generator().manual_seed(31 + N)
    d_out = torch.randn(B, H, seq, d, generator=g).to(dtype)
    m = 4 * d
    dst = [torch.randn(*s, generator=g) * 0.1 for s in ((B, H, d, m), (B, H, m), (B, H, m, d), (B, H, d))] if sg else None
    two = call(P, c, d_out, K, 0, dst)
    one = call(P, c, d_out, K, P.TTT_HINT_ONE_WORKGROUP, dst)
    same_bits(two, one, "two workgroups vs one")
    # the producer publishing with a device-scope release on every mini-batch (the path of a pair that does not share an L2)
    wide = call(P, c, d_out, K, P.TTT_HINT_TEST_OTHER_XCD, dst)
    same_bits(wide, one, "device-scope release vs one workgroup")
    again = call(P, c, d_out, K, 0, dst)
    same_bits(again, two, "second call")


@pytest.mark.parametrize("dtype,d", [(torch.float32, 64), (torch.bfloat16, 96)], ids=["f32-d64", "bf16-d96"])
def test_one_workgroup_kernel_still_matches_oracle(P, dtype, d):
    """The one-workgroup kernel serves more than 128 units and TTT_HINT_ONE_WORKGROUP; the other oracle tests no
    longer reach it at their sizes."""
    print(f"case mlp bwd one workgroup vs oracle d{d} {dtype}", flush=True)
    got, ref = run_case(P, 1, 2, d, 16, 3, dtype, "ref", True, kernel_hint=P.TTT_HINT_ONE_WORKGROUP)
    bf = dtype == torch.bfloat16
    for k in GRADS:
        io_out = k in ("d_xq", "d_xk", "d_xv", "d_lr")
        assert_close(got[k], ref[k], TOL[dtype] if (io_out or bf) else 1e-4, k, min_frac=0.99 if bf else 0.999)


def test_more_units_than_pairs_of_cus_run_on_one_workgroup(P):
    """129 units: the library keeps every unit on one workgroup (two would no longer be resident together)."""
    print("case mlp bwd 129 units", flush=True)
    B, H, d, K, N = 3, 43, 32, 16, 2
    c = mlp_case(P, 77, B, H, N * K, d, K, torch.bfloat16, "ref")
    d_out = torch.randn(B, H, N * K, d, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
    a = call(P, c, d_out, K, 0)
    b = call(P, c, d_out, K, P.TTT_HINT_ONE_WORKGROUP)
    same_bits(a, b, "129 units")
    n = np_inputs(c)
    sl = slice(1, 2)
    ref = orc.mlp_backward(n["W1"], n["b1"], n["W2"], n["b2"], n["xq"][sl], n["xk"][sl], n["xv"][sl], n["token_eta"],
                           n["lr"][sl], n["gamma"], n["beta"], d_out[sl].double().numpy(), K=K)
    for k in ("d_xq", "d_xk", "d_xv", "d_lr", "d_W1", "d_W2"):
        assert_close(a[k][sl], ref[k], TOL[torch.bfloat16], k, min_frac=0.99)


def test_lost_partner_is_loud(P):
    """Both workgroups of every unit give up waiting at once (TTT_HINT_TEST_LOST_PARTNER): all kernels run to their
    end, every unit's d_b1 is NaN and the status word counts the workgroups."""
    print("case mlp bwd pipe lost partner", flush=True)
    B, H, d, K, N = 2, 3, 64, 16, 4
    c = mlp_case(P, 5, B, H, N * K, d, K, torch.float32, "ref")
    d_out = torch.randn(B, H, N * K, d, generator=torch.Generator().manual_seed(4))
    before = P.mlp_fwd_lost_workgroups()
    got = call(P, c, d_out, K, P.TTT_HINT_TEST_LOST_PARTNER)
    assert bool(torch.isnan(got["d_b1"]).all()), "d_b1 of every unit must be NaN"
    assert P.mlp_fwd_lost_workgroups() - before == 2 * B * H
    # and the next ordinary call is unaffected
    ok = call(P, c, d_out, K, 0)
    one = call(P, c, d_out, K, P.TTT_HINT_ONE_WORKGROUP)
    same_bits(ok, one, "call after a lost partner")
    assert P.mlp_fwd_lost_workgroups() - before == 2 * B * H


def test_saved_pair_and_static_scratch_use_two_workgroups(P):
    """ttt_mlp_bwd_saved and ttt_mlp_bwd_static take the same path as ttt_mlp_bwd: same bits."""
    print("case mlp bwd pipe saved/static", flush=True)
    B, H, d, K, N = 1, 4, 96, 16, 5
    dtype = torch.bfloat16
    c = mlp_case(P, 15, B, H, N * K, d, K, dtype, "baseline")
    d_out = torch.randn(B, H, N * K, d, generator=torch.Generator().manual_seed(8)).to(dtype)
    plain = call(P, c, d_out, K, 0)
    dv = to_dev(c)
    fw = P.ttt_mlp_forward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W1"], dv["b1"], dv["W2"], dv["b2"], dv["token_eta"],
                               dv["lr"], dv["gamma"], dv["beta"], K, save_for_backward=True)
    sv = P.ttt_mlp_backward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W1"], dv["b1"], dv["W2"], dv["b2"], dv["token_eta"],
                                dv["lr"], dv["gamma"], dv["beta"], d_out.to("cuda:0"), K, saved=fw[5])
    st = P.ttt_mlp_backward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W1"], dv["b1"], dv["W2"], dv["b2"], dv["token_eta"],
                                dv["lr"], dv["gamma"], dv["beta"], d_out.to("cuda:0"), K, static_scratch=True)
    torch.cuda.synchronize()
    same_bits(sv, plain, "saved")
    same_bits(st, plain, "static scratch")
