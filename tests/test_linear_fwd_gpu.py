"""GPU parity: ttt_linear_fwd (through the C ABI) against the float64 oracle.

Shapes mirror the reference's own fused-vs-Burn tests
(rust/fused/src/linear_fused_tile/tests.rs:23-66) plus the benchmark's config 0.
"""
import importlib

import numpy as np
import pytest
import torch

from helpers import TOL, assert_close, np_inputs, to_dev
from oracle import ttt_oracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def P():
    return importlib.import_module("ttt-rs_amd")


def run_case(P, c, K, ci=1, ckpt=False, per_batch=False):
    d = to_dev(c)
    W, b = d["W0"], d["b0"]
    if per_batch:
        B = d["xq"].shape[0]
        W = W.unsqueeze(0).repeat(B, 1, 1, 1)
        b = b.unsqueeze(0).repeat(B, 1, 1)
    res = P.ttt_linear_forward_raw(d["xq"], d["xk"], d["xv"], W, b, d["token_eta"], d["lr"],
                                   d["gamma"], d["beta"], K, 1e-6, ci, want_checkpoints=ckpt)
    torch.cuda.synchronize()
    return res


def oracle_case(c, K, ci=0):
    n = np_inputs(c)
    return orc.linear_forward(n["W0"], n["b0"], n["xq"], n["xk"], n["xv"], n["token_eta"], n["lr"],
                              n["gamma"], n["beta"], K=K, checkpoint_interval=ci)


# (B, H, d, K, stages) -- reference tile tests: tests.rs:23-66; last rows: config-0 shape and d=64 multi
SHAPES = [(2, 2, 32, 8, 1), (1, 4, 32, 16, 1), (2, 2, 64, 8, 1), (2, 2, 32, 8, 4), (1, 4, 32, 8, 2),
          (1, 4, 64, 16, 16), (3, 2, 64, 16, 5), (2, 3, 32, 5, 3), (1, 1, 64, 1, 4)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("B,H,d,K,N", SHAPES)
def test_fwd_matches_oracle_reference_style_inputs(P, B, H, d, K, N, dtype):
    print(f"case ref-style B{B} H{H} d{d} K{K} N{N} {dtype}", flush=True)
    c = P.synthetic.reference_test_inputs(7 + B + d + K + N, B, H, N * K, d, K, io_dtype=dtype)
    out, W, b = run_case(P, c, K)
    ro, rW, rb = oracle_case(c, K)
    tol = TOL[dtype]
    assert_close(out, ro, tol, "out")
    assert_close(W, rW, tol, "W_out")
    assert_close(b, rb, tol, "b_out")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("B,H,d,K,N", [(1, 4, 64, 16, 16), (2, 2, 32, 16, 8)])
def test_fwd_matches_oracle_baseline_style_inputs(P, B, H, d, K, N, dtype):
    """N(0,1) activations, sigmoid lr / d, gamma=1, beta=0 (benchmark config 0 is the first row)."""
    print(f"case baseline-style B{B} H{H} d{d} K{K} N{N} {dtype}", flush=True)
    c = P.synthetic.baseline_inputs(0, B, H, N * K, d, K, io_dtype=dtype)
    out, W, b = run_case(P, c, K)
    ro, rW, rb = oracle_case(c, K)
    tol = TOL[dtype]
    assert_close(out, ro, tol, "out")
    assert_close(W, rW, tol, "W_out")
    assert_close(b, rb, tol, "b_out")


@pytest.mark.parametrize("ci", [1, 2, 4, 5])
def test_checkpoints_hold_state_entering_stage(P, ci):
    print(f"case checkpoints ci={ci}", flush=True)
    B, H, d, K, N = 2, 2, 64, 16, 9
    c = P.synthetic.reference_test_inputs(3, B, H, N * K, d, K)
    out, W, b, Wc, bc = run_case(P, c, K, ci=ci, ckpt=True, per_batch=True)
    ro, rW, rb, rWc, rbc = oracle_case(c, K, ci=ci)
    assert Wc.shape == rWc.shape and bc.shape == rbc.shape
    assert_close(out, ro, 1e-4, "out")
    assert_close(Wc, rWc, 1e-4, "W_ckpt")
    assert_close(bc, rbc, 1e-4, "b_ckpt")
    # first checkpoint is the initial state: the kernels carry the state minus its row means and add them back
    # when they write a checkpoint, so it is reproduced to an ulp of the larger of the two, not bit for bit
    w0 = c["W0"].unsqueeze(0).expand(B, H, d, d)
    assert (Wc[:, :, 0].cpu() - w0).abs().max() <= 2.0 ** -22 * w0.abs().max()
    # the final state of a sequence that never updates it IS the initial state bit for bit (test_lr_zero_...)


def test_lr_zero_leaves_state_untouched(P):
    print("case lr=0", flush=True)
    B, H, d, K, N = 2, 2, 64, 16, 3
    c = P.synthetic.reference_test_inputs(5, B, H, N * K, d, K)
    c["lr"].zero_()
    out, W, b = run_case(P, c, K)
    assert torch.equal(W.cpu(), c["W0"].unsqueeze(0).expand(B, H, d, d))
    assert torch.equal(b.cpu(), c["b0"].unsqueeze(0).expand(B, H, d))
    ro, _, _ = oracle_case(c, K)
    assert_close(out, ro, 1e-4, "out")


def test_chained_single_stage_calls_equal_multi_stage(P):
    """reference tests.rs:49-66."""
    print("case chained", flush=True)
    B, H, d, K, N = 2, 2, 32, 8, 4
    c = to_dev(P.synthetic.reference_test_inputs(11, B, H, N * K, d, K))
    out, W, b = P.ttt_linear_forward_raw(c["xq"], c["xk"], c["xv"], c["W0"], c["b0"], c["token_eta"],
                                         c["lr"], c["gamma"], c["beta"], K)
    Ws = c["W0"].unsqueeze(0).repeat(B, 1, 1, 1)
    bs = c["b0"].unsqueeze(0).repeat(B, 1, 1)
    outs = []
    for t in range(N):
        sl = slice(t * K, (t + 1) * K)
        o, Ws, bs = P.ttt_linear_forward_raw(c["xq"][:, :, sl].contiguous(), c["xk"][:, :, sl].contiguous(),
                                             c["xv"][:, :, sl].contiguous(), Ws, bs, c["token_eta"],
                                             c["lr"][:, :, sl].contiguous(), c["gamma"], c["beta"], K)
        outs.append(o)
    torch.cuda.synchronize()
    # every call splits its initial state into row means and the rest afresh, so the chain and the single call round
    # differently in the last bits: they agree far inside the parity tolerance, not bit for bit
    assert_close(torch.cat(outs, 2), out.double().cpu().numpy(), 1e-5, "chained out")
    assert_close(Ws, W.double().cpu().numpy(), 1e-5, "chained W")
    assert_close(bs, b.double().cpu().numpy(), 1e-5, "chained b")


def test_inner_model_forward_with_remainder(P):
    """Host class: full mini-batches in one launch, trailing remainder as one short
    mini-batch (rust/core/src/inner.rs:40-47)."""
    print("case remainder", flush=True)
    B, H, d, K, seq = 2, 2, 64, 16, 16 * 3 + 5
    c = P.synthetic.reference_test_inputs(13, B, H, seq, d, K)
    te_seq = c["token_eta"].repeat(seq // K + 1)[:seq]
    dv = to_dev(c)
    model = P.FusedTileMulti(P.ModelConfig(H, d, P.TTTConfig(mini_batch_size=K)), dv["W0"], dv["b0"],
                             dv["gamma"], dv["beta"])
    assert model.name() == "FusedTileMultiTTTLinear"
    state = model.init_state(B)
    inputs = P.TTTInputsInner(P.Qkv(dv["xq"], dv["xk"], dv["xv"]), te_seq.to("cuda:0"), dv["lr"])
    out = model.forward(state, inputs)
    torch.cuda.synchronize()
    n = np_inputs(c)
    ro, rW, rb = orc.linear_forward(n["W0"], n["b0"], n["xq"], n["xk"], n["xv"], te_seq.double().numpy(),
                                    n["lr"], n["gamma"], n["beta"], K=K)
    assert_close(out, ro, 1e-4, "out")
    assert_close(state.weight, rW, 1e-4, "W")
    assert_close(state.bias, rb, 1e-4, "b")


@pytest.mark.parametrize("d", [64, 128])
def test_sequence_windows_in_place(P, d):
    """desc.seq_stride: a window of a longer sequence is processed where it lies (inputs, lr and
    the output share the pitch); the result equals the packed call bit for bit."""
    print(f"case windows d={d}", flush=True)
    B, H, K, seq = 2, 2, 16, 16 * 6
    c = to_dev(P.synthetic.reference_test_inputs(21, B, H, seq, d, K))
    lo, hi = 32, 80
    win = lambda t: t[:, :, lo:hi]
    out_full = torch.full_like(c["xq"], float("nan"))
    o1, W1, b1 = P.ttt_linear_forward_raw(win(c["xq"]), win(c["xk"]), win(c["xv"]), c["W0"], c["b0"],
                                          c["token_eta"], win(c["lr"]), c["gamma"], c["beta"], K,
                                          out=win(out_full))
    o2, W2, b2 = P.ttt_linear_forward_raw(win(c["xq"]).contiguous(), win(c["xk"]).contiguous(),
                                          win(c["xv"]).contiguous(), c["W0"], c["b0"], c["token_eta"],
                                          win(c["lr"]).contiguous(), c["gamma"], c["beta"], K)
    torch.cuda.synchronize()
    assert o1.data_ptr() == win(out_full).data_ptr()
    assert torch.equal(o1, o2) and torch.equal(W1, W2) and torch.equal(b1, b2)
    assert torch.isnan(out_full[:, :, :lo]).all() and torch.isnan(out_full[:, :, hi:]).all()


@pytest.mark.parametrize("fmt", [0, 1], ids=["rowmajor", "packed"])
@pytest.mark.parametrize("B,H,d,N", [(1, 4, 64, 16), (3, 2, 64, 5), (2, 3, 32, 3), (1, 1, 64, 1), (2, 2, 32, 2), (1, 2, 64, 9)])
def test_f32_forward_with_control_wave_equals_forward_with_own_loads(P, B, H, d, N, fmt):
    """f32 I/O, whole mini-batches of 16 tokens, a CU per workgroup: the library's choice is the kernel with a control
    wave that copies the operands global -> LDS (the compute waves issue no loads); TTT_HINT_ALL_LOADS keeps the loads in
    the compute waves.  Same arithmetic in the same order: the same bits, output, final state and checkpoints; and the
    oracle holds the library's choice at the f32 bar."""
    print(f"case f32 fwd control wave B{B} H{H} d{d} N{N} fmt{fmt}", flush=True)
    K = 16
    c = P.synthetic.reference_test_inputs(61 + B + H + d + N, B, H, N * K, d, K)
    dv = to_dev(c)

    def run(hint):
        r = P.ttt_linear_forward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W0"], dv["b0"], dv["token_eta"], dv["lr"],
                                     dv["gamma"], dv["beta"], K, 1e-6, 1, want_checkpoints=True,
                                     packed_checkpoints=fmt, kernel_hint=hint)
        torch.cuda.synchronize()
        return r

    ctl, own, again = run(0), run(P.TTT_HINT_ALL_LOADS), run(0)
    for name, x, y, z in zip(("out", "W", "b", "W_ckpt", "b_ckpt"), ctl, own, again):
        assert torch.equal(x, y), f"{name}: control wave against own loads"
        assert torch.equal(x, z), f"{name}: second call"
    ro, rW, rb = oracle_case(c, K)
    assert_close(ctl[0], ro, TOL[torch.float32], "out")
    assert_close(ctl[1], rW, TOL[torch.float32], "W")
    assert_close(ctl[2], rb, TOL[torch.float32], "b")
