"""GPU parity: ttt_mlp_bwd through the C ABI against the float64 oracle (itself pinned to torch
autograd in test_oracle_pins.py)."""
import importlib

import numpy as np
import pytest
import torch

from helpers import TOL, assert_close, np_inputs, to_dev
from oracle import ttt_oracle as orc
from test_mlp_fwd_gpu import mlp_case

pytestmark = pytest.mark.gpu

GRADS = ("d_xq", "d_xk", "d_xv", "d_W1", "d_b1", "d_W2", "d_b2", "d_lr", "d_token_eta", "d_gamma", "d_beta")


@pytest.fixture(scope="module")
def P():
    return importlib.import_module("ttt-rs_amd")


def run_case(P, B, H, d, K, N, dtype, style, state_grads=False, seed=0, kernel_hint=0):
    seq = N * K
    c = mlp_case(P, 300 + d + K + seed, B, H, seq, d, K, dtype, style)
    g = torch.Generator().manual_seed(77 + seed)
    d_out = torch.randn(B, H, seq, d, generator=g).to(dtype)
    dst = None
    if state_grads:
        m = 4 * d
        dst = [torch.randn(*s, generator=g) * 0.1 for s in ((B, H, d, m), (B, H, m), (B, H, m, d), (B, H, d))]
    dv = to_dev(c)
    got = P.ttt_mlp_backward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W1"], dv["b1"], dv["W2"], dv["b2"],
                                 dv["token_eta"], dv["lr"], dv["gamma"], dv["beta"], d_out.to("cuda:0"), K,
                                 d_state_out=None if dst is None else [x.to("cuda:0") for x in dst],
                                 kernel_hint=kernel_hint)
    torch.cuda.synchronize()
    n = np_inputs(c)
    ref = orc.mlp_backward(n["W1"], n["b1"], n["W2"], n["b2"], n["xq"], n["xk"], n["xv"], n["token_eta"], n["lr"],
                           n["gamma"], n["beta"], d_out.double().numpy(), K=K,
                           d_state_out=None if dst is None else [x.double().numpy() for x in dst])
    return got, ref


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("B,H,d,K,N,style,state_grads", [
    (2, 2, 32, 8, 3, "ref", False), (1, 2, 64, 16, 4, "ref", True), (1, 2, 96, 16, 3, "baseline", False),
    (1, 1, 128, 16, 2, "ref", False), (1, 2, 32, 16, 1, "ref", True)])
def test_mlp_bwd_matches_oracle(P, B, H, d, K, N, style, state_grads, dtype):
    print(f"case mlp bwd {style} B{B} H{H} d{d} K{K} N{N} {dtype} state_grads={state_grads}", flush=True)
    got, ref = run_case(P, B, H, d, K, N, dtype, style, state_grads)
    # bf16 rounds the stored activation gradients.  With bf16 I/O up to head_dim 96 the update factors the scan rolls
    # back and differentiates are those of the bf16-operand forward (rounded to bf16 as that forward applied them)
    # and the scan's own products take bf16 operands, so every gradient is held to the bf16 bar there;
    # f32 I/O and head_dim 128 (f32 forward sweep, f32 products) keep 1e-4 for the gradients stored in f32.
    bf16_factors = dtype == torch.bfloat16 and d <= 96
    for k in GRADS:
        io_out = k in ("d_xq", "d_xk", "d_xv", "d_lr")
        assert_close(got[k], ref[k], TOL[dtype] if (io_out or bf16_factors) else 1e-4, k,
                     min_frac=0.99 if bf16_factors else 0.999)


@pytest.mark.parametrize("d,N,style,sg", [(32, 3, "ref", False), (64, 4, "ref", True), (96, 3, "baseline", False)])
def test_mlp_bwd_bf16_with_f32_products(P, d, N, style, sg):
    """bf16 I/O up to head_dim 96: the scan with its products kept in f32 (TTT_HINT_F32_PRODUCTS) and the default scan
    (bf16 operands) are two compilations of the same kernel; both are held to the oracle, and to each other."""
    print(f"case mlp bwd bf16 f32-products d{d}", flush=True)
    got32, ref = run_case(P, 1, 2, d, 16, N, torch.bfloat16, style, sg, kernel_hint=P.TTT_HINT_F32_PRODUCTS)
    got16, _ = run_case(P, 1, 2, d, 16, N, torch.bfloat16, style, sg)
    tol = TOL[torch.bfloat16]
    for k in GRADS:
        assert_close(got32[k], ref[k], tol, k + " (f32 products)", min_frac=0.99)
        assert_close(got16[k], ref[k], tol, k + " (bf16 operands)", min_frac=0.99)
        assert_close(got16[k], got32[k].double().cpu().numpy(), tol, k + " (bf16 operands vs f32 products)", min_frac=0.99)


def test_mlp_bwd_is_linear_in_upstream_gradient(P):
    print("case mlp bwd linearity", flush=True)
    B, H, d, K, N = 1, 2, 64, 16, 3
    c = mlp_case(P, 411, B, H, N * K, d, K, torch.float32, "ref")
    dv = to_dev(c)
    g = torch.Generator().manual_seed(5)
    dO = torch.randn(B, H, N * K, d, generator=g).to("cuda:0")
    f = lambda x: P.ttt_mlp_backward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W1"], dv["b1"], dv["W2"], dv["b2"],
                                         dv["token_eta"], dv["lr"], dv["gamma"], dv["beta"], x, K)
    g1, g2 = f(dO), f(2.0 * dO)
    torch.cuda.synchronize()
    for k in GRADS:
        assert_close(g2[k], 2.0 * g1[k].double().cpu().numpy(), 1e-5, k)


def test_mlp_bwd_long_sequence_rollback(P):
    """128 mini-batches at the TTT-MLP benchmark head size: the state is rolled back 128 times from
    the final state, so this bounds the accumulated rounding of the roll-back."""
    print("case mlp bwd long", flush=True)
    got, ref = run_case(P, 1, 2, 96, 16, 128, torch.float32, "baseline", seed=3)
    for k in GRADS:
        assert_close(got[k], ref[k], 1e-4, k)


def test_mlp_inner_model_backward_from_parameters(P):
    """FusedMlp.backward with state0 = None: [H,..] parameters broadcast over batch; the parameter
    gradient is the batch sum of the per-batch state gradients."""
    print("case mlp model backward", flush=True)
    B, H, d, K, N = 2, 2, 32, 16, 2
    c = mlp_case(P, 512, B, H, N * K, d, K, torch.float32, "ref")
    dv = to_dev(c)
    model = P.FusedMlp(P.ModelConfig(H, d, P.TTTConfig(mini_batch_size=K)), dv["W1"], dv["b1"], dv["W2"],
                       dv["b2"], dv["gamma"], dv["beta"])
    g = torch.Generator().manual_seed(9)
    dO = torch.randn(B, H, N * K, d, generator=g)
    got = model.backward(None, P.TTTInputsInner(P.Qkv(dv["xq"], dv["xk"], dv["xv"]), dv["token_eta"], dv["lr"]),
                         dO.to("cuda:0"))
    torch.cuda.synchronize()
    n = np_inputs(c)
    ref = orc.mlp_backward(n["W1"], n["b1"], n["W2"], n["b2"], n["xq"], n["xk"], n["xv"], n["token_eta"], n["lr"],
                           n["gamma"], n["beta"], dO.double().numpy(), K=K)
    for k in GRADS:
        assert_close(got[k], ref[k], 1e-4, k)
    assert_close(got["d_W1"].sum(0), ref["d_W1"].sum(0), 1e-4, "parameter grad W1")


def test_mlp_bwd_d128_is_deterministic(P):
    """head_dim 128 is the variant at the register limit (the read-modify-write passes over the state prefetch one
    job ahead in a second register set).  Nothing in it may depend on timing: the same call twice gives the same
    bits in every output written by plain stores (the three outputs accumulated with floating-point atomics over
    units are compared to 1e-5)."""
    print("case mlp bwd d128 determinism", flush=True)
    B, H, d, K, N = 2, 2, 128, 16, 3
    for dtype in (torch.float32, torch.bfloat16):
        c = mlp_case(P, 640, B, H, N * K, d, K, dtype, "ref")
        dv = to_dev(c)
        g = torch.Generator().manual_seed(13)
        dO = torch.randn(B, H, N * K, d, generator=g).to(dtype).to("cuda:0")
        runs = []
        for _ in range(3):
            runs.append(P.ttt_mlp_backward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W1"], dv["b1"], dv["W2"], dv["b2"],
                                               dv["token_eta"], dv["lr"], dv["gamma"], dv["beta"], dO, K))
            torch.cuda.synchronize()
        for r in runs[1:]:
            for k in ("d_xq", "d_xk", "d_xv", "d_W1", "d_b1", "d_W2", "d_b2", "d_lr"):
                assert torch.equal(r[k], runs[0][k]), (k, dtype)
            for k in ("d_token_eta", "d_gamma", "d_beta"):
                assert_close(r[k], runs[0][k].double().cpu().numpy(), 1e-5, k)


@pytest.mark.parametrize("dtype,d,K,N", [(torch.bfloat16, 96, 16, 4), (torch.bfloat16, 64, 7, 3), (torch.bfloat16, 32, 16, 1),
                                         (torch.float32, 64, 16, 3), (torch.float32, 128, 16, 2)],
                         ids=["bf16-d96", "bf16-d64-K7", "bf16-d32-one", "f32-d64", "f32-d128"])
def test_mlp_forward_saving_and_backward_from_saved(P, dtype, d, K, N):
    """ttt_mlp_fwd_saving + ttt_mlp_bwd_saved against ttt_mlp_fwd + ttt_mlp_bwd: the same kernels without the backward's
    own forward sweep, so outputs, final state and the eight per-unit gradients are the same bits (the three that
    are accumulated with floating-point atomics to 1e-5); and against the oracle like the plain pair."""
    print(f"case mlp saving fwd + saved bwd {dtype} d{d} K{K} N{N}", flush=True)
    B, H = 2, 2
    c = mlp_case(P, 700 + d + K, B, H, N * K, d, K, dtype, "ref")
    g = torch.Generator().manual_seed(41)
    dO = torch.randn(B, H, N * K, d, generator=g).to(dtype)
    dv = to_dev(c)
    args = (dv["xq"], dv["xk"], dv["xv"], dv["W1"], dv["b1"], dv["W2"], dv["b2"], dv["token_eta"], dv["lr"], dv["gamma"],
            dv["beta"])
    plain_f = P.ttt_mlp_forward_raw(*args, K)
    plain_b = P.ttt_mlp_backward_raw(*args, dO.to("cuda:0"), K)
    sv = P.ttt_mlp_forward_raw(*args, K, save_for_backward=True)
    got = P.ttt_mlp_backward_raw(*args, dO.to("cuda:0"), K, saved=sv[5])
    torch.cuda.synchronize()
    for i, name in enumerate(("out", "W1", "b1", "W2", "b2")):
        assert torch.equal(sv[i], plain_f[i]), name
    for k in GRADS:
        if k in ("d_token_eta", "d_gamma", "d_beta"):
            assert_close(got[k], plain_b[k].double().cpu().numpy(), 1e-5, k)
        else:
            assert torch.equal(got[k], plain_b[k]), k
    n = np_inputs(c)
    ref = orc.mlp_backward(n["W1"], n["b1"], n["W2"], n["b2"], n["xq"], n["xk"], n["xv"], n["token_eta"], n["lr"],
                           n["gamma"], n["beta"], dO.double().numpy(), K=K)
    bf = dtype == torch.bfloat16
    for k in GRADS:
        io_out = k in ("d_xq", "d_xk", "d_xv", "d_lr")
        assert_close(got[k], ref[k], TOL[dtype] if (io_out or bf) else 1e-4, k, min_frac=0.99 if bf else 0.999)


def test_mlp_forward_saving_is_refused_on_pairs_of_cus(P):
    c = to_dev(mlp_case(P, 5, 1, 2, 32, 128, 16, torch.bfloat16, "ref"))
    with pytest.raises(P.TttError, match="pairs of CUs"):
        P.ttt_mlp_forward_raw(c["xq"], c["xk"], c["xv"], c["W1"], c["b1"], c["W2"], c["b2"], c["token_eta"], c["lr"],
                              c["gamma"], c["beta"], 16, save_for_backward=True)
