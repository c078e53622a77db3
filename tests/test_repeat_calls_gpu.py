"""GPU: every register-resident kernel called three times on the same inputs gives the same bits, and its short
mini-batch cases (K < 16, three or more mini-batches) match the oracle.

Why both in one place.  These kernels mix the two bf16 matrix-instruction forms (k = 16 and k = 32) and wait for
their global->LDS copies with counted waits ("all but the n youngest memory operations").  A matrix instruction that
accumulates in place onto the result of one of the other form too soon, or a wait that counts one store too many,
does not fail every time: it reads a value that is sometimes there already.  The symptom is a result that changes
between calls, or that is wrong only for some mini-batch lengths.  So each variant (kernel, waves per unit,
checkpoint format) is held to bit equality across calls for every output written by plain stores, and to the
oracle at mini-batch lengths below 16, where the masked rows are the ones an undercounted wait would read early.
"""
import importlib

import pytest
import torch

from helpers import TOL, assert_close, to_dev
from test_linear_bwd_gpu import compare, oracle_bwd
from test_mlp_fwd_gpu import mlp_case

pytestmark = pytest.mark.gpu

PLAIN_LINEAR = ("grad_xq", "grad_xk", "grad_xv", "grad_weight", "grad_bias", "grad_ttt_lr_eta")
ATOMIC_LINEAR = ("grad_token_eta", "grad_ln_weight", "grad_ln_bias")


@pytest.fixture(scope="module")
def P():
    return importlib.import_module("ttt-rs_amd")


def same_bits(runs, what):
    for r in runs[1:]:
        for i, (x, y) in enumerate(zip(runs[0], r)):
            if x is None:
                assert y is None
                continue
            assert torch.equal(x, y), f"{what}: output {i} differs between calls"


@pytest.mark.parametrize("fmt", [None, 0, 1, 2], ids=["no-ckpt", "f32-ckpt", "packed", "factors"])
@pytest.mark.parametrize("hint", [0, 1])
@pytest.mark.parametrize("d,K", [(32, 16), (64, 16), (64, 7), (96, 16), (96, 5), (128, 16), (128, 3)])
def test_linear_fwd_repeat_calls(P, d, K, hint, fmt):
    """bf16 forward: the skewed multi-wave kernel (default) and the single-wave kernel (hint 1), without checkpoints
    and with each checkpoint format (the forward that saves update factors is a compilation of its own)."""
    if fmt == 2 and d > 96:
        pytest.skip("update factors exist up to head_dim 96")
    B, H, N = 2, 3, 5
    print(f"case fwd repeat d{d} K{K} hint{hint} fmt{fmt}", flush=True)
    c = P.synthetic.reference_test_inputs(900 + d + K, B, H, N * K, d, K, io_dtype=torch.bfloat16)
    dv = to_dev(c)
    runs = []
    for _ in range(3):
        r = P.ttt_linear_forward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W0"], dv["b0"], dv["token_eta"], dv["lr"],
                                     dv["gamma"], dv["beta"], K, 1e-6, 1, want_checkpoints=fmt is not None,
                                     packed_checkpoints=fmt or 0, kernel_hint=hint)
        torch.cuda.synchronize()
        # packed and factor checkpoints fill only part of their f32-sized allocations (the rest is whatever the
        # allocator handed out), so those tensors are compared through what the backward makes of them, below
        runs.append(tuple(r) if fmt in (None, 0) else tuple(r[:3]))
    same_bits(runs, f"forward d{d} K{K} hint{hint} fmt{fmt}")


# (d, K, mini-batches, waves hint): every NW / tiles-per-wave combination of the feature-split backward and the
# single-wave kernel (bf16, head_dim <= 64)
BWD_CASES = [(32, 16, 4, 0), (32, 7, 4, 0), (32, 7, 4, 1), (64, 16, 4, 0), (64, 7, 5, 0), (64, 3, 4, 2), (64, 7, 4, 1),
             (96, 16, 3, 0), (96, 7, 4, 0), (128, 16, 3, 0), (128, 5, 4, 0), (32, 32, 3, 0), (32, 21, 4, 0)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("fmt", [0, 1, 2], ids=["f32-ckpt", "packed", "factors"])
@pytest.mark.parametrize("d,K,N,hint", BWD_CASES)
def test_linear_bwd_repeat_calls_and_short_mini_batches(P, d, K, N, hint, fmt, dtype):
    f32 = dtype == torch.float32
    if fmt == 2 and (f32 or d > 96):
        pytest.skip("update factors: bf16 I/O up to head_dim 96")
    if K > 16 and fmt != 0:
        pytest.skip("mini-batches of more than 16 tokens: f32 row-major checkpoints only")
    if f32 and hint == 1:
        pytest.skip("f32 I/O: no single-wave kernel")
    if f32 and d == 128 and fmt != 0:
        pytest.skip("f32 I/O at head_dim 128 reads f32 row-major checkpoints only")
    if hint == 1 and d > 64:
        pytest.skip("single-wave kernel up to head_dim 64")
    B, H = 2, 2
    print(f"case bwd repeat d{d} K{K} N{N} hint{hint} fmt{fmt} {dtype}", flush=True)
    c = P.synthetic.reference_test_inputs(950 + d + K + N, B, H, N * K, d, K, io_dtype=dtype)
    dv = to_dev(c)
    dO = torch.randn(B, H, N * K, d, generator=torch.Generator().manual_seed(21)).to(dtype)
    dOd = dO.to("cuda:0")
    fw = P.ttt_linear_forward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W0"], dv["b0"], dv["token_eta"], dv["lr"],
                                  dv["gamma"], dv["beta"], K, 1e-6, 1, want_checkpoints=True, packed_checkpoints=fmt)
    runs = []
    for _ in range(3):
        g = P.ttt_linear_backward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W0"], dv["b0"], dv["token_eta"], dv["lr"],
                                      dv["gamma"], dv["beta"], fw[3], fw[4], dOd, K, 1e-6, 1, packed_checkpoints=fmt,
                                      kernel_hint=hint)
        torch.cuda.synchronize()
        runs.append(g)
    for r in runs[1:]:
        for k in PLAIN_LINEAR:
            assert torch.equal(r[k], runs[0][k]), f"{k} differs between calls"
        for k in ATOMIC_LINEAR:  # floating-point atomics over units: the order of the additions is not fixed
            assert_close(r[k], runs[0][k].double().cpu().numpy(), 1e-5, k)
    compare(runs[0], oracle_bwd(c, dO, K), TOL[dtype])


@pytest.mark.parametrize("hint_name", ["default", "two-cu"])
@pytest.mark.parametrize("d,K", [(32, 16), (64, 16), (64, 7), (96, 16), (96, 5), (128, 16), (128, 7)])
def test_mlp_fwd_repeat_calls(P, d, K, hint_name):
    """bf16 TTT-MLP forward: the one-CU register-resident kernel (head_dim <= 96) and the two-CU kernel
    (head_dim 128; head_dim 96 with TTT_HINT_TWO_CU)."""
    if hint_name == "two-cu" and d != 96:
        pytest.skip("the hint selects another kernel at head_dim 96 only")
    hint = P.TTT_HINT_TWO_CU if hint_name == "two-cu" else 0
    B, H, N = 2, 2, 5
    print(f"case mlp fwd repeat d{d} K{K} {hint_name}", flush=True)
    c = mlp_case(P, 970 + d + K, B, H, N * K, d, K, torch.bfloat16, "ref")
    dv = to_dev(c)
    runs = []
    for _ in range(3):
        r = P.ttt_mlp_forward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W1"], dv["b1"], dv["W2"], dv["b2"], dv["token_eta"],
                                  dv["lr"], dv["gamma"], dv["beta"], K, kernel_hint=hint)
        torch.cuda.synchronize()
        runs.append(tuple(r))
    same_bits(runs, f"mlp forward d{d} K{K} {hint_name}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("d,K", [(32, 7), (64, 16), (96, 16), (96, 5)])
def test_mlp_bwd_repeat_calls(P, d, K, dtype):
    """TTT-MLP backward (its forward sweep is the register-resident forward for bf16 I/O up to head_dim 96);
    head_dim 128 has its own test in test_mlp_bwd_gpu.py."""
    B, H, N = 2, 2, 4
    print(f"case mlp bwd repeat d{d} K{K} {dtype}", flush=True)
    c = mlp_case(P, 990 + d + K, B, H, N * K, d, K, dtype, "ref")
    dv = to_dev(c)
    dO = torch.randn(B, H, N * K, d, generator=torch.Generator().manual_seed(23)).to(dtype).to("cuda:0")
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


@pytest.mark.parametrize("fmt", [None, 0, 1, 2], ids=["no-ckpt", "f32-ckpt", "packed", "factors"])
@pytest.mark.parametrize("B,H,K,N", [(2, 3, 16, 5), (1, 2, 7, 4), (1, 1, 16, 1), (2, 2, 16, 2), (3, 2, 5, 7)])
def test_linear_fwd_own_loads_variant_gives_the_same_bits(P, B, H, K, N, fmt):
    """bf16, head_dim 64, two waves per unit: the variant in which a wave loads only the features it owns and the
    full rows cross LDS (the library's choice above 256 units; TTT_HINT_OWN_LOADS asks for it at any size) against
    the variant in which every wave loads every row (TTT_HINT_ALL_LOADS): the same arithmetic on the same values."""
    if fmt == 2 and N < 2:
        pytest.skip("one mini-batch is saved packed")
    d = 64
    print(f"case fwd own loads B{B} H{H} K{K} N{N} fmt{fmt}", flush=True)
    c = P.synthetic.reference_test_inputs(1200 + K + N, B, H, N * K, d, K, io_dtype=torch.bfloat16)
    dv = to_dev(c)
    runs = []
    for hint in (P.TTT_HINT_ALL_LOADS, P.TTT_HINT_OWN_LOADS, P.TTT_HINT_OWN_LOADS):
        r = P.ttt_linear_forward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W0"], dv["b0"], dv["token_eta"], dv["lr"],
                                     dv["gamma"], dv["beta"], K, 1e-6, 1, want_checkpoints=fmt is not None,
                                     packed_checkpoints=fmt or 0, kernel_hint=hint)
        torch.cuda.synchronize()
        runs.append(tuple(r) if fmt in (None, 0) else tuple(r[:3]))
    same_bits(runs, f"forward own/all loads K{K} N{N} fmt{fmt}")
    if fmt in (1, 2):  # what the backward makes of the saved state must agree as well
        dO = torch.randn(B, H, N * K, d, generator=torch.Generator().manual_seed(31)).to(torch.bfloat16).to("cuda:0")
        gs = []
        for hint in (P.TTT_HINT_ALL_LOADS, P.TTT_HINT_OWN_LOADS):
            fw = P.ttt_linear_forward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W0"], dv["b0"], dv["token_eta"], dv["lr"],
                                          dv["gamma"], dv["beta"], K, 1e-6, 1, want_checkpoints=True,
                                          packed_checkpoints=fmt, kernel_hint=hint)
            gs.append(P.ttt_linear_backward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W0"], dv["b0"], dv["token_eta"],
                                                dv["lr"], dv["gamma"], dv["beta"], fw[3], fw[4], dO, K, 1e-6, 1,
                                                packed_checkpoints=fmt))
        torch.cuda.synchronize()
        for k in PLAIN_LINEAR:
            assert torch.equal(gs[0][k], gs[1][k]), k
