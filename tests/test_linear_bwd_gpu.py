"""GPU parity: ttt_linear_bwd (through the C ABI) against the float64 oracle backward, which is
itself pinned to torch autograd through the primal formulation (tests/test_oracle_pins.py).

Shapes mirror the reference's multi-stage backward tests
(rust/fused/src/linear_fused_tile/tests.rs:68-89: (2,2,32,8) with 1,2,4 stages and
checkpoint intervals 1,2,4) plus d=64 / K=16 cases.  Unlike the reference's tests
(rust/core/src/test_utils.rs:473-607) the LayerNorm parameter gradients are compared too.
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


def run_bwd(P, c, dO, K, ci, state_grads=None, bwd_hint=0):
    d = to_dev(c)
    out, W, b, Wc, bc = P.ttt_linear_forward_raw(d["xq"], d["xk"], d["xv"], d["W0"], d["b0"], d["token_eta"],
                                                 d["lr"], d["gamma"], d["beta"], K, 1e-6, ci,
                                                 want_checkpoints=True)
    gw = gb = None
    if state_grads is not None:
        gw, gb = (x.to("cuda:0") for x in state_grads)
    g = P.ttt_linear_backward_raw(d["xq"], d["xk"], d["xv"], d["W0"], d["b0"], d["token_eta"], d["lr"],
                                  d["gamma"], d["beta"], Wc, bc, dO.to("cuda:0"), K, 1e-6, ci, gw, gb,
                                  kernel_hint=bwd_hint)
    torch.cuda.synchronize()
    return g


def oracle_bwd(c, dO, K, state_grads=None):
    n = np_inputs(c)
    kw = {}
    if state_grads is not None:
        kw = dict(d_W_out=state_grads[0].double().numpy(), d_b_out=state_grads[1].double().numpy())
    return orc.linear_backward(n["W0"], n["b0"], n["xq"], n["xk"], n["xv"], n["token_eta"], n["lr"],
                               n["gamma"], n["beta"], dO.double().numpy(), K=K, **kw)


NAMES = [("grad_xq", "d_xq"), ("grad_xk", "d_xk"), ("grad_xv", "d_xv"), ("grad_weight", "d_W0"),
         ("grad_bias", "d_b0"), ("grad_ttt_lr_eta", "d_lr"), ("grad_token_eta", "d_token_eta"),
         ("grad_ln_weight", "d_gamma"), ("grad_ln_bias", "d_beta")]


def compare(g, r, tol):
    for gn, rn in NAMES:
        # bf16 I/O, products with bf16 operands: in a tensor of fewer than 1000 elements a single element
        # outside the elementwise band is already more than 0.1 %, so one such element is let through there
        n = np.asarray(r[rn]).size
        min_frac = 0.999 if tol < 1e-3 else min(0.999, 1.0 - 1.5 / n)
        assert_close(g[gn], r[rn], tol, gn, min_frac=min_frac)


# (B, H, d, K, stages, checkpoint_interval)
CASES = [(2, 2, 32, 8, 1, 1), (2, 2, 32, 8, 2, 1), (2, 2, 32, 8, 4, 2), (2, 2, 32, 8, 4, 4),
         (1, 2, 64, 16, 3, 1), (2, 3, 64, 16, 8, 3), (1, 2, 64, 5, 3, 2)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("B,H,d,K,N,ci", CASES)
def test_bwd_matches_oracle_reference_style_inputs(P, B, H, d, K, N, ci, dtype):
    print(f"case bwd ref-style B{B} H{H} d{d} K{K} N{N} ci{ci} {dtype}", flush=True)
    c = P.synthetic.reference_test_inputs(100 + B + d + K + N + ci, B, H, N * K, d, K, io_dtype=dtype)
    g = torch.Generator().manual_seed(5)
    # reference backward tests differentiate output.sum(): dOut = 1; use random dOut as well
    dO = torch.randn(B, H, N * K, d, generator=g).to(dtype)
    compare(run_bwd(P, c, dO, K, ci), oracle_bwd(c, dO, K), TOL[dtype])
    ones = torch.ones(B, H, N * K, d).to(dtype)
    compare(run_bwd(P, c, ones, K, ci), oracle_bwd(c, ones, K), TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_bwd_matches_oracle_baseline_style_inputs(P, dtype):
    """N(0,1) activations, gamma=1, beta=0, sigmoid lr/d, dOut ~ N(0,1) (benchmark config 2 style)."""
    print(f"case bwd baseline-style {dtype}", flush=True)
    B, H, d, K, N = 2, 2, 64, 16, 8
    if d == 64 and K == 16:  # benchmark-style inputs at the benchmark's head size
        c = P.synthetic.baseline_inputs(2, B, H, N * K, d, K, io_dtype=dtype, with_dout=True)
        dO = c.pop("d_out")
        compare(run_bwd(P, c, dO, K, 1), oracle_bwd(c, dO, K), TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("d,K", [(32, 8), (64, 16)])
def test_bwd_with_upstream_state_gradients(P, d, K, dtype):
    """d_W_out / d_b_out (the reference assumes zero, launch.rs:188-194; the ABI accepts them)."""
    print(f"case bwd state grads d{d} K{K} {dtype}", flush=True)
    B, H, N = 2, 2, 3
    c = P.synthetic.reference_test_inputs(77, B, H, N * K, d, K, io_dtype=dtype)
    g = torch.Generator().manual_seed(6)
    dO = torch.randn(B, H, N * K, d, generator=g).to(dtype)
    sg = (torch.randn(B, H, d, d, generator=g), torch.randn(B, H, d, generator=g))
    compare(run_bwd(P, c, dO, K, 1, sg), oracle_bwd(c, dO, K, sg), TOL[dtype])


def test_bwd_bf16_lds_kernel_on_request(P):
    """The LDS-tile kernel (f32 products) stays selectable for bf16 I/O."""
    print("case bwd bf16 lds kernel", flush=True)
    B, H, d, K, N = 1, 2, 64, 16, 3
    c = P.synthetic.reference_test_inputs(79, B, H, N * K, d, K, io_dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(8)
    dO = torch.randn(B, H, N * K, d, generator=g).to(torch.bfloat16)
    compare(run_bwd(P, c, dO, K, 1, bwd_hint=P.TTT_HINT_LDS_TILES), oracle_bwd(c, dO, K), TOL[torch.bfloat16])


def test_bwd_is_linear_in_upstream_gradient(P):
    print("case bwd linearity", flush=True)
    B, H, d, K, N = 1, 2, 64, 16, 4
    c = P.synthetic.reference_test_inputs(78, B, H, N * K, d, K)
    g = torch.Generator().manual_seed(7)
    dO = torch.randn(B, H, N * K, d, generator=g)
    g1 = run_bwd(P, c, dO, K, 2)
    g3 = run_bwd(P, c, 3.0 * dO, K, 2)
    for k in g1:
        assert_close(g3[k], 3.0 * g1[k].double(), 1e-5, k)


MW_CASES = [(2, 2, 32, 8, 1), (2, 2, 32, 8, 2), (1, 2, 64, 16, 3), (2, 3, 64, 16, 8), (1, 2, 64, 5, 3)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("B,H,d,K,N", MW_CASES)
def test_bwd_multi_wave_kernel(P, B, H, d, K, N, dtype):
    """The feature-split kernel (several waves per (batch, head), exchanges through LDS), forced for both
    I/O types; with upstream state gradients so that every term of the scan is exercised."""
    print(f"case bwd multi-wave B{B} H{H} d{d} K{K} N{N} {dtype}", flush=True)
    c = P.synthetic.reference_test_inputs(300 + B + d + K + N, B, H, N * K, d, K, io_dtype=dtype)
    g = torch.Generator().manual_seed(9)
    dO = torch.randn(B, H, N * K, d, generator=g).to(dtype)
    sg = (0.1 * torch.randn(B, H, d, d, generator=g), 0.1 * torch.randn(B, H, d, generator=g))
    compare(run_bwd(P, c, dO, K, 1, sg, bwd_hint=4), oracle_bwd(c, dO, K, sg), TOL[dtype])
    if d == 64 and K == 16:  # benchmark-style inputs at the benchmark's head size
        c = P.synthetic.baseline_inputs(2, B, H, N * K, d, K, io_dtype=dtype, with_dout=True)
        dO = c.pop("d_out")
        compare(run_bwd(P, c, dO, K, 1, bwd_hint=4), oracle_bwd(c, dO, K), TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("B,H,d,K,N", [(1, 2, 96, 16, 3), (2, 1, 96, 7, 2), (1, 2, 128, 16, 3)])
def test_bwd_wide_heads(P, B, H, d, K, N, dtype):
    """head_dim 96 and 128: the feature-split kernel; f32 I/O at head_dim 128 (its f32 staging does not fit a CU) the
    LDS-tile kernel with the state read in place from the checkpoints and the state gradient kept in d_W0."""
    print(f"case bwd wide B{B} H{H} d{d} K{K} N{N} {dtype}", flush=True)
    c = P.synthetic.reference_test_inputs(400 + B + d + K + N, B, H, N * K, d, K, io_dtype=dtype)
    g = torch.Generator().manual_seed(10)
    dO = torch.randn(B, H, N * K, d, generator=g).to(dtype)
    sg = (0.1 * torch.randn(B, H, d, d, generator=g), 0.1 * torch.randn(B, H, d, generator=g))
    compare(run_bwd(P, c, dO, K, 1, sg), oracle_bwd(c, dO, K, sg), TOL[dtype])
    if K == 16:
        c = P.synthetic.baseline_inputs(4, B, H, N * K, d, K, io_dtype=dtype, with_dout=True)
        dO = c.pop("d_out")
        compare(run_bwd(P, c, dO, K, 1), oracle_bwd(c, dO, K), TOL[dtype])


def test_bwd_head_dim_128_needs_a_checkpoint_per_mini_batch(P):
    c = P.synthetic.reference_test_inputs(1, 1, 1, 32, 128, 16)
    with pytest.raises(Exception, match="checkpoint_interval 1"):
        run_bwd(P, c, torch.ones(1, 1, 32, 128), 16, 2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("B,H,K,N,ci", [(1, 2, 16, 4, 2), (2, 1, 7, 5, 3), (1, 2, 16, 6, 6)])
def test_bwd_head_dim_96_with_coarser_checkpoints(P, B, H, K, N, ci, dtype):
    """head_dim 96 with a checkpoint every ci mini-batches: the LDS-tile kernel re-simulates the state in LDS and keeps
    the state gradient in the d_W0 buffer."""
    print(f"case bwd d96 ci{ci} B{B} H{H} K{K} N{N} {dtype}", flush=True)
    c = P.synthetic.reference_test_inputs(430 + B + K + N + ci, B, H, N * K, 96, K, io_dtype=dtype)
    g = torch.Generator().manual_seed(12)
    dO = torch.randn(B, H, N * K, 96, generator=g).to(dtype)
    sg = (0.1 * torch.randn(B, H, 96, 96, generator=g), 0.1 * torch.randn(B, H, 96, generator=g))
    compare(run_bwd(P, c, dO, K, ci, sg), oracle_bwd(c, dO, K, sg), TOL[dtype])
    compare(run_bwd(P, c, dO, K, ci), oracle_bwd(c, dO, K), TOL[dtype])


def test_bwd_f32_head_dim_128_longer_sequence(P):
    """f32 I/O at head_dim 128 over 24 mini-batches and two batch entries (per-batch checkpoints read in place)."""
    print("case bwd f32 d128 long", flush=True)
    B, H, d, K, N = 2, 2, 128, 16, 24
    c = P.synthetic.baseline_inputs(6, B, H, N * K, d, K, with_dout=True)
    dO = c.pop("d_out")
    compare(run_bwd(P, c, dO, K, 1), oracle_bwd(c, dO, K), 1e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("waves", ["1", "4"])
@pytest.mark.parametrize("B,H,d,K,N", [(2, 2, 32, 8, 3), (2, 3, 64, 16, 8), (1, 2, 64, 5, 3), (1, 2, 96, 16, 3), (1, 2, 128, 16, 3)])
def test_bwd_packed_checkpoints_change_nothing(P, B, H, d, K, N, waves, dtype):
    """Checkpoints stored as operand fragments in kernel order (bf16 I/O: as bf16).  The forward's outputs do not
    depend on the checkpoint format at all.  The backward works on the state minus its row means either way: a
    packed checkpoint holds that difference as the forward had it, an f32 row-major checkpoint holds the state
    itself and the backward subtracts the row means again, which reproduces the difference to an ulp of the
    state.  So the two runs agree far inside the parity tolerance (f32: 1e-5; bf16 operands: where that ulp
    moves a value across a bf16 rounding boundary a single operand changes by 2^-8, hence 5e-3), not bit for bit."""
    if (d > 64 or dtype == torch.float32) and waves == "1":
        pytest.skip("wide heads and f32 I/O have the feature-split kernel only")
    if d == 128 and dtype == torch.float32:
        pytest.skip("f32 I/O at head_dim 128 reads f32 row-major checkpoints only")
    print(f"case bwd packed ckpt B{B} H{H} d{d} K{K} N{N} waves {waves} {dtype}", flush=True)
    c = P.synthetic.reference_test_inputs(500 + B + d + K + N, B, H, N * K, d, K, io_dtype=dtype)
    dv = to_dev(c)
    g = torch.Generator().manual_seed(11)
    dO = torch.randn(B, H, N * K, d, generator=g).to(dtype).to("cuda:0")
    res = []
    for packed in (False, True):
        out, W, b, Wc, bc = P.ttt_linear_forward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W0"], dv["b0"], dv["token_eta"],
                                                     dv["lr"], dv["gamma"], dv["beta"], K, 1e-6, 1,
                                                     want_checkpoints=True, packed_checkpoints=packed)
        gr = P.ttt_linear_backward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W0"], dv["b0"], dv["token_eta"], dv["lr"],
                                       dv["gamma"], dv["beta"], Wc, bc, dO, K, 1e-6, 1, packed_checkpoints=packed,
                                       kernel_hint=int(waves))
        torch.cuda.synchronize()
        res.append((out, W, b, gr))
    assert torch.equal(res[0][0], res[1][0]) and torch.equal(res[0][1], res[1][1]) and torch.equal(res[0][2], res[1][2])
    for k in res[0][3]:
        assert_close(res[1][3][k], res[0][3][k].double(), 1e-5 if dtype == torch.float32 else 5e-3, k, min_frac=0.99)
    compare(res[1][3], oracle_bwd(c, dO.cpu(), K), TOL[dtype])


@pytest.mark.parametrize("B,H,d,K,N", [(2, 2, 32, 8, 3), (2, 3, 64, 16, 8), (1, 2, 64, 5, 3), (1, 2, 96, 16, 3),
                                       (1, 2, 64, 16, 1), (1, 3, 64, 16, 2), (1, 2, 64, 16, 40), (1, 2, 96, 16, 24),
                                       (2, 1, 32, 16, 48), (1, 2, 96, 7, 5)])
@pytest.mark.parametrize("eta_last", ["positive", "zero"])
def test_bwd_from_update_factors(P, B, H, d, K, N, eta_last):
    """checkpoint_format 2 (bf16 I/O): the forward saves the final state and the [16 x d] factor of every state
    update instead of the states; the backward walks the state back from the end with the operands the forward
    multiplied.  The forward's outputs do not depend on the format beyond the last bit (the forward that saves
    factors is a compilation of its own, free to fuse a multiply and an add where the other does not).  The
    recovered states differ from the saved ones by f32 roundings, which move a bf16 operand here and there, as the two state formats differ among themselves:
    the gradients agree with those from packed states to 5e-3 and with the oracle to the bf16 bar.  One mini-batch
    (N = 1) is saved packed by the library; token_eta[K-1] = 0 means the forward never changed the state and the
    walk back must not either."""
    dtype = torch.bfloat16
    print(f"case bwd factor ckpt B{B} H{H} d{d} K{K} N{N} eta_last {eta_last}", flush=True)
    c = P.synthetic.reference_test_inputs(700 + B + d + K + N, B, H, N * K, d, K, io_dtype=dtype)
    if eta_last == "zero":
        c["token_eta"] = c["token_eta"].clone()
        c["token_eta"][K - 1] = 0.0
    dv = to_dev(c)
    g = torch.Generator().manual_seed(12)
    dO = torch.randn(B, H, N * K, d, generator=g).to(dtype).to("cuda:0")
    res = []
    for fmt in (1, 2):
        out, W, b, Wc, bc = P.ttt_linear_forward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W0"], dv["b0"], dv["token_eta"],
                                                     dv["lr"], dv["gamma"], dv["beta"], K, 1e-6, 1,
                                                     want_checkpoints=True, packed_checkpoints=fmt)
        gr = P.ttt_linear_backward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W0"], dv["b0"], dv["token_eta"], dv["lr"],
                                       dv["gamma"], dv["beta"], Wc, bc, dO, K, 1e-6, 1, packed_checkpoints=fmt)
        torch.cuda.synchronize()
        res.append((out, W, b, gr))
    assert_close(res[1][0], res[0][0].double(), 2.0 ** -7, "out")
    assert_close(res[1][1], res[0][1].double(), 1e-5, "W")
    assert_close(res[1][2], res[0][2].double(), 1e-5, "b")
    for k in res[0][3]:
        assert_close(res[1][3][k], res[0][3][k].double(), 5e-3, k, min_frac=0.99)
    compare(res[1][3], oracle_bwd(c, dO.cpu(), K), TOL[dtype])


def test_update_factors_and_the_wave_hint(P):
    """Only the feature-split backward walks the state back: a hint that asks for the single-wave kernel changes
    nothing, bit for bit (non-atomic outputs); a hint of two waves selects the two-wave feature-split kernel (the
    library's choice between 257 and 512 units), whose gradients agree with the four-wave kernel's to rounding and
    with the oracle to the bf16 bar."""
    B, H, d, K, N = 2, 2, 64, 16, 5
    c = P.synthetic.reference_test_inputs(811, B, H, N * K, d, K, io_dtype=torch.bfloat16)
    dv = to_dev(c)
    dO = torch.randn(B, H, N * K, d, generator=torch.Generator().manual_seed(13)).to(torch.bfloat16)
    fw = P.ttt_linear_forward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W0"], dv["b0"], dv["token_eta"], dv["lr"],
                                  dv["gamma"], dv["beta"], K, 1e-6, 1, want_checkpoints=True, packed_checkpoints=2)
    res = [P.ttt_linear_backward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W0"], dv["b0"], dv["token_eta"], dv["lr"],
                                     dv["gamma"], dv["beta"], fw[3], fw[4], dO.to("cuda:0"), K, 1e-6, 1,
                                     packed_checkpoints=2, kernel_hint=hint) for hint in (0, 1, 2)]
    torch.cuda.synchronize()
    for k in ("grad_xq", "grad_xk", "grad_xv", "grad_weight", "grad_bias", "grad_ttt_lr_eta"):
        assert torch.equal(res[0][k], res[1][k]), k
        assert_close(res[2][k], res[0][k].double(), 5e-3, "two waves " + k, min_frac=0.99)
    compare(res[2], oracle_bwd(c, dO, K), TOL[torch.bfloat16])


def test_update_factors_rejected_where_unsupported(P):
    c = P.synthetic.reference_test_inputs(2, 1, 1, 64, 32, 16)
    dv = to_dev(c)
    with pytest.raises(Exception, match="update-factor checkpoints"):
        P.ttt_linear_forward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W0"], dv["b0"], dv["token_eta"], dv["lr"],
                                 dv["gamma"], dv["beta"], 16, 1e-6, 1, want_checkpoints=True, packed_checkpoints=2)


def test_packed_checkpoints_rejected_where_unsupported(P):
    c = P.synthetic.reference_test_inputs(2, 1, 1, 64, 32, 16)
    dv = to_dev(c)
    with pytest.raises(Exception, match="packed checkpoints"):
        P.ttt_linear_forward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W0"], dv["b0"], dv["token_eta"], dv["lr"],
                                 dv["gamma"], dv["beta"], 16, 1e-6, 2, want_checkpoints=True, packed_checkpoints=True)


def test_bwd_gives_eta_logit_gradients_as_the_fwd_bwd_configuration_asks(P):
    """Benchmark-style inputs (lr = base_lr * sigmoid(logits) / d): the gradient w.r.t. the logits, i.e.
    grad_ttt_lr_eta chained through the gate (rust/layer/src/ttt.rs:205-227), against the oracle's chain, which
    tests/test_oracle_pins.py pins by finite differences through the forward."""
    B, H, d, K, N = 2, 3, 64, 16, 4
    print(f"case bwd eta logits B{B} H{H} d{d} K{K} N{N}", flush=True)
    c = P.synthetic.baseline_inputs(2, B, H, N * K, d, K, io_dtype=torch.float32, with_dout=True)
    logits = c.pop("lr_logits")
    dO = c.pop("d_out")
    g = run_bwd(P, c, dO, K, 1)
    got = P.ttt_lr_eta_logit_grad(g["grad_ttt_lr_eta"], logits.to("cuda:0"), 1.0, d)
    r = oracle_bwd(c, dO, K)
    ref = orc.lr_logit_grad(r["d_lr"], logits.double().numpy(), 1.0, d)
    assert_close(got, ref, 1e-4, "grad_lr_logits")
