"""GPU parity: ttt_mlp_fwd and the LDS-resident TTT-Linear forward (head_dim 96/128) through the
C ABI against the float64 oracle."""
import importlib

import pytest
import torch

from helpers import TOL, assert_close, np_inputs, to_dev
from oracle import ttt_oracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def P():
    return importlib.import_module("ttt-rs_amd")


def mlp_case(P, seed, B, H, seq, d, K, dtype, style):
    if style == "baseline":
        return P.synthetic.baseline_inputs(3, B, H, seq, d, K, io_dtype=dtype, mlp=True)
    c = P.synthetic.reference_test_inputs(seed, B, H, seq, d, K, io_dtype=dtype)
    g = torch.Generator().manual_seed(seed + 1)
    n = lambda *s: torch.randn(*s, generator=g) * 0.02
    c.pop("W0"), c.pop("b0")
    c["W1"], c["b1"], c["W2"], c["b2"] = n(H, d, 4 * d), n(H, 4 * d), n(H, 4 * d, d), n(H, d)
    return c


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("style", ["ref", "baseline"])
@pytest.mark.parametrize("B,H,d,K,N", [(2, 2, 32, 8, 3), (1, 2, 64, 16, 4), (2, 2, 96, 16, 4),
                                       (1, 2, 128, 16, 3), (1, 1, 96, 7, 2)])
def test_mlp_fwd_matches_oracle(P, B, H, d, K, N, style, dtype):
    print(f"case mlp {style} B{B} H{H} d{d} K{K} N{N} {dtype}", flush=True)
    c = mlp_case(P, 200 + d + K, B, H, N * K, d, K, dtype, style)
    dv = to_dev(c)
    got = P.ttt_mlp_forward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W1"], dv["b1"], dv["W2"], dv["b2"],
                                dv["token_eta"], dv["lr"], dv["gamma"], dv["beta"], K)
    torch.cuda.synchronize()
    n = np_inputs(c)
    ref = orc.mlp_forward(n["W1"], n["b1"], n["W2"], n["b2"], n["xq"], n["xk"], n["xv"], n["token_eta"],
                          n["lr"], n["gamma"], n["beta"], K=K)
    # bf16 I/O runs the register-resident kernels (one CU for d <= 96, a pair of CUs for d = 128),
    # whose products take bf16 operands (f32 accumulation and state): everything is held to the bf16
    # bar.  f32 I/O computes in f32 throughout.
    f32_products = dtype == torch.float32
    # With bf16 products the biases, which start at zero in the baseline style and are pure sums of
    # rounded update rows, carry a tail just above the elementwise floor (0.2 % of the largest entry):
    # for them the share of elements inside the elementwise bound is asked to be 99 %, not 99.9 %.
    for name, g, r in zip(("out", "W1", "b1", "W2", "b2"), got, ref):
        loose = not f32_products and name in ("b1", "b2")
        assert_close(g, r, 1e-4 if (f32_products and name != "out") else TOL[dtype], name,
                     min_frac=0.99 if loose else 0.999)


@pytest.mark.parametrize("B,H,K,N", [(2, 2, 16, 4), (1, 1, 7, 2), (1, 3, 16, 9)])
def test_mlp_fwd_d96_one_cu_and_two_cu_kernels(P, B, H, K, N):
    """head_dim 96, bf16 I/O: the one-CU register-resident kernel (default) and, with TTT_HINT_TWO_CU, the kernel
    that spreads a unit over a pair of CUs as head_dim 128 always does.  Both against the oracle, and close to each
    other."""
    print(f"case mlp d96 one/two CU B{B} H{H} K{K} N{N}", flush=True)
    d = 96
    c = mlp_case(P, 410 + K + N, B, H, N * K, d, K, torch.bfloat16, "ref")
    dv = to_dev(c)
    args = (dv["xq"], dv["xk"], dv["xv"], dv["W1"], dv["b1"], dv["W2"], dv["b2"], dv["token_eta"], dv["lr"], dv["gamma"],
            dv["beta"], K)
    two = P.ttt_mlp_forward_raw(*args, kernel_hint=P.TTT_HINT_TWO_CU)
    two_again = P.ttt_mlp_forward_raw(*args, kernel_hint=P.TTT_HINT_TWO_CU)
    one = P.ttt_mlp_forward_raw(*args)
    torch.cuda.synchronize()
    n = np_inputs(c)
    ref = orc.mlp_forward(n["W1"], n["b1"], n["W2"], n["b2"], n["xq"], n["xk"], n["xv"], n["token_eta"],
                          n["lr"], n["gamma"], n["beta"], K=K)
    for name, g2, g1, ga, r in zip(("out", "W1", "b1", "W2", "b2"), two, one, two_again, ref):
        assert torch.equal(g2, ga), f"{name}: the two-CU kernel is not deterministic"
        assert_close(g2, r, TOL[torch.bfloat16], "two-CU " + name, min_frac=0.99 if name in ("b1", "b2") else 0.999)
        assert_close(g1, r, TOL[torch.bfloat16], "one-CU " + name, min_frac=0.99 if name in ("b1", "b2") else 0.999)
    # different kernels (the order in which the halves of the hidden axis are summed differs): not the same bits
    assert (two[0].float() - one[0].float()).abs().max().item() <= 2.0 ** -5


def test_mlp_fwd_bf16_lds_kernel_keeps_f32_products(P):
    """kernel_hint TTT_HINT_LDS_TILES selects the LDS-tile kernel for bf16 I/O too: f32 products, so the
    state meets the f32 bar."""
    print("case mlp bf16 lds kernel", flush=True)
    B, H, d, K, N = 2, 2, 96, 16, 4
    c = mlp_case(P, 77, B, H, N * K, d, K, torch.bfloat16, "ref")
    dv = to_dev(c)
    got = P.ttt_mlp_forward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W1"], dv["b1"], dv["W2"], dv["b2"],
                                dv["token_eta"], dv["lr"], dv["gamma"], dv["beta"], K,
                                kernel_hint=P.TTT_HINT_LDS_TILES)
    torch.cuda.synchronize()
    n = np_inputs(c)
    ref = orc.mlp_forward(n["W1"], n["b1"], n["W2"], n["b2"], n["xq"], n["xk"], n["xv"], n["token_eta"],
                          n["lr"], n["gamma"], n["beta"], K=K)
    for name, g, r in zip(("out", "W1", "b1", "W2", "b2"), got, ref):
        assert_close(g, r, TOL[torch.bfloat16] if name == "out" else 1e-4, name)


def test_mlp_inner_model_with_remainder(P):
    print("case mlp remainder", flush=True)
    B, H, d, K, seq = 2, 2, 64, 16, 37
    c = mlp_case(P, 31, B, H, seq, d, K, torch.float32, "ref")
    te_seq = c["token_eta"].repeat(seq // K + 1)[:seq]
    dv = to_dev(c)
    model = P.FusedMlp(P.ModelConfig(H, d, P.TTTConfig(mini_batch_size=K)), dv["W1"], dv["b1"], dv["W2"],
                       dv["b2"], dv["gamma"], dv["beta"])
    state = model.init_state(B)
    out = model.forward(state, P.TTTInputsInner(P.Qkv(dv["xq"], dv["xk"], dv["xv"]), te_seq.to("cuda:0"),
                                                dv["lr"]))
    torch.cuda.synchronize()
    n = np_inputs(c)
    ref = orc.mlp_forward(n["W1"], n["b1"], n["W2"], n["b2"], n["xq"], n["xk"], n["xv"],
                          te_seq.double().numpy(), n["lr"], n["gamma"], n["beta"], K=K)
    for name, g, r in zip(("out", "W1", "b1", "W2", "b2"), (out, state.w1, state.b1, state.w2, state.b2), ref):
        assert_close(g, r, 1e-4, name)


@pytest.mark.parametrize("kernel", ["registers", "lds"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("B,H,d,K,N,ci", [(2, 2, 96, 16, 4, 1), (1, 3, 128, 16, 5, 2), (1, 2, 128, 6, 3, 1)])
def test_linear_fwd_wide_heads(P, B, H, d, K, N, ci, dtype, kernel):
    """head_dim 96 / 128: the register-resident kernel (default; bf16 I/O multiplies bf16 operands) and the
    LDS-tile kernel (kernel_hint TTT_HINT_LDS_TILES; f32 arithmetic for both I/O dtypes)."""
    print(f"case linear wide B{B} H{H} d{d} K{K} N{N} ci{ci} {dtype} {kernel}", flush=True)
    c = P.synthetic.reference_test_inputs(300 + d, B, H, N * K, d, K, io_dtype=dtype)
    dv = to_dev(c)
    out, W, b, Wc, bc = P.ttt_linear_forward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W0"], dv["b0"],
                                                 dv["token_eta"], dv["lr"], dv["gamma"], dv["beta"], K,
                                                 1e-6, ci, want_checkpoints=True,
                                                 kernel_hint=P.TTT_HINT_LDS_TILES if kernel == "lds" else 0)
    torch.cuda.synchronize()
    n = np_inputs(c)
    ro, rW, rb, rWc, rbc = orc.linear_forward(n["W0"], n["b0"], n["xq"], n["xk"], n["xv"], n["token_eta"],
                                              n["lr"], n["gamma"], n["beta"], K=K, checkpoint_interval=ci)
    assert_close(out, ro, TOL[dtype], "out")
    state_tol = 1e-4 if (dtype == torch.float32 or kernel == "lds") else TOL[dtype]
    for name, g, r in (("W", W, rW), ("b", b, rb), ("W_ckpt", Wc, rWc), ("b_ckpt", bc, rbc)):
        assert_close(g, r, state_tol, name)


def test_mlp_fwd_d128_lost_partner_is_loud(P):
    """head_dim 128, bf16 I/O: two workgroups share a unit and wait for each other.  With the waits made to give up
    at once (TTT_HINT_TEST_LOST_PARTNER; every kernel still runs to its end) the call still returns TTT_OK -- it
    cannot know -- and every output of every unit is NaN, so the failure cannot pass for a result.  More units than
    one launch holds (256 CUs: 128 units per launch) also exercises the batched launches."""
    print("case mlp d128 lost partner", flush=True)
    B, H, d, K, N = 1, 3, 128, 16, 3
    c = mlp_case(P, 91, B, H, N * K, d, K, torch.bfloat16, "ref")
    dv = to_dev(c)
    args = (dv["xq"], dv["xk"], dv["xv"], dv["W1"], dv["b1"], dv["W2"], dv["b2"], dv["token_eta"], dv["lr"], dv["gamma"],
            dv["beta"], K)
    import ctypes
    def lost_workgroups():
        n = ctypes.c_int64(-1)
        P.check(P.lib().ttt_mlp_fwd_lost_workgroups(ctypes.byref(n)))
        return n.value
    torch.cuda.synchronize()
    before = lost_workgroups()
    got = P.ttt_mlp_forward_raw(*args, kernel_hint=P.TTT_HINT_TEST_LOST_PARTNER)
    torch.cuda.synchronize()
    for name, t in zip(("out", "W1", "b1", "W2", "b2"), got):
        assert torch.isnan(t.float()).all(), f"{name}: a lost partner left finite values"
    # the device's status word counts the workgroups that gave up: both of every pair here
    assert lost_workgroups() == before + 2 * B * H
    # and the same call without the hook is healthy afterwards (nothing sticky in the library)
    ok = P.ttt_mlp_forward_raw(*args)
    torch.cuda.synchronize()
    for t in ok:
        assert torch.isfinite(t.float()).all()
    assert lost_workgroups() == before + 2 * B * H


@pytest.mark.parametrize("d", [96, 128])
def test_mlp_fwd_two_cu_pair_on_two_xcds_takes_device_scope_stores(P, d):
    """The two workgroups of a pair tell each other at start which XCD they run on; a pair on two XCDs exchanges through
    device-scope stores instead of words that stay in one XCD's L2.  TTT_HINT_TEST_OTHER_XCD makes every pair take that
    path: same kernel, same order of operations, so the same bits as the default path, and nothing lost."""
    print(f"case mlp two-CU other-XCD path d{d}", flush=True)
    B, H, K, N = 1, 3, 16, 5
    dv = to_dev(mlp_case(P, 95 + d, B, H, N * K, d, K, torch.bfloat16, "ref"))
    args = (dv["xq"], dv["xk"], dv["xv"], dv["W1"], dv["b1"], dv["W2"], dv["b2"], dv["token_eta"], dv["lr"], dv["gamma"],
            dv["beta"], K)
    torch.cuda.synchronize()
    before = P.mlp_fwd_lost_workgroups()
    ref = P.ttt_mlp_forward_raw(*args, kernel_hint=P.TTT_HINT_TWO_CU)
    got = P.ttt_mlp_forward_raw(*args, kernel_hint=P.TTT_HINT_TWO_CU | P.TTT_HINT_TEST_OTHER_XCD)
    torch.cuda.synchronize()
    for name, x, y in zip(("out", "W1", "b1", "W2", "b2"), got, ref):
        assert torch.isfinite(x.float()).all(), name
        assert torch.equal(x, y), f"{name}: device-scope exchange differs from the L2-resident one"
    assert P.mlp_fwd_lost_workgroups() == before


def test_mlp_fwd_d128_more_units_than_one_launch(P):
    """160 units of head_dim 128 need 320 workgroups: more than the CUs of the device, so the pairs go in two
    launches; every unit must come out as when it is computed alone."""
    print("case mlp d128 batched launches", flush=True)
    B, H, d, K, N = 20, 8, 128, 16, 2
    c = mlp_case(P, 92, B, H, N * K, d, K, torch.bfloat16, "ref")
    dv = to_dev(c)
    call = lambda x: P.ttt_mlp_forward_raw(x["xq"], x["xk"], x["xv"], x["W1"], x["b1"], x["W2"], x["b2"], x["token_eta"],
                                           x["lr"], x["gamma"], x["beta"], K)
    full = call(dv)
    torch.cuda.synchronize()
    for b in (0, 15, 16, 19):  # units on both sides of the launch boundary (128 units = 16 batch entries)
        one = {k: (v[b:b + 1].contiguous() if k in ("xq", "xk", "xv", "lr") else v) for k, v in dv.items()}
        r = call(one)
        torch.cuda.synchronize()
        for name, f, o in zip(("out", "W1", "b1", "W2", "b2"), full, r):
            assert torch.equal(f[b:b + 1], o), (b, name)
