"""GPU test of the C++ host classes (ttt-rs_amd/host/fused_tile_multi.hpp, fused_mlp.hpp): a small compiled
driver (host/host_driver.cpp -> lib/libttt_host_driver.so, built by ttt-rs_amd/build.py) constructs the classes
the way a C++ caller would and runs forward (full mini-batches + remainder) and backward on device buffers owned
by this process.  Both the C++ classes and the Python mirror are thin layers over the same C ABI, so their
results must agree bit for bit (outputs accumulated with floating-point atomics: to 1e-5); the Python mirror
itself is held to the oracle by the other GPU tests."""
import ctypes as C
import importlib
import os

import pytest
import torch

from helpers import assert_close, to_dev
from test_mlp_fwd_gpu import mlp_case

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def P():
    return importlib.import_module("ttt-rs_amd")


@pytest.fixture(scope="module")
def drv(P):
    path = os.path.join(os.path.dirname(P.LIB_PATH), "libttt_host_driver.so")
    assert os.path.exists(path), f"{path} is missing: run python ttt-rs_amd/build.py"
    P.lib()  # the driver links against the library; load it first from its in-tree path
    L = C.CDLL(path)
    L.ttt_host_last_error.restype = C.c_char_p
    return L


def ptr(t):
    return C.c_void_p(None if t is None else t.data_ptr())


def dt(P, t):
    return P.TTT_BF16 if t.dtype == torch.bfloat16 else P.TTT_F32


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_cpp_linear_forward_with_remainder_equals_python_mirror(P, drv, dtype):
    B, H, d, K, seq = 2, 2, 64, 16, 16 * 3 + 5
    print(f"case host C++ linear forward+remainder {dtype}", flush=True)
    c = to_dev(P.synthetic.reference_test_inputs(13, B, H, seq, d, K, io_dtype=dtype))
    te_seq = c["token_eta"].repeat(seq // K + 1)[:seq].contiguous()
    model = P.FusedTileMulti(P.ModelConfig(H, d, P.TTTConfig(mini_batch_size=K)), c["W0"], c["b0"], c["gamma"], c["beta"])
    state = model.init_state(B)
    ref = model.forward(state, P.TTTInputsInner(P.Qkv(c["xq"], c["xk"], c["xv"]), te_seq, c["lr"]))
    out = torch.full_like(c["xq"], float("nan"))
    st = [torch.full((B, H, d, d), float("nan"), device="cuda:0"), torch.full((B, H, d), float("nan"), device="cuda:0"),
          torch.full((B, H, d, d), float("nan"), device="cuda:0"), torch.full((B, H, d), float("nan"), device="cuda:0")]
    cur = C.c_int(-1)
    rc = drv.ttt_host_linear_forward(B, H, d, K, seq, dt(P, c["xq"]), C.c_float(1e-6), 1, 0, ptr(c["W0"]), ptr(c["b0"]),
                                     ptr(c["gamma"]), ptr(c["beta"]), ptr(c["xq"]), ptr(c["xk"]), ptr(c["xv"]),
                                     ptr(te_seq), ptr(c["lr"]), ptr(out), *[ptr(t) for t in st], None, None,
                                     C.byref(cur), C.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert rc == P.TTT_OK, drv.ttt_host_last_error()
    # two launches (full mini-batches, remainder): the final state is back in the first pair
    assert cur.value == 0
    assert torch.equal(out, ref)
    assert torch.equal(st[0], state.weight) and torch.equal(st[1], state.bias)


@pytest.mark.parametrize("dtype,packed", [(torch.float32, 0), (torch.bfloat16, 1), (torch.bfloat16, 2)],
                         ids=["f32", "bf16-packed", "bf16-factors"])
def test_cpp_linear_forward_backward_equals_python_mirror(P, drv, dtype, packed):
    B, H, d, K, N = 2, 3, 64, 16, 4
    seq = N * K
    print(f"case host C++ linear forward+backward {dtype} packed={packed}", flush=True)
    c = to_dev(P.synthetic.reference_test_inputs(17, B, H, seq, d, K, io_dtype=dtype))
    g = torch.Generator().manual_seed(3)
    dO = torch.randn(B, H, seq, d, generator=g).to(dtype).to("cuda:0")
    out_r, W_r, b_r, Wc_r, bc_r = P.ttt_linear_forward_raw(c["xq"], c["xk"], c["xv"], c["W0"], c["b0"], c["token_eta"],
                                                         c["lr"], c["gamma"], c["beta"], K, 1e-6, 1,
                                                         want_checkpoints=True, packed_checkpoints=packed)
    ref = P.ttt_linear_backward_raw(c["xq"], c["xk"], c["xv"], c["W0"], c["b0"], c["token_eta"], c["lr"], c["gamma"],
                                    c["beta"], Wc_r, bc_r, dO, K, 1e-6, 1, packed_checkpoints=packed)
    f32 = dict(dtype=torch.float32, device="cuda:0")
    out = torch.empty_like(c["xq"])
    st = [torch.empty((B, H, d, d), **f32), torch.empty((B, H, d), **f32), torch.empty((B, H, d, d), **f32),
          torch.empty((B, H, d), **f32)]
    Wc, bc = torch.empty((B, H, N, d, d), **f32), torch.empty((B, H, N, d), **f32)
    cur = C.c_int(-1)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    common = (B, H, d, K, seq, dt(P, c["xq"]), C.c_float(1e-6), 1, packed, ptr(c["W0"]), ptr(c["b0"]), ptr(c["gamma"]),
              ptr(c["beta"]), ptr(c["xq"]), ptr(c["xk"]), ptr(c["xv"]), ptr(c["token_eta"]), ptr(c["lr"]))
    rc = drv.ttt_host_linear_forward(*common, ptr(out), *[ptr(t) for t in st], ptr(Wc), ptr(bc), C.byref(cur), stream)
    assert rc == P.TTT_OK, drv.ttt_host_last_error()
    got = {k: torch.empty_like(v) for k, v in ref.items()}
    # the class takes the same path as the mirror: a workspace where the library can use one (f32 I/O: two workgroups
    # per unit), so the results can be held to each other bit for bit
    ws = torch.empty((64 << 20,), dtype=torch.uint8, device="cuda:0")
    rc = drv.ttt_host_linear_backward(*common, ptr(Wc), ptr(bc), ptr(dO), ptr(got["grad_xq"]), ptr(got["grad_xk"]),
                                      ptr(got["grad_xv"]), ptr(got["grad_weight"]), ptr(got["grad_bias"]),
                                      ptr(got["grad_ttt_lr_eta"]), ptr(got["grad_token_eta"]), ptr(got["grad_ln_weight"]),
                                      ptr(got["grad_ln_bias"]), stream, ptr(ws), C.c_longlong(ws.numel()))
    torch.cuda.synchronize()
    assert rc == P.TTT_OK, drv.ttt_host_last_error()
    assert cur.value == 1  # one launch: the final state is in the second pair
    assert torch.equal(out, out_r) and torch.equal(st[2], W_r) and torch.equal(st[3], b_r)
    # (update factors: only the first slot of the bias buffer is written, with the final bias)
    assert torch.equal(bc[:, :, 0], bc_r[:, :, 0]) if packed == 2 else torch.equal(bc, bc_r)
    for k in ("grad_xq", "grad_xk", "grad_xv", "grad_weight", "grad_bias", "grad_ttt_lr_eta"):
        assert torch.equal(got[k], ref[k]), k
    for k in ("grad_token_eta", "grad_ln_weight", "grad_ln_bias"):  # atomically accumulated
        assert_close(got[k], ref[k].double().cpu().numpy(), 1e-5, k)


def test_cpp_mlp_forward_remainder_and_backward_equal_python_mirror(P, drv):
    B, H, d, K = 1, 2, 64, 16
    f32 = dict(dtype=torch.float32, device="cuda:0")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def states():
        m = 4 * d
        mk = lambda: [torch.empty((B, H, d, m), **f32), torch.empty((B, H, m), **f32), torch.empty((B, H, m, d), **f32),
                      torch.empty((B, H, d), **f32)]
        a, b = mk(), mk()
        arr = lambda ts: (C.c_void_p * 4)(*[t.data_ptr() for t in ts])
        return a, b, arr(a), arr(b)

    # forward with a remainder (bf16 I/O: the register-resident kernel)
    seq = 2 * K + 7
    print("case host C++ mlp forward+remainder bf16", flush=True)
    c = to_dev(mlp_case(P, 31, B, H, seq, d, K, torch.bfloat16, "ref"))
    te_seq = c["token_eta"].repeat(seq // K + 1)[:seq].contiguous()
    model = P.FusedMlp(P.ModelConfig(H, d, P.TTTConfig(mini_batch_size=K)), c["W1"], c["b1"], c["W2"], c["b2"],
                       c["gamma"], c["beta"])
    state = model.init_state(B)
    ref = model.forward(state, P.TTTInputsInner(P.Qkv(c["xq"], c["xk"], c["xv"]), te_seq, c["lr"]))
    out = torch.empty_like(c["xq"])
    sa, sb, pa, pb = states()
    cur = C.c_int(-1)
    rc = drv.ttt_host_mlp_forward_backward(B, H, d, K, seq, P.TTT_BF16, C.c_float(1e-6), ptr(c["W1"]), ptr(c["b1"]),
                                           ptr(c["W2"]), ptr(c["b2"]), ptr(c["gamma"]), ptr(c["beta"]), ptr(c["xq"]),
                                           ptr(c["xk"]), ptr(c["xv"]), ptr(te_seq), ptr(c["lr"]), ptr(out), pa, pb,
                                           C.byref(cur), *([None] * 12), None, stream)
    torch.cuda.synchronize()
    assert rc == P.TTT_OK, drv.ttt_host_last_error()
    assert cur.value == 0
    assert torch.equal(out, ref)
    for t, r in zip(sa, (state.w1, state.b1, state.w2, state.b2)):
        assert torch.equal(t, r)

    # forward + backward over whole mini-batches, f32 I/O
    seq = 3 * K
    print("case host C++ mlp forward+backward f32", flush=True)
    c = to_dev(mlp_case(P, 32, B, H, seq, d, K, torch.float32, "ref"))
    g = torch.Generator().manual_seed(4)
    dO = torch.randn(B, H, seq, d, generator=g).to("cuda:0")
    ref = P.ttt_mlp_backward_raw(c["xq"], c["xk"], c["xv"], c["W1"], c["b1"], c["W2"], c["b2"], c["token_eta"], c["lr"],
                                 c["gamma"], c["beta"], dO, K)
    out_r = P.ttt_mlp_forward_raw(c["xq"], c["xk"], c["xv"], c["W1"], c["b1"], c["W2"], c["b2"], c["token_eta"], c["lr"],
                                  c["gamma"], c["beta"], K)[0]
    got = {k: torch.empty_like(v) for k, v in ref.items()}
    desc = P.TttDesc(B, H, seq, d, K, 1e-6, 1, P.TTT_F32, 0, 0)
    ws = torch.empty(P.lib().ttt_mlp_bwd_workspace_bytes(C.byref(desc)) // 4, **f32)
    out = torch.empty_like(c["xq"])
    sa, sb, pa, pb = states()
    rc = drv.ttt_host_mlp_forward_backward(B, H, d, K, seq, P.TTT_F32, C.c_float(1e-6), ptr(c["W1"]), ptr(c["b1"]),
                                           ptr(c["W2"]), ptr(c["b2"]), ptr(c["gamma"]), ptr(c["beta"]), ptr(c["xq"]),
                                           ptr(c["xk"]), ptr(c["xv"]), ptr(c["token_eta"]), ptr(c["lr"]), ptr(out), pa, pb,
                                           C.byref(cur), ptr(dO), ptr(got["d_xq"]), ptr(got["d_xk"]), ptr(got["d_xv"]),
                                           ptr(got["d_W1"]), ptr(got["d_b1"]), ptr(got["d_W2"]), ptr(got["d_b2"]),
                                           ptr(got["d_lr"]), ptr(got["d_token_eta"]), ptr(got["d_gamma"]),
                                           ptr(got["d_beta"]), ptr(ws), stream)
    torch.cuda.synchronize()
    assert rc == P.TTT_OK, drv.ttt_host_last_error()
    assert cur.value == 1
    assert torch.equal(out, out_r)
    for k in ("d_xq", "d_xk", "d_xv", "d_W1", "d_b1", "d_W2", "d_b2", "d_lr"):
        assert torch.equal(got[k], ref[k]), k
    for k in ("d_token_eta", "d_gamma", "d_beta"):
        assert_close(got[k], ref[k].double().cpu().numpy(), 1e-5, k)


def test_cpp_lost_workgroup_guard(P, drv):
    """LostWorkgroupGuard around a TTT-MLP forward at head_dim 128 (two workgroups per unit): silent on a healthy
    run, an error when the waits are made to give up at once (TTT_HINT_TEST_LOST_PARTNER)."""
    print("case host C++ lost-workgroup guard", flush=True)
    B, H, d, K, N = 1, 2, 128, 16, 2
    dv = to_dev(mlp_case(P, 93, B, H, N * K, d, K, torch.bfloat16, "ref"))
    args = (dv["xq"], dv["xk"], dv["xv"], dv["W1"], dv["b1"], dv["W2"], dv["b2"], dv["token_eta"], dv["lr"], dv["gamma"],
            dv["beta"], K)
    drv.ttt_host_lost_guard_new.restype = C.c_void_p
    drv.ttt_host_lost_guard_verify_and_free.argtypes = [C.c_void_p]
    torch.cuda.synchronize()
    g = drv.ttt_host_lost_guard_new()
    assert g
    P.ttt_mlp_forward_raw(*args)
    torch.cuda.synchronize()
    assert drv.ttt_host_lost_guard_verify_and_free(g) == P.TTT_OK
    g = drv.ttt_host_lost_guard_new()
    P.ttt_mlp_forward_raw(*args, kernel_hint=P.TTT_HINT_TEST_LOST_PARTNER)
    torch.cuda.synchronize()
    assert drv.ttt_host_lost_guard_verify_and_free(g) == P.TTT_ERR_HIP
    assert b"partner" in drv.ttt_host_last_error()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_cpp_linear_adam_forward_with_remainder_equals_python_mirror(P, drv, dtype):
    """FusedLinearAdam of host/fused_others.hpp: full mini-batches in one launch, the remainder as one short mini-batch
    that continues from the moments and the step count, both as in-place windows of the sequence."""
    B, H, d, K, seq = 2, 2, 64, 16, 16 * 3 + 5
    print(f"case host C++ linear-adam forward+remainder {dtype}", flush=True)
    c = to_dev(P.synthetic.reference_test_inputs(23, B, H, seq, d, K, io_dtype=dtype))
    te_seq = c["token_eta"].repeat(seq // K + 1)[:seq].contiguous()
    hp = P.TTTLinearAdamConfig(beta1=0.8, beta2=0.95, epsilon=1e-7, lr=5e-3)
    model = P.FusedLinearAdam(P.ModelConfig(H, d, P.TTTConfig(mini_batch_size=K)), hp, c["W0"], c["b0"], c["gamma"],
                              c["beta"])
    state = model.init_state(B)
    ref = model.forward(state, P.TTTInputsInner(P.Qkv(c["xq"], c["xk"], c["xv"]), te_seq, c["lr"]))
    nan = lambda *s: torch.full(s, float("nan"), device="cuda:0")
    sets = [[nan(B, H, d, d), nan(B, H, d), nan(B, H, d, d), nan(B, H, d), nan(B, H, d, d), nan(B, H, d)] for _ in range(2)]
    arr = lambda ts: (C.c_void_p * len(ts))(*[t.data_ptr() for t in ts])
    out = torch.full_like(c["xq"], float("nan"))
    cur, step = C.c_int(-1), C.c_int(-1)
    rc = drv.ttt_host_linear_adam_forward(B, H, d, K, seq, dt(P, c["xq"]), C.c_float(1e-6), C.c_float(hp.beta1),
                                          C.c_float(hp.beta2), C.c_float(hp.epsilon), C.c_float(hp.lr), ptr(c["W0"]),
                                          ptr(c["b0"]), ptr(c["gamma"]), ptr(c["beta"]), ptr(c["xq"]), ptr(c["xk"]),
                                          ptr(c["xv"]), ptr(te_seq), ptr(c["lr"]), ptr(out), arr(sets[0]), arr(sets[1]),
                                          C.byref(cur), C.byref(step),
                                          C.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert rc == P.TTT_OK, drv.ttt_host_last_error()
    assert cur.value == 0 and step.value == state.step == 4   # two launches: back in the first set
    assert torch.equal(out, ref)
    got = sets[0]
    for g, r, name in zip(got, (state.weight, state.bias, state.weight_m, state.bias_m, state.weight_v, state.bias_v),
                          ("weight", "bias", "weight_m", "bias_m", "weight_v", "bias_v")):
        assert torch.equal(g, r), name


@pytest.mark.parametrize("n_hidden,d", [(2, 32), (4, 32), (2, 64)])
def test_cpp_mlpn_forward_with_remainder_equals_python_mirror(P, drv, n_hidden, d):
    """FusedMlpN of host/fused_others.hpp against the Python mirror, sequence with a remainder (the C++ class works on
    windows of the sequence in place, the Python mirror on copies of the slices)."""
    from test_mlpn_gpu import make_case
    B, H, K, seq = 2, 2, 16, 16 * 2 + 7
    print(f"case host C++ mlp{n_hidden} d{d} forward+remainder", flush=True)
    c, Ws, bs = make_case(P, 31 + n_hidden, B, H, seq, d, K, n_hidden, torch.bfloat16)
    c = to_dev(c)
    Ws, bs = [w.to("cuda:0") for w in Ws], [b.to("cuda:0") for b in bs]
    te_seq = c["token_eta"].repeat(seq // K + 1)[:seq].contiguous()
    model = P.FusedMlpN(P.ModelConfig(H, d, P.TTTConfig(mini_batch_size=K)), Ws, bs, c["gamma"], c["beta"])
    assert model.name() == f"TTTMLP{n_hidden}"
    state = model.init_state(B)
    ref = model.forward(state, P.TTTInputsInner(P.Qkv(c["xq"], c["xk"], c["xv"]), te_seq, c["lr"]))
    nan = lambda *s: torch.full(s, float("nan"), device="cuda:0")
    wa, wb = [nan(B, *w.shape) for w in Ws], [nan(B, *w.shape) for w in Ws]
    ba, bb = [nan(B, *b.shape) for b in bs], [nan(B, *b.shape) for b in bs]
    arr = lambda ts: (C.c_void_p * len(ts))(*[t.data_ptr() for t in ts])
    out = torch.full_like(c["xq"], float("nan"))
    cur = C.c_int(-1)
    rc = drv.ttt_host_mlpn_forward(B, H, d, K, seq, dt(P, c["xq"]), C.c_float(1e-6), n_hidden, arr(Ws), arr(bs),
                                   ptr(c["gamma"]), ptr(c["beta"]), ptr(c["xq"]), ptr(c["xk"]), ptr(c["xv"]), ptr(te_seq),
                                   ptr(c["lr"]), ptr(out), arr(wa), arr(ba), arr(wb), arr(bb), C.byref(cur),
                                   C.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert rc == P.TTT_OK, drv.ttt_host_last_error()
    assert cur.value == 0
    assert torch.equal(out, ref)
    for i in range(n_hidden + 1):
        assert torch.equal(wa[i], state.weights[i]), f"weight {i}"
        assert torch.equal(ba[i], state.biases[i]), f"bias {i}"
