"""GPU parity of ttt_mlpn_fwd (TTT-MLP with 2, 3 or 4 hidden layers: rust/core/src/mlp2.rs, mlp3.rs, mlp4.rs) through
the C ABI against the float64 oracle, which is pinned to primal per-token gradient descent in
tests/test_oracle_pins.py."""
import importlib

import pytest
import torch

from helpers import TOL, assert_close, np_inputs, to_dev
from oracle import ttt_oracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def P():
    return importlib.import_module("ttt-rs_amd")


def make_case(P, seed, B, H, seq, d, K, n_hidden, dtype):
    c = P.synthetic.reference_test_inputs(seed, B, H, seq, d, K, io_dtype=dtype)
    g = torch.Generator().manual_seed(seed + 1)
    m = 4 * d
    dims = [d] + [m] * n_hidden + [d]
    c.pop("W0"), c.pop("b0")
    Ws = [torch.randn(H, dims[i], dims[i + 1], generator=g) * 0.02 for i in range(n_hidden + 1)]
    bs = [torch.randn(H, dims[i + 1], generator=g) * 0.02 for i in range(n_hidden + 1)]
    return c, Ws, bs


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("n_hidden,B,H,d,K,N", [(2, 2, 2, 32, 16, 3), (3, 1, 2, 32, 8, 3), (4, 1, 2, 32, 16, 2),
                                                (2, 1, 2, 64, 16, 3), (2, 2, 1, 64, 5, 2), (2, 1, 1, 32, 16, 1)])
def test_mlpn_fwd_matches_oracle(P, n_hidden, B, H, d, K, N, dtype):
    print(f"case mlpn hidden{n_hidden} B{B} H{H} d{d} K{K} N{N} {dtype}", flush=True)
    c, Ws, bs = make_case(P, 1700 + n_hidden + d + K, B, H, N * K, d, K, n_hidden, dtype)
    dv = to_dev(c)
    dev = lambda ts: [t.to("cuda:0") for t in ts]
    out, Wo, bo = P.ttt_mlpn_forward_raw(dv["xq"], dv["xk"], dv["xv"], dev(Ws), dev(bs), dv["token_eta"], dv["lr"],
                                         dv["gamma"], dv["beta"], K)
    torch.cuda.synchronize()
    n = np_inputs(c)
    ro, rW, rb = orc.mlpn_forward([w.double().numpy() for w in Ws], [b.double().numpy() for b in bs], n["xq"], n["xk"],
                                  n["xv"], n["token_eta"], n["lr"], n["gamma"], n["beta"], K=K)
    # f32 products for both I/O types: the state is held to 1e-4, the output to the I/O type's bar
    assert_close(out, ro, TOL[dtype], "out")
    for i in range(n_hidden + 1):
        assert_close(Wo[i], rW[i], 1e-4, f"W[{i}]")
        assert_close(bo[i], rb[i], 1e-4, f"b[{i}]", min_frac=0.99)


def test_mlpn_fwd_chained_calls_repeat_calls_and_refusals(P):
    n_hidden, B, H, d, K, N = 2, 1, 2, 32, 16, 4
    c, Ws, bs = make_case(P, 1800, B, H, N * K, d, K, n_hidden, torch.float32)
    dv = to_dev(c)
    dev = lambda ts: [t.to("cuda:0") for t in ts]
    args = lambda sl: (dv["xq"][:, :, sl].contiguous(), dv["xk"][:, :, sl].contiguous(), dv["xv"][:, :, sl].contiguous())
    run = lambda sl, W, b: P.ttt_mlpn_forward_raw(*args(sl), W, b, dv["token_eta"], dv["lr"][:, :, sl].contiguous(),
                                                  dv["gamma"], dv["beta"], K)
    whole = [run(slice(None), dev(Ws), dev(bs)) for _ in range(3)]
    h = (N // 2) * K
    first = run(slice(0, h), dev(Ws), dev(bs))
    second = run(slice(h, N * K), first[1], first[2])
    torch.cuda.synchronize()
    for r in whole[1:]:   # nothing in the kernel depends on timing
        assert torch.equal(r[0], whole[0][0])
        for x, y in zip(r[1] + r[2], whole[0][1] + whole[0][2]):
            assert torch.equal(x, y)
    # the state carried from one call to the next is the state the single call carries (same arithmetic, same order)
    assert torch.equal(torch.cat([first[0], second[0]], 2), whole[0][0])
    for x, y in zip(second[1] + second[2], whole[0][1] + whole[0][2]):
        assert torch.equal(x, y)
    for bad_d, bad_n in ((64, 3), (96, 2), (32, 5), (32, 1)):
        cc, W2, b2 = make_case(P, 1801, 1, 1, 16, bad_d, 16, bad_n, torch.float32)
        dd = to_dev(cc)
        with pytest.raises(P.TttError) as e:
            P.ttt_mlpn_forward_raw(dd["xq"], dd["xk"], dd["xv"], dev(W2), dev(b2), dd["token_eta"], dd["lr"], dd["gamma"],
                                   dd["beta"], 16)
        assert e.value.code == P.TTT_ERR_UNSUPPORTED
