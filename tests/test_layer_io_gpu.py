"""GPU parity of the two elementwise passes either side of the inner loop (ttt_inner_inputs,
ttt_layer_epilogue) through the C ABI against the float64 oracle."""
import importlib

import numpy as np
import pytest
import torch

from helpers import TOL, assert_close, to_np
from oracle import ttt_oracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def P():
    return importlib.import_module("ttt-rs_amd")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("B,seq,H,d,K,mode", [(2, 37, 3, 64, 16, "wrap"), (1, 50, 4, 32, 8, "global"),
                                              (2, 16, 2, 96, 16, "none"), (1, 33, 2, 128, 16, "wrap")])
def test_inner_inputs_match_oracle(P, B, seq, H, d, K, mode, dtype):
    print(f"case inner inputs B{B} seq{seq} H{H} d{d} K{K} {mode} {dtype}", flush=True)
    g = torch.Generator().manual_seed(seq + d)
    xq, xk, xv = (torch.randn(B, seq, H, d, generator=g).to(dtype) for _ in range(3))
    lg = torch.randn(B, seq, H, generator=g).to(dtype)
    bias = torch.randn(H, generator=g) * 0.5
    tidx = 1.0 / torch.arange(1, K + 1, dtype=torch.float32)
    ltidx = torch.randn(K, generator=g) * 0.3 - 0.2   # some sums negative: the clamp matters
    start = 21
    if mode == "none":
        rope, off, wrap, cs = None, 0, 0, (None, None)
    elif mode == "wrap":   # ttt.rs:186-189: (start_idx % mini_batch, Some(mini_batch))
        off, wrap = start % K, K
        rope = P.rope_cos_sin(K, 0, None, d, "cuda:0")
        cs = orc.rope_cos_sin(seq, off, wrap, d)
    else:                  # RopeGlobal: (start_idx, None)
        off, wrap = start, 0
        rope = P.rope_cos_sin(start + seq, 0, None, d, "cuda:0")
        cs = orc.rope_cos_sin(seq, off, None, d)
    dev = lambda t: t.to("cuda:0")
    got = P.inner_loop_inputs_raw(dev(xq), dev(xk), dev(xv), dev(lg), dev(bias), 0.8, dev(tidx), dev(ltidx), K,
                                  rope=rope, pos_offset=off, pos_wrap=wrap)
    torch.cuda.synchronize()
    q, k, v, lr, te = orc.inner_loop_inputs(to_np(xq), to_np(xk), to_np(xv), to_np(lg), to_np(bias), 0.8,
                                            to_np(tidx), to_np(ltidx), K, cs[0], cs[1])
    tol = TOL[dtype]
    assert_close(got.qkv.xq, q, tol, "xq")
    assert_close(got.qkv.xk, k, tol, "xk")
    assert np.array_equal(to_np(got.qkv.xv), v), "xv is a pure head split"
    assert_close(got.ttt_lr_eta, lr, tol, "lr")
    assert_close(got.token_eta, te, 1e-6, "token_eta")
    if mode == "none":
        assert np.array_equal(to_np(got.qkv.xq), q), "without RoPE xq is a pure head split"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("B,H,seq,d,gated", [(2, 12, 33, 64, True), (1, 4, 7, 32, False), (1, 16, 5, 128, True),
                                             (2, 3, 9, 96, True)])
def test_layer_epilogue_matches_oracle(P, B, H, seq, d, gated, dtype):
    print(f"case epilogue B{B} H{H} seq{seq} d{d} gated={gated} {dtype}", flush=True)
    g = torch.Generator().manual_seed(H * d + seq)
    x = (torch.randn(B, H, seq, d, generator=g) * 2 + 0.3).to(dtype)
    gam = 1.0 + 0.2 * torch.randn(H * d, generator=g)
    bet = 0.1 * torch.randn(H * d, generator=g)
    gate = torch.randn(B, seq, H * d, generator=g).to(dtype) if gated else None
    out = P.layer_epilogue_raw(x.to("cuda:0"), gam.to("cuda:0"), bet.to("cuda:0"),
                               None if gate is None else gate.to("cuda:0"))
    torch.cuda.synchronize()
    ref = orc.layer_epilogue(to_np(x), to_np(gam), to_np(bet), None if gate is None else to_np(gate))
    assert_close(out, ref, TOL[dtype], "out")


def test_layer_io_rejects_bad_arguments(P):
    x = torch.zeros(1, 2, 4, 20, device="cuda:0")   # head_dim not a multiple of 8
    with pytest.raises(P.TttError) as e:
        P.layer_epilogue_raw(x, torch.ones(40, device="cuda:0"), torch.zeros(40, device="cuda:0"))
    assert e.value.code == P.TTT_ERR_UNSUPPORTED
    x = torch.zeros(1, 40, 4, 64, device="cuda:0")  # hidden 2560 > 2048
    with pytest.raises(P.TttError) as e:
        P.layer_epilogue_raw(x, torch.ones(2560, device="cuda:0"), torch.zeros(2560, device="cuda:0"))
    assert e.value.code == P.TTT_ERR_UNSUPPORTED
