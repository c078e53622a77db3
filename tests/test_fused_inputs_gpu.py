"""GPU parity of ttt_linear_fwd_fused_inputs: the TTT-Linear forward that forms its operands from the projections
(head split, rotary embedding, lr gate, token_eta inside the kernel's tile loads) against

  * ttt_inner_inputs followed by ttt_linear_fwd on the same values (the two-pass path it replaces): the operands it
    stores must be the same bits, its outputs the same to rounding of a separately compiled kernel;
  * the float64 oracle: inner_loop_inputs (rust/layer/src/ttt.rs:147-268) followed by linear_forward
    (rust/core/src/linear.rs:91-149) on the operands rounded to the I/O type, as the kernel rounds them.
"""
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


def make_case(P, B, seq, H, d, K, mode, seed):
    g = torch.Generator().manual_seed(seed)
    dt = torch.bfloat16
    c = dict(xq=torch.randn(B, seq, H, d, generator=g).to(dt), xk=torch.randn(B, seq, H, d, generator=g).to(dt),
             xv=torch.randn(B, seq, H, d, generator=g).to(dt), lg=torch.randn(B, seq, H, generator=g).to(dt),
             bias=torch.randn(H, generator=g) * 0.5, tidx=1.0 / torch.arange(1, K + 1, dtype=torch.float32),
             ltidx=torch.randn(K, generator=g) * 0.1, W0=torch.randn(H, d, d, generator=g) * 0.02,
             b0=torch.randn(H, d, generator=g) * 0.02, gamma=1.0 + 0.1 * torch.randn(H, d, generator=g),
             beta=0.1 * torch.randn(H, d, generator=g))
    start = 21
    if mode == "none":
        c.update(rope=None, off=0, wrap=0, cs=(None, None))
    elif mode == "wrap":  # ttt.rs:186-189: (start_idx % mini_batch, Some(mini_batch))
        c.update(off=start % K, wrap=K, rope=P.rope_cos_sin(K, 0, None, d, "cuda:0"),
                 cs=orc.rope_cos_sin(seq, start % K, K, d))
    else:  # RopeGlobal: (start_idx, None)
        c.update(off=start, wrap=0, rope=P.rope_cos_sin(start + seq, 0, None, d, "cuda:0"),
                 cs=orc.rope_cos_sin(seq, start, None, d))
    return c


def run_both(P, c, K, **kw):
    dev = lambda t: t.to("cuda:0")
    args = [dev(c[k]) for k in ("xq", "xk", "xv", "lg", "bias")] + [0.8, dev(c["tidx"]), dev(c["ltidx"])]
    fused = P.ttt_linear_forward_fused_inputs_raw(*args, dev(c["W0"]), dev(c["b0"]), dev(c["gamma"]), dev(c["beta"]), K,
                                                  rope=c["rope"], pos_offset=c["off"], pos_wrap=c["wrap"],
                                                  save_inputs=True, **kw)
    ins = P.inner_loop_inputs_raw(*args, K, rope=c["rope"], pos_offset=c["off"], pos_wrap=c["wrap"])
    two = P.ttt_linear_forward_raw(ins.qkv.xq, ins.qkv.xk, ins.qkv.xv, dev(c["W0"]), dev(c["b0"]), ins.token_eta,
                                   ins.ttt_lr_eta, dev(c["gamma"]), dev(c["beta"]), K, 1e-6,
                                   kw.get("checkpoint_interval", 1), want_checkpoints=kw.get("want_checkpoints", False),
                                   packed_checkpoints=kw.get("packed_checkpoints", 0), kernel_hint=2)
    torch.cuda.synchronize()
    return fused, ins, two


@pytest.mark.parametrize("mode", ["wrap", "global", "none"])
@pytest.mark.parametrize("B,seq,H,d,K", [(2, 64, 3, 64, 16), (1, 80, 2, 64, 16), (2, 35, 2, 64, 7), (1, 16, 2, 64, 16),
                                         (2, 48, 3, 32, 16), (1, 40, 2, 32, 8), (1, 32, 1, 64, 16)])
def test_fused_inputs_forward_matches_two_pass_and_oracle(P, B, seq, H, d, K, mode):
    print(f"case fused inputs B{B} seq{seq} H{H} d{d} K{K} {mode}", flush=True)
    c = make_case(P, B, seq, H, d, K, mode, 1000 + seq + d + K)
    fused, ins, two = run_both(P, c, K)
    saved = fused[-1]
    # the operands the kernel used are what the separate pass writes, bit for bit
    assert torch.equal(saved.qkv.xq, ins.qkv.xq), "rotated xq"
    assert torch.equal(saved.qkv.xk, ins.qkv.xk), "rotated xk"
    assert torch.equal(saved.qkv.xv, ins.qkv.xv), "xv"
    assert torch.equal(saved.ttt_lr_eta, ins.ttt_lr_eta), "lr"
    assert torch.equal(saved.token_eta, ins.token_eta), "token_eta"
    # same arithmetic on the same operands in a kernel compiled separately: equal to the last bits
    assert_close(fused[0], two[0].double().cpu().numpy(), 2.0 ** -7, "out vs two-pass")
    assert_close(fused[1], two[1].double().cpu().numpy(), 1e-5, "W vs two-pass")
    assert_close(fused[2], two[2].double().cpu().numpy(), 1e-5, "b vs two-pass")
    # oracle: producers in float64, operands rounded to bf16 as both GPU paths round them, then the inner loop
    q, k, v, lr, te = orc.inner_loop_inputs(to_np(c["xq"]), to_np(c["xk"]), to_np(c["xv"]), to_np(c["lg"]),
                                            to_np(c["bias"]), 0.8, to_np(c["tidx"]), to_np(c["ltidx"]), K, *c["cs"])
    assert_close(saved.qkv.xq, q, TOL[torch.bfloat16], "xq vs oracle")
    assert_close(saved.qkv.xk, k, TOL[torch.bfloat16], "xk vs oracle")
    assert_close(saved.ttt_lr_eta, lr, TOL[torch.bfloat16], "lr vs oracle")
    rnd = lambda t: t.double().cpu().numpy()
    n_full = (seq // K) * K
    ref = orc.linear_forward(to_np(c["W0"]), to_np(c["b0"]), rnd(saved.qkv.xq)[:, :, :n_full], rnd(saved.qkv.xk)[:, :, :n_full],
                             rnd(saved.qkv.xv)[:, :, :n_full], te[:K], rnd(saved.ttt_lr_eta)[:, :, :n_full],
                             to_np(c["gamma"]), to_np(c["beta"]), K=K)
    if n_full == seq:
        assert_close(fused[0], ref[0], TOL[torch.bfloat16], "out vs oracle")
        assert_close(fused[1], ref[1], TOL[torch.bfloat16], "W vs oracle")
        assert_close(fused[2], ref[2], TOL[torch.bfloat16], "b vs oracle")


@pytest.mark.parametrize("fmt", [0, 1], ids=["f32-ckpt", "packed"])
def test_fused_inputs_checkpoints_feed_the_backward(P, fmt):
    """The checkpoints and saved operands of the fused forward are what ttt_linear_bwd needs: its gradients equal
    those computed from the two-pass forward's outputs."""
    B, seq, H, d, K = 2, 64, 2, 64, 16
    c = make_case(P, B, seq, H, d, K, "wrap", 77)
    fused, ins, two = run_both(P, c, K, want_checkpoints=True, packed_checkpoints=fmt)
    dev = lambda t: t.to("cuda:0")
    dO = torch.randn(B, H, seq, d, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16).to("cuda:0")
    grads = []
    for fw, x in ((fused, fused[-1]), (two, ins)):
        grads.append(P.ttt_linear_backward_raw(x.qkv.xq, x.qkv.xk, x.qkv.xv, dev(c["W0"]), dev(c["b0"]), x.token_eta,
                                               x.ttt_lr_eta, dev(c["gamma"]), dev(c["beta"]), fw[3], fw[4], dO, K, 1e-6, 1,
                                               packed_checkpoints=fmt))
    torch.cuda.synchronize()
    for k in grads[0]:
        assert_close(grads[0][k], grads[1][k].double().cpu().numpy(), 5e-3, k, min_frac=0.99)


def test_fused_inputs_repeat_calls_are_identical(P):
    B, seq, H, d, K = 2, 96, 3, 64, 16
    for mode in ("wrap", "global"):
        c = make_case(P, B, seq, H, d, K, mode, 5)
        runs = [run_both(P, c, K)[0] for _ in range(3)]
        for r in runs[1:]:
            for i in range(3):
                assert torch.equal(r[i], runs[0][i]), (mode, i)


def test_fused_inputs_refuses_what_it_has_no_kernel_for(P):
    c = make_case(P, 1, 32, 2, 64, 16, "wrap", 9)
    dev = lambda t: t.to("cuda:0")
    args = [dev(c[k]) for k in ("xq", "xk", "xv", "lg", "bias")] + [0.8, dev(c["tidx"]), dev(c["ltidx"])]
    with pytest.raises(P.TttError) as e:  # positions that neither repeat with the mini-batch nor run over the sequence
        P.ttt_linear_forward_fused_inputs_raw(*args, dev(c["W0"]), dev(c["b0"]), dev(c["gamma"]), dev(c["beta"]), 16,
                                              rope=P.rope_cos_sin(64, 0, None, 64, "cuda:0"), pos_offset=0, pos_wrap=5)
    assert e.value.code == P.TTT_ERR_UNSUPPORTED
    f32 = [a.float() if torch.is_tensor(a) and a.dtype == torch.bfloat16 else a for a in args]
    with pytest.raises(P.TttError) as e:
        P.ttt_linear_forward_fused_inputs_raw(*f32, dev(c["W0"]), dev(c["b0"]), dev(c["gamma"]), dev(c["beta"]), 16)
    assert e.value.code == P.TTT_ERR_UNSUPPORTED
