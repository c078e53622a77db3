"""GPU parity of ttt_linear_adam_fwd (TTT-Linear with the Adam inner optimiser, rust/core/src/linear_adam.rs) through
the C ABI against the float64 oracle, which is pinned to torch.optim.Adam in tests/test_oracle_pins.py."""
import importlib

import numpy as np
import pytest
import torch

from helpers import TOL, assert_close, np_inputs, to_dev
from oracle import ttt_oracle as orc

pytestmark = pytest.mark.gpu

HP = dict(beta1=0.9, beta2=0.999, adam_eps=1e-8, adam_lr=1e-3)   # the reference's defaults (linear_adam.rs:49-61)


@pytest.fixture(scope="module")
def P():
    return importlib.import_module("ttt-rs_amd")


def run(P, dv, K, moments=None, step=0, sl=slice(None), W=None, b=None, **hp):
    return P.ttt_linear_adam_forward_raw(dv["xq"][:, :, sl].contiguous(), dv["xk"][:, :, sl].contiguous(),
                                         dv["xv"][:, :, sl].contiguous(), dv["W0"] if W is None else W,
                                         dv["b0"] if b is None else b, dv["token_eta"], dv["lr"][:, :, sl].contiguous(),
                                         dv["gamma"], dv["beta"], K, moments=moments, step=step, **hp)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("hp", [HP, dict(beta1=0.5, beta2=0.9, adam_eps=1e-6, adam_lr=2e-2)], ids=["defaults", "fast"])
@pytest.mark.parametrize("B,H,d,K,N", [(2, 2, 32, 8, 3), (1, 2, 64, 16, 4), (2, 3, 64, 16, 9), (1, 2, 64, 5, 3),
                                       (1, 1, 32, 16, 1)])
def test_linear_adam_fwd_matches_oracle(P, B, H, d, K, N, hp, dtype):
    print(f"case linear adam B{B} H{H} d{d} K{K} N{N} {dtype} {hp}", flush=True)
    c = P.synthetic.reference_test_inputs(1300 + d + K + N, B, H, N * K, d, K, io_dtype=dtype)
    dv = to_dev(c)
    out, W, b, mo, step = run(P, dv, K, **hp)
    torch.cuda.synchronize()
    n = np_inputs(c)
    ro, st = orc.linear_adam_forward(n["W0"], n["b0"], n["xq"], n["xk"], n["xv"], n["token_eta"], n["lr"], n["gamma"],
                                     n["beta"], K=K, **hp)
    assert step == st["step"] == N
    tol = TOL[dtype]
    # bf16: a sign flip of a near-zero gradient element (see below) moves a state element by up to adam_lr, which the
    # next mini-batches' outputs see: 99 % of the elements inside the elementwise band, all inside the max-norm bar
    assert_close(out, ro, tol, "out", min_frac=0.999 if dtype == torch.float32 else 0.99)
    # the state moves by at most adam_lr per element and step: compare the movement, not the state, so that an
    # optimiser that did nothing cannot pass
    W0 = np.broadcast_to(n["W0"][None], st["W"].shape)
    b0 = np.broadcast_to(n["b0"][None], st["b"].shape)
    f32 = dtype == torch.float32
    dW, db = W.double().cpu().numpy() - W0, b.double().cpu().numpy() - b0
    if f32:
        assert_close(dW, st["W"] - W0, 1e-3, "W movement", min_frac=0.99)
        assert_close(db, st["b"] - b0, 1e-3, "b movement", min_frac=0.9)
    else:
        # Adam normalises the step: an element whose gradient is near zero moves by up to adam_lr in a direction that
        # the bf16 rounding of the operands can flip, so single elements may differ by the whole step.  The moments
        # below compare the gradients themselves; here: nearly all elements agree, none moves further than Adam can
        for got, ref, name in ((dW, st["W"] - W0, "W"), (db, st["b"] - b0, "b")):
            ok = np.abs(got - ref) <= 0.05 * np.abs(ref).max()
            assert ok.mean() >= 0.95, f"{name} movement: only {ok.mean():.4f} of the elements within 5 % of the largest"
            assert np.abs(got).max() <= 1.05 * hp["adam_lr"] * N / (1.0 - hp["beta1"]), f"{name} moved further than Adam can"
    for got, name in zip(mo, ("Wm", "bm", "Wv", "bv")):
        assert_close(got, st[name], 1e-4 if f32 else tol, name, min_frac=0.999 if f32 else 0.99)


def test_linear_adam_continues_from_saved_moments(P):
    """Two calls over the halves of a sequence, the second starting from the state, moments and step count the first
    left, equal one call over the whole (to f32 rounding: the state is re-centred at the start of a call)."""
    B, H, d, K, N = 2, 2, 64, 16, 6
    c = P.synthetic.reference_test_inputs(1400, B, H, N * K, d, K, io_dtype=torch.float32)
    dv = to_dev(c)
    whole = run(P, dv, K, **HP)
    h = (N // 2) * K
    first = run(P, dv, K, sl=slice(0, h), **HP)
    second = run(P, dv, K, moments=first[3], step=first[4], sl=slice(h, N * K), W=first[1], b=first[2], **HP)
    torch.cuda.synchronize()
    assert second[4] == whole[4] == N
    assert_close(torch.cat([first[0], second[0]], 2), whole[0].double().cpu().numpy(), 1e-5, "out")
    assert_close(second[1], whole[1].double().cpu().numpy(), 1e-6, "W")
    for a_, b_, name in zip(second[3], whole[3], ("Wm", "bm", "Wv", "bv")):
        assert_close(a_, b_.double().cpu().numpy(), 1e-5, name)


def test_linear_adam_repeat_calls_are_identical_and_bad_arguments_are_refused(P):
    B, H, d, K, N = 1, 2, 64, 16, 5
    c = P.synthetic.reference_test_inputs(1500, B, H, N * K, d, K, io_dtype=torch.bfloat16)
    dv = to_dev(c)
    runs = [run(P, dv, K, **HP) for _ in range(3)]
    torch.cuda.synchronize()
    for r in runs[1:]:
        assert torch.equal(r[0], runs[0][0]) and torch.equal(r[1], runs[0][1]) and torch.equal(r[2], runs[0][2])
        for x, y in zip(r[3], runs[0][3]):
            assert torch.equal(x, y)
    with pytest.raises(P.TttError) as e:   # a step count without moments
        run(P, dv, K, step=3, **HP)
    assert e.value.code == P.TTT_ERR_SHAPE
    c96 = P.synthetic.reference_test_inputs(1501, 1, 1, 32, 96, 16, io_dtype=torch.bfloat16)
    with pytest.raises(P.TttError) as e:
        run(P, to_dev(c96), 16, **HP)
    assert e.value.code == P.TTT_ERR_UNSUPPORTED


def test_linear_adam_inner_model_with_remainder(P):
    """FusedLinearAdam.forward over a sequence that is not a multiple of the mini-batch: the remainder is one short
    mini-batch (inner.rs:40-47) that continues from the moments and the step count of the full ones."""
    B, H, d, K, seq = 2, 2, 64, 16, 16 * 3 + 5
    c = P.synthetic.reference_test_inputs(1600, B, H, seq, d, K, io_dtype=torch.float32)
    dv = to_dev(c)
    model = P.FusedLinearAdam(P.ModelConfig(H, d, P.TTTConfig(mini_batch_size=K)), P.TTTLinearAdamConfig(lr=5e-3),
                              dv["W0"], dv["b0"], dv["gamma"], dv["beta"])
    assert model.name() == "TTTLinearAdam"
    state = model.init_state(B)
    te_seq = c["token_eta"].repeat(seq // K + 1)[:seq]   # token_eta [seq], sliced per mini-batch (inner.rs:123-130)
    out = model.forward(state, P.TTTInputsInner(P.Qkv(dv["xq"], dv["xk"], dv["xv"]), te_seq.to("cuda:0"), dv["lr"]))
    torch.cuda.synchronize()
    n = np_inputs(c)
    ro, st = orc.linear_adam_forward(n["W0"], n["b0"], n["xq"], n["xk"], n["xv"], te_seq.double().numpy(), n["lr"],
                                     n["gamma"], n["beta"], K=K, adam_lr=5e-3)
    assert state.step == st["step"] == 4
    assert_close(out, ro, 1e-4, "out")
    W0 = np.broadcast_to(n["W0"][None], st["W"].shape)
    assert_close(state.weight.double().cpu().numpy() - W0, st["W"] - W0, 1e-3, "W movement", min_frac=0.99)
    assert_close(state.weight_v, st["Wv"], 1e-4, "Wv")
