"""GPU parity of ttt_stack_fwd (inner models applied layer by layer) through the C ABI.

The long-context benchmark configuration is an 8-layer stack (6 TTT-Linear then 2 TTT-MLP layers, B=4, H=16,
d=128, seq=8192, bf16 I/O) in which layer l runs on (previous output + fresh N(0,1) projections).  (batch, head)
units never mix, so the float64 oracle carried through all eight layers on a two-unit slice is exact for those
units.  Two comparisons:
  * per layer, on the layer input the GPU actually produced (the oracle is fed the GPU's previous output): the
    usual bf16 bar for every layer at full depth;
  * free running: the oracle chains its own outputs (rounded to bf16 where the definition stores them).  Rounding
    differences of one layer are inputs of the next, so the bar widens with depth; the last layer is held to
    three times the single-layer bar.
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


def make_layers(P, B, H, seq, d, K, dtype, kinds, seed0=40):
    layers = []
    for li, mlp in enumerate(kinds):
        c = P.synthetic.baseline_inputs(seed0 + li, B, H, seq, d, K, io_dtype=dtype, mlp=mlp)
        c["pq"], c["pk"], c["pv"] = c.pop("xq"), c.pop("xk"), c.pop("xv")
        layers.append(c)
    return layers


def bf16_round(x):
    return torch.from_numpy(np.asarray(x, dtype=np.float32)).to(torch.bfloat16).double().numpy()


def oracle_layer(L, x, bs, hs, K, dtype):
    """One layer of the float64 oracle on units (bs, hs); x: its input [len(bs), len(hs), seq, d] or None."""
    rnd = bf16_round if dtype == torch.bfloat16 else (lambda v: np.asarray(v, dtype=np.float32).astype(np.float64))
    sl = lambda t: to_np(t[bs][:, hs])
    par = lambda t: to_np(t[hs])
    q, k, v = sl(L["pq"]), sl(L["pk"]), sl(L["pv"])
    if x is not None:
        # the sums are formed in f32 and rounded to the I/O type
        q, k, v = rnd(np.float32(x) + np.float32(q)), rnd(np.float32(x) + np.float32(k)), rnd(np.float32(x) + np.float32(v))
    if "W2" in L:
        return orc.mlp_forward(par(L["W1"]), par(L["b1"]), par(L["W2"]), par(L["b2"]), q, k, v, to_np(L["token_eta"]),
                               sl(L["lr"]), par(L["gamma"]), par(L["beta"]), K=K)
    return orc.linear_forward(par(L["W0"]), par(L["b0"]), q, k, v, to_np(L["token_eta"]), sl(L["lr"]), par(L["gamma"]),
                              par(L["beta"]), K=K)


def run_stack_layerwise(P, dl, K, n, chunk_tokens=0, aux_stream=None):
    """The first n layers through ttt_stack_fwd: output and states of layer n-1."""
    out, states = P.ttt_stack_forward_raw(dl[:n], dl[0]["token_eta"], K, chunk_tokens=chunk_tokens, aux_stream=aux_stream)
    torch.cuda.synchronize()
    return out, states[n - 1]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_small_stack_matches_oracle_layer_by_layer(P, dtype):
    B, H, d, K, seq = 2, 2, 64, 16, 64
    kinds = [False, False, True, False, True]
    print(f"case stack small {dtype}", flush=True)
    layers = make_layers(P, B, H, seq, d, K, dtype, kinds, seed0=70)
    dl = [{k: v.to("cuda:0") for k, v in L.items()} for L in layers]
    bs, hs = [0, 1], [0, 1]
    x_gpu = None
    for n in range(1, len(kinds) + 1):
        out, st = run_stack_layerwise(P, dl, K, n)
        ref = oracle_layer(layers[n - 1], None if x_gpu is None else to_np(x_gpu), bs, hs, K, dtype)
        tol = TOL[dtype]
        assert_close(out, ref[0], tol, f"layer {n - 1} out")
        for g, r, nm in zip(st, ref[1:], ("W1", "b1", "W2", "b2")):
            f32_products = dtype == torch.float32
            assert_close(g, r, 1e-4 if f32_products else tol, f"layer {n - 1} {nm}", min_frac=0.999 if f32_products else 0.99)
        x_gpu = out.cpu()
    # the stack call equals the chain of single-layer calls on explicitly formed sums, bit for bit
    x = None
    for L in dl:
        q, k, v = (L["pq"], L["pk"], L["pv"]) if x is None else (x + L["pq"], x + L["pk"], x + L["pv"])
        if "W2" in L:
            x = P.ttt_mlp_forward_raw(q, k, v, L["W1"], L["b1"], L["W2"], L["b2"], L["token_eta"], L["lr"], L["gamma"],
                                      L["beta"], K)[0]
        else:
            x = P.ttt_linear_forward_raw(q, k, v, L["W0"], L["b0"], L["token_eta"], L["lr"], L["gamma"], L["beta"], K)[0]
    torch.cuda.synchronize()
    assert torch.equal(x, out)


@pytest.mark.parametrize("chunk,two_streams", [(0, False), (2048, True)], ids=["one-launch-per-layer", "wavefront-2048-two-streams"])
def test_config4_stack_chain_full_size(P, chunk, two_streams):
    """Both plans -- one launch per layer, and the wavefront bench.py times (windows of 2048 tokens, TTT-MLP launches
    on a second stream) -- against the float64 oracle carried through all eight layers on two units."""
    B, H, d, K, seq = 4, 16, 128, 16, 8192
    kinds = [False] * 6 + [True] * 2
    dtype = torch.bfloat16
    print(f"case stack config 4 (8 layers, B4 H16 d128 seq8192 bf16), chunk {chunk}, second stream {two_streams}", flush=True)
    layers = make_layers(P, B, H, seq, d, K, dtype, kinds)
    dl = [{k: v.to("cuda:0") for k, v in L.items()} for L in layers]
    aux = torch.cuda.Stream("cuda:0") if two_streams else None
    bs, hs = [1], [3, 12]          # two units
    x_gpu, x_free = None, None
    tol = TOL[dtype]
    for n in range(1, 9):
        out, st = run_stack_layerwise(P, dl, K, n, chunk, aux)
        assert torch.isfinite(out.float()).all()
        sub = out[bs][:, hs]
        # (1) this layer alone, on the input the GPU produced
        ref = oracle_layer(layers[n - 1], None if x_gpu is None else to_np(x_gpu), bs, hs, K, dtype)
        assert_close(sub, ref[0], tol, f"layer {n - 1} out (given the GPU's input)")
        for g, r, nm in zip(st, ref[1:], ("W1", "b1", "W2", "b2")):
            # the biases are sums of 512 update rows of bf16-rounded factors that largely cancel: max-norm bar only
            assert_close(g[bs][:, hs], r, tol, f"layer {n - 1} {nm}", min_frac=0.0 if nm.startswith("b") else 0.99)
        # (2) free-running oracle chain
        free = oracle_layer(layers[n - 1], x_free, bs, hs, K, dtype)
        x_free = bf16_round(free[0])
        rel = np.abs(to_np(sub) - free[0]).max() / np.abs(free[0]).max()
        print(f"  layer {n - 1}: free-running max-norm relative difference {rel:.3e}", flush=True)
        x_gpu = sub.cpu()
    assert_close(sub, free[0], 3 * tol, "last layer, free-running chain", min_frac=0.99)


def rel_max(a, b):
    a, b = a.double(), b.double()
    return float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("d,seq,chunk,n_aux", [(64, 128, 32, 1), (64, 128, 64, 0), (64, 128, 16, 1), (64, 128, 16, 0),
                                               (128, 128, 32, 1), (128, 128, 16, 0), (32, 128, 32, 1), (96, 128, 32, 0),
                                               (64, 512, 256, 1), (128, 512, 256, 0)])
def test_small_stack_wavefront(P, dtype, d, seq, chunk, n_aux):
    """Sequence windows, with and without the second stream: same results as one launch per layer (each window
    re-centres and re-rounds the carried state once, so the bar is a tight tolerance, not bit equality), same bar
    against the oracle, and the same bits on a second call (a missing wait would show as a difference)."""
    B, H, K = 2, 2, 16
    kinds = [False, True, False, False, True]
    print(f"case stack wavefront small {dtype} d {d} seq {seq} chunk {chunk} streams {n_aux}", flush=True)
    layers = make_layers(P, B, H, seq, d, K, dtype, kinds, seed0=90)
    dl = [{k: v.to("cuda:0") for k, v in L.items()} for L in layers]
    te = dl[0]["token_eta"]
    aux = torch.cuda.Stream("cuda:0") if n_aux else None
    plain, plain_st = P.ttt_stack_forward_raw(dl, te, K)
    wave, wave_st = P.ttt_stack_forward_raw(dl, te, K, chunk_tokens=chunk, aux_stream=aux)
    again, again_st = P.ttt_stack_forward_raw(dl, te, K, chunk_tokens=chunk, aux_stream=aux)
    torch.cuda.synchronize()
    assert torch.equal(wave, again)
    for a, b in zip(wave_st, again_st):
        for x, y in zip(a, b):
            assert torch.equal(x, y)
    tol = TOL[dtype]
    # against the plain plan: differences come from one more rounding of the state per window (f32) and from the
    # bf16 roundings of outputs that those perturb (bf16)
    assert rel_max(wave, plain) <= (2e-5 if dtype == torch.float32 else tol)
    for a, b in zip(wave_st, plain_st):
        for x, y in zip(a, b):
            assert rel_max(x, y) <= (2e-5 if dtype == torch.float32 else tol)
    # against the oracle, layer by layer on the input the GPU produced
    bs, hs = [0, 1], [0, 1]
    x_gpu = None
    for n in range(1, len(kinds) + 1):
        out, states = P.ttt_stack_forward_raw(dl[:n], te, K, chunk_tokens=chunk, aux_stream=aux)
        torch.cuda.synchronize()
        ref = oracle_layer(layers[n - 1], None if x_gpu is None else to_np(x_gpu), bs, hs, K, dtype)
        assert_close(out, ref[0], tol, f"layer {n - 1} out")
        for g, r, nm in zip(states[n - 1], ref[1:], ("W1", "b1", "W2", "b2")):
            f32_products = dtype == torch.float32
            assert_close(g, r, 1e-4 if f32_products else tol, f"layer {n - 1} {nm}", min_frac=0.999 if f32_products else 0.99)
        x_gpu = out.cpu()


@pytest.mark.parametrize("kinds,d,seq,chunk,n_aux", [
    ([False, True, False], 64, 96, 32, 1),      # three windows: the last one writes the caller's state buffers
    ([True], 64, 96, 32, 1),                    # a single layer, still in windows
    ([False] * 10, 32, 160, 16, 0),             # ten windows of one kind on a diagonal: two launches (eight per launch)
    ([True] * 3 + [False] * 9, 32, 160, 16, 1),  # Linear layers above MLP layers, more than eight at once
], ids=["odd-windows", "one-layer", "ten-linear", "mlp-below-linear"])
def test_stack_wavefront_plans(P, kinds, d, seq, chunk, n_aux):
    """Plans the other tests do not reach, against the one-launch-per-layer plan (itself held to the oracle above)."""
    B, H, K = 1, 2, 16
    dtype = torch.float32
    print(f"case stack plan {kinds} d {d} seq {seq} chunk {chunk} streams {n_aux}", flush=True)
    layers = make_layers(P, B, H, seq, d, K, dtype, kinds, seed0=120)
    dl = [{k: v.to("cuda:0") for k, v in L.items()} for L in layers]
    te = dl[0]["token_eta"]
    aux = torch.cuda.Stream("cuda:0") if n_aux else None
    plain, plain_st = P.ttt_stack_forward_raw(dl, te, K)
    wave, wave_st = P.ttt_stack_forward_raw(dl, te, K, chunk_tokens=chunk, aux_stream=aux)
    again, _ = P.ttt_stack_forward_raw(dl, te, K, chunk_tokens=chunk, aux_stream=aux)
    torch.cuda.synchronize()
    assert torch.equal(wave, again)
    # rounding differences of a layer are inputs of the next: the bar widens with depth
    bar = 2e-5 * len(kinds)
    assert rel_max(wave, plain) <= bar
    for a, b in zip(wave_st, plain_st):
        for x, y in zip(a, b):
            assert rel_max(x, y) <= bar


def test_stack_wavefront_rejects_bad_plans(P):
    B, H, d, K, seq = 1, 2, 64, 16, 64
    layers = make_layers(P, B, H, seq, d, K, torch.bfloat16, [False, True], seed0=95)
    dl = [{k: v.to("cuda:0") for k, v in L.items()} for L in layers]
    aux = torch.cuda.Stream("cuda:0")
    for bad in (24, 48, 128):   # not a multiple of the mini-batch; not a divisor of seq; longer than seq
        with pytest.raises(P.TttError):
            P.ttt_stack_forward_raw(dl, dl[0]["token_eta"], K, chunk_tokens=bad, aux_stream=aux)
    torch.cuda.synchronize()


def test_stack_reports_lost_workgroups(P):
    """A stack with a TTT-MLP layer at head_dim 128 (two workgroups per unit): the mirror reads the kernel's status
    word around the call.  With the waits made to give up at once the call would return NaN outputs and TTT_OK; the
    word moves, which the test reads itself (the mirror does not raise for the testing hint), and a healthy call
    afterwards leaves it where it was."""
    B, H, d, K, seq = 1, 2, 128, 16, 64
    print("case stack lost workgroups", flush=True)
    layers = make_layers(P, B, H, seq, d, K, torch.bfloat16, [False, True], seed0=97)
    dl = [{k: v.to("cuda:0") for k, v in L.items()} for L in layers]
    torch.cuda.synchronize()
    before = P.mlp_fwd_lost_workgroups()
    out, _ = P.ttt_stack_forward_raw(dl, dl[0]["token_eta"], K, kernel_hint=P.TTT_HINT_TEST_LOST_PARTNER)
    torch.cuda.synchronize()
    assert torch.isnan(out.float()).all()
    assert P.mlp_fwd_lost_workgroups() == before + 2 * B * H
    out, _ = P.ttt_stack_forward_raw(dl, dl[0]["token_eta"], K)   # check_lost defaults to on here
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    assert P.mlp_fwd_lost_workgroups() == before + 2 * B * H


def test_config4_stack_wavefront_full_size(P):
    """The long-context stack as bench.py runs it (windows of 2048 tokens, TTT-MLP launches on a second stream)
    against the plain plan on all 64 units, at the bf16 bar widened for depth as in the chain test, and bit-equal
    on a second call."""
    B, H, d, K, seq = 4, 16, 128, 16, 8192
    kinds = [False] * 6 + [True] * 2
    dtype = torch.bfloat16
    print("case stack config 4 wavefront (chunk 2048, 2 streams)", flush=True)
    layers = make_layers(P, B, H, seq, d, K, dtype, kinds)
    dl = [{k: v.to("cuda:0") for k, v in L.items()} for L in layers]
    te = dl[0]["token_eta"]
    aux = torch.cuda.Stream("cuda:0")
    plain, plain_st = P.ttt_stack_forward_raw(dl, te, K)
    wave, wave_st = P.ttt_stack_forward_raw(dl, te, K, chunk_tokens=2048, aux_stream=aux)
    again, _ = P.ttt_stack_forward_raw(dl, te, K, chunk_tokens=2048, aux_stream=aux)
    torch.cuda.synchronize()
    assert torch.isfinite(wave.float()).all()
    assert torch.equal(wave, again)
    tol = TOL[dtype]
    r = rel_max(wave, plain)
    print(f"  wavefront vs plain, last layer output: max-norm relative difference {r:.3e}", flush=True)
    assert r <= 3 * tol
    for li, (a, b) in enumerate(zip(wave_st, plain_st)):
        for x, y, nm in zip(a, b, ("W1", "b1", "W2", "b2")):
            rr = rel_max(x, y)
            print(f"  layer {li} {nm}: {rr:.3e}", flush=True)
            assert rr <= 3 * tol, (li, nm, rr)
