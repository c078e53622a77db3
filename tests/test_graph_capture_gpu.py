"""GPU: the entry points can be recorded into a HIP graph and replayed.

The library enqueues kernels on the caller's stream and nothing else: outputs that are accumulated with atomics are
cleared by fill kernels, not by memset nodes (memset nodes recorded into a graph have given wrong results on
replays after the first), and per-kernel set-up (the request for more than 64 KiB of LDS) happens on the first
eager call of a kernel, which a caller makes before capturing anyway.  Every test records one call sequence,
replays it several times with eager work and synchronisations of the program in between, and compares every
replay with the eager result of the same inputs: bit for bit where nothing is accumulated with atomics, to 1e-5
where it is (d_token_eta, d_gamma, d_beta: the order of the atomic additions is free).
"""
import importlib

import pytest
import torch

from helpers import assert_close, to_dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def P():
    return importlib.import_module("ttt-rs_amd")


ATOMIC = ("grad_token_eta", "grad_ln_weight", "grad_ln_bias")


def replay_and_compare(record, eager, refresh, names_atomic=()):
    """record(): the calls to capture, returning a dict of output tensors; eager(): the same calls outside a graph;
    refresh(i): overwrite the (static) input tensors in place with the i-th set of values."""
    refresh(0)
    eager()  # first eager call: per-kernel set-up happens here, not under capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            held = record()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for i in (1, 2, 0, 3):
        refresh(i)
        want = {k: v.clone() for k, v in eager().items()}
        torch.cuda.synchronize()
        for v in held.values():  # what the replay must overwrite
            v.fill_(float("nan")) if v.is_floating_point() else v.zero_()
        scratch = torch.randn(1 << 16, device="cuda:0").sum()  # the program's own eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.isfinite(scratch)
        for k, v in want.items():
            if k in names_atomic:
                assert_close(held[k], v.double(), 1e-5, f"replay {i} {k}", min_frac=0.99)
            else:
                assert torch.equal(held[k], v), f"replay {i}: {k} differs from the eager call"


@pytest.mark.parametrize("dtype,fmt", [(torch.float32, 0), (torch.bfloat16, 1), (torch.bfloat16, 2)],
                         ids=["f32", "bf16-packed", "bf16-factors"])
def test_linear_forward_backward_replays(P, dtype, fmt):
    B, H, d, K, N = 2, 3, 64, 16, 6
    print(f"case graph capture linear fwd+bwd {dtype} format {fmt}", flush=True)
    sets = [to_dev(P.synthetic.reference_test_inputs(900 + i, B, H, N * K, d, K, io_dtype=dtype)) for i in range(4)]
    gen = torch.Generator().manual_seed(5)
    douts = [torch.randn(B, H, N * K, d, generator=gen).to(dtype).to("cuda:0") for _ in range(4)]
    x = {k: v.clone() for k, v in sets[0].items()}
    dO = douts[0].clone()

    def refresh(i):
        for k in x:
            x[k].copy_(sets[i][k])
        dO.copy_(douts[i])

    def calls():
        out, W, b, Wc, bc = P.ttt_linear_forward_raw(x["xq"], x["xk"], x["xv"], x["W0"], x["b0"], x["token_eta"], x["lr"],
                                                     x["gamma"], x["beta"], K, 1e-6, 1, want_checkpoints=True,
                                                     packed_checkpoints=fmt)
        g = P.ttt_linear_backward_raw(x["xq"], x["xk"], x["xv"], x["W0"], x["b0"], x["token_eta"], x["lr"], x["gamma"],
                                      x["beta"], Wc, bc, dO, K, 1e-6, 1, packed_checkpoints=fmt)
        return dict(out=out, W=W, b=b, **g)

    replay_and_compare(calls, calls, refresh, ATOMIC)


@pytest.mark.parametrize("d", [64, 128], ids=["d64-one-cu", "d128-two-cus"])
def test_mlp_forward_replays(P, d):
    B, H, K, N = 1, 2, 16, 4
    print(f"case graph capture mlp fwd d{d}", flush=True)
    sets = [to_dev(P.synthetic.baseline_inputs(940 + i, B, H, N * K, d, K, io_dtype=torch.bfloat16, mlp=True))
            for i in range(4)]
    x = {k: v.clone() for k, v in sets[0].items()}

    def refresh(i):
        for k in x:
            x[k].copy_(sets[i][k])

    def calls():
        r = P.ttt_mlp_forward_raw(x["xq"], x["xk"], x["xv"], x["W1"], x["b1"], x["W2"], x["b2"], x["token_eta"], x["lr"],
                                  x["gamma"], x["beta"], K)
        return dict(zip(("out", "W1", "b1", "W2", "b2"), r))

    replay_and_compare(calls, calls, refresh)


@pytest.mark.parametrize("streams", [1, 2], ids=["one-stream", "two-streams"])
def test_stack_wavefront_replays(P, streams):
    """ttt_stack_fwd as a wavefront over sequence windows.  With a second stream the call forks from the stream it is
    given and joins it again before it returns (events), which a capture records as parallel branches."""
    from test_stack_gpu import make_layers
    B, H, d, K, seq, chunk = 2, 2, 64, 16, 128, 32
    kinds = [False, True, False, True]
    print(f"case graph capture stack, {streams} stream(s)", flush=True)
    sets = [[{k: v.to("cuda:0") for k, v in L.items()}
             for L in make_layers(P, B, H, seq, d, K, torch.bfloat16, kinds, seed0=300 + 10 * i)] for i in range(4)]
    x = [{k: v.clone() for k, v in L.items()} for L in sets[0]]
    aux = torch.cuda.Stream("cuda:0") if streams == 2 else None

    def refresh(i):
        for L, S in zip(x, sets[i]):
            for k in L:
                L[k].copy_(S[k])

    def calls():
        out, states = P.ttt_stack_forward_raw(x, x[0]["token_eta"], K, chunk_tokens=chunk, aux_stream=aux)
        res = dict(out=out)
        for li, st in enumerate(states):
            for si, t in enumerate(st):
                res[f"state{li}_{si}"] = t
        return res

    replay_and_compare(calls, calls, refresh)


def test_other_forwards_replay(P):
    """The forward on the projections, the Adam forward and the forward of a TTT-MLP with two hidden layers, recorded
    together in one graph: each enqueues one kernel and nothing else."""
    print("case graph capture fused inputs + adam + mlp2", flush=True)
    B, H, d, K, N = 2, 2, 32, 16, 4
    seq = N * K
    dt = torch.bfloat16
    gen = torch.Generator().manual_seed(21)
    sets = [to_dev(P.synthetic.reference_test_inputs(950 + i, B, H, seq, d, K, io_dtype=dt)) for i in range(4)]
    raws = [dict(q=torch.randn(B, seq, H, d, generator=gen).to(dt).to("cuda:0"),
                 k=torch.randn(B, seq, H, d, generator=gen).to(dt).to("cuda:0"),
                 v=torch.randn(B, seq, H, d, generator=gen).to(dt).to("cuda:0"),
                 lg=torch.randn(B, seq, H, generator=gen).to(dt).to("cuda:0")) for _ in range(4)]
    dims = [d, 4 * d, 4 * d, d]
    Ws = [(torch.randn(H, dims[i], dims[i + 1], generator=gen) * 0.02).to("cuda:0") for i in range(3)]
    bs = [(torch.randn(H, dims[i + 1], generator=gen) * 0.02).to("cuda:0") for i in range(3)]
    bias = torch.zeros(H, device="cuda:0")
    tidx = (1.0 / torch.arange(1, K + 1, dtype=torch.float32)).to("cuda:0")
    ltidx = torch.zeros(K, device="cuda:0")
    rope = P.rope_cos_sin(K, 0, None, d, "cuda:0")
    x = {k: v.clone() for k, v in sets[0].items()}
    r = {k: v.clone() for k, v in raws[0].items()}

    def refresh(i):
        for k in x:
            x[k].copy_(sets[i][k])
        for k in r:
            r[k].copy_(raws[i][k])

    def calls():
        f = P.ttt_linear_forward_fused_inputs_raw(r["q"], r["k"], r["v"], r["lg"], bias, 0.8, tidx, ltidx, x["W0"], x["b0"],
                                                  x["gamma"], x["beta"], K, rope=rope, pos_offset=0, pos_wrap=K)
        a = P.ttt_linear_adam_forward_raw(x["xq"], x["xk"], x["xv"], x["W0"], x["b0"], x["token_eta"], x["lr"], x["gamma"],
                                          x["beta"], K)
        m = P.ttt_mlpn_forward_raw(x["xq"], x["xk"], x["xv"], Ws, bs, x["token_eta"], x["lr"], x["gamma"], x["beta"], K)
        return {"fused out": f[0], "fused W": f[1], "adam out": a[0], "adam W": a[1], "adam Wv": a[3][2],
                "mlp2 out": m[0], "mlp2 W2": m[1][1], "mlp2 b3": m[2][2]}

    replay_and_compare(calls, calls, refresh)


def test_mlp_training_pair_and_long_mini_batches_replay(P):
    """ttt_mlp_fwd_saving + ttt_mlp_bwd_saved (the forward's kernel, the copies of the final state into `saved`, the
    fills and the reverse scan) and the TTT-Linear forward + backward at a mini-batch of 32 tokens (the LDS-tile kernels
    on two tiles of token rows), recorded in one graph."""
    print("case graph capture mlp saving pair + K32 linear", flush=True)
    from test_mlp_fwd_gpu import mlp_case
    B, H, d, N = 2, 2, 32, 3
    dt = torch.bfloat16
    gen = torch.Generator().manual_seed(33)
    msets = [to_dev(mlp_case(P, 970 + i, B, H, N * 16, d, 16, dt, "ref")) for i in range(4)]
    lsets = [to_dev(P.synthetic.reference_test_inputs(980 + i, B, H, N * 32, d, 32, io_dtype=dt)) for i in range(4)]
    mdo = [torch.randn(B, H, N * 16, d, generator=gen).to(dt).to("cuda:0") for _ in range(4)]
    ldo = [torch.randn(B, H, N * 32, d, generator=gen).to(dt).to("cuda:0") for _ in range(4)]
    m = {k: v.clone() for k, v in msets[0].items()}
    x = {k: v.clone() for k, v in lsets[0].items()}
    dm, dl = mdo[0].clone(), ldo[0].clone()

    def refresh(i):
        for k in m:
            m[k].copy_(msets[i][k])
        for k in x:
            x[k].copy_(lsets[i][k])
        dm.copy_(mdo[i])
        dl.copy_(ldo[i])

    def calls():
        margs = (m["xq"], m["xk"], m["xv"], m["W1"], m["b1"], m["W2"], m["b2"], m["token_eta"], m["lr"], m["gamma"],
                 m["beta"])
        f = P.ttt_mlp_forward_raw(*margs, 16, save_for_backward=True)
        g = P.ttt_mlp_backward_raw(*margs, dm, 16, saved=f[5])
        lf = P.ttt_linear_forward_raw(x["xq"], x["xk"], x["xv"], x["W0"], x["b0"], x["token_eta"], x["lr"], x["gamma"],
                                      x["beta"], 32, want_checkpoints=True)
        lg = P.ttt_linear_backward_raw(x["xq"], x["xk"], x["xv"], x["W0"], x["b0"], x["token_eta"], x["lr"], x["gamma"],
                                       x["beta"], lf[3], lf[4], dl, 32)
        return {"mlp out": f[0], "mlp W2": f[3], "mlp d_xk": g["d_xk"], "mlp d_W1": g["d_W1"],
                "mlp d_token_eta": g["d_token_eta"], "mlp d_gamma": g["d_gamma"], "lin out": lf[0], "lin W": lf[1],
                "lin grad_xq": lg["grad_xq"], "lin grad_weight": lg["grad_weight"],
                "lin grad_token_eta": lg["grad_token_eta"], "lin grad_ln_bias": lg["grad_ln_bias"]}

    replay_and_compare(calls, calls, refresh,
                       names_atomic=("mlp d_token_eta", "mlp d_gamma", "lin grad_token_eta", "lin grad_ln_bias"))
