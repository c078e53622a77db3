"""GPU parity on seeded random shapes: TTT-Linear forward + backward and TTT-MLP forward through the C ABI against
the float64 oracle.  The other GPU tests use the reference's own shapes and the benchmark shapes; this one draws
(batch, heads, head_dim, mini_batch, stages, per-batch state, style of inputs) from a fixed seed, so that shapes
nobody thought of are covered too (odd head counts, every head_dim with short and long mini-batches, one stage).
Bars: the max-norm bar of the other tests (1e-4 / 2e-2) for every tensor; the elementwise band on 99.9 % of the
elements for f32 and on 99 % for bf16 I/O (products with bf16 operands: on these small tensors, mini-batches of one
token included, a few elements in a thousand leave the band while the max-norm error stays far inside its bar)."""
import importlib
import random

import pytest
import torch

from helpers import TOL, assert_close, np_inputs, to_dev
from oracle import ttt_oracle as orc
from test_linear_bwd_gpu import NAMES, compare, oracle_bwd
from test_mlp_fwd_gpu import mlp_case

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def P():
    return importlib.import_module("ttt-rs_amd")


def draw(seed, n, dims):
    rng = random.Random(seed)
    cases = []
    for _ in range(n):
        cs = dict(B=rng.choice([1, 2, 3]), H=rng.choice([1, 2, 3, 5]), d=rng.choice(dims),
                  K=rng.choice([1, 3, 4, 8, 11, 16]), N=rng.choice([1, 2, 5, 9]),
                  style=rng.choice(["ref", "baseline"]), seed=rng.randrange(1 << 20))
        # at least 24 tokens, so that the 99.9 % rule of the elementwise band has more than a few hundred elements to
        # speak of (in a tensor of 320 bf16 values one element outside the band is already 0.3 %)
        cs["N"] = max(cs["N"], -(-24 // cs["K"]))
        cases.append(cs)
    return cases


def linear_inputs(P, cs, dtype):
    gen = P.synthetic.reference_test_inputs if cs["style"] == "ref" else P.synthetic.baseline_inputs
    return gen(cs["seed"], cs["B"], cs["H"], cs["N"] * cs["K"], cs["d"], cs["K"], io_dtype=dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("cs", draw(2024, 10, [32, 64, 96, 128]), ids=lambda c: "B{B}H{H}d{d}K{K}N{N}{style}".format(**c))
def test_linear_forward_random_shape(P, cs, dtype):
    print(f"case random linear fwd {cs} {dtype}", flush=True)
    K = cs["K"]
    c = linear_inputs(P, cs, dtype)
    d = to_dev(c)
    out, W, b = P.ttt_linear_forward_raw(d["xq"], d["xk"], d["xv"], d["W0"], d["b0"], d["token_eta"], d["lr"],
                                         d["gamma"], d["beta"], K)[:3]
    torch.cuda.synchronize()
    n = np_inputs(c)
    ro, rW, rb = orc.linear_forward(n["W0"], n["b0"], n["xq"], n["xk"], n["xv"], n["token_eta"], n["lr"], n["gamma"],
                                    n["beta"], K=K)[:3]
    tol = TOL[dtype]
    frac = 0.99 if dtype == torch.bfloat16 else 0.999
    few = cs["B"] * cs["H"] * cs["d"] < 1000   # one element of a small tensor is already more than 0.1 %
    assert_close(out, ro, tol, "out", min_frac=frac)
    assert_close(W, rW, tol, "W", min_frac=frac)
    assert_close(b, rb, tol, "b", min_frac=0.99 if few else frac)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("cs", draw(7, 8, [32, 64]), ids=lambda c: "B{B}H{H}d{d}K{K}N{N}{style}".format(**c))
def test_linear_backward_random_shape(P, cs, dtype):
    print(f"case random linear bwd {cs} {dtype}", flush=True)
    K = cs["K"]
    c = linear_inputs(P, cs, dtype)
    c.pop("d_out", None)
    g = torch.Generator().manual_seed(cs["seed"] + 1)
    dO = torch.randn(cs["B"], cs["H"], cs["N"] * K, cs["d"], generator=g).to(dtype)
    d = to_dev(c)
    ref = oracle_bwd(c, dO, K)
    # f32 matrices as checkpoints; with bf16 I/O also the update factors (the states are walked back from the end)
    for fmt in ((0,) if dtype == torch.float32 else (0, 2)):
        fw = P.ttt_linear_forward_raw(d["xq"], d["xk"], d["xv"], d["W0"], d["b0"], d["token_eta"], d["lr"], d["gamma"],
                                      d["beta"], K, want_checkpoints=True, packed_checkpoints=fmt)
        got = P.ttt_linear_backward_raw(d["xq"], d["xk"], d["xv"], d["W0"], d["b0"], d["token_eta"], d["lr"],
                                        d["gamma"], d["beta"], fw[3], fw[4], dO.to("cuda:0"), K, packed_checkpoints=fmt)
        torch.cuda.synchronize()
        if dtype == torch.float32:
            compare(got, ref, TOL[dtype])
        else:
            import numpy as np
            for gn, rn in NAMES:
                n = np.asarray(ref[rn]).size   # in a tensor of 64 elements one element outside the band is 1.6 %
                assert_close(got[gn], ref[rn], TOL[dtype], f"format {fmt} {gn}", min_frac=min(0.99, 1.0 - 1.5 / n))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("cs", draw(99, 6, [32, 64, 96, 128]), ids=lambda c: "B{B}H{H}d{d}K{K}N{N}{style}".format(**c))
def test_mlp_forward_random_shape(P, cs, dtype):
    print(f"case random mlp fwd {cs} {dtype}", flush=True)
    K = cs["K"]
    c = mlp_case(P, cs["seed"], cs["B"], cs["H"], cs["N"] * K, cs["d"], K, dtype, cs["style"])
    d = to_dev(c)
    got = P.ttt_mlp_forward_raw(d["xq"], d["xk"], d["xv"], d["W1"], d["b1"], d["W2"], d["b2"], d["token_eta"], d["lr"],
                                d["gamma"], d["beta"], K)
    torch.cuda.synchronize()
    n = np_inputs(c)
    ref = orc.mlp_forward(n["W1"], n["b1"], n["W2"], n["b2"], n["xq"], n["xk"], n["xv"], n["token_eta"], n["lr"],
                          n["gamma"], n["beta"], K=K)
    tol = TOL[dtype]
    frac = 0.99 if dtype == torch.bfloat16 else 0.999
    for g, r, nm in zip(got, ref, ("out", "W1", "b1", "W2", "b2")):
        assert_close(g, r, tol, nm, min_frac=0.99 if nm.startswith("b") else frac)


def draw_tiles(seed, n):
    """Shapes served by the LDS-tile backward's variants: mini-batches of 17 - 32 tokens at head_dim 32 (any checkpoint
    interval), head_dim 96 with a checkpoint interval above 1, head_dim 128 with f32 I/O."""
    rng = random.Random(seed)
    cases = []
    for _ in range(n):
        kind = rng.choice(["k32", "d96", "d128"])
        cs = dict(B=rng.choice([1, 2]), H=rng.choice([1, 2, 3]), style=rng.choice(["ref", "baseline"]),
                  seed=rng.randrange(1 << 20), kind=kind)
        if kind == "k32":
            cs.update(d=32, K=rng.choice([17, 20, 27, 32]), N=rng.choice([1, 2, 5]), ci=rng.choice([1, 2, 3]))
        elif kind == "d96":
            cs.update(d=96, K=rng.choice([3, 8, 16]), N=rng.choice([3, 4, 7]), ci=rng.choice([2, 3, 5]))
        else:
            cs.update(d=128, K=rng.choice([5, 16]), N=rng.choice([2, 3, 6]), ci=1)
        cs["N"] = max(cs["N"], -(-24 // cs["K"]))
        cases.append(cs)
    return cases


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("cs", draw_tiles(31, 9), ids=lambda c: "{kind}B{B}H{H}K{K}N{N}ci{ci}{style}".format(**c))
def test_linear_tile_kernels_random_shape(P, cs, dtype):
    if cs["kind"] == "d128" and dtype == torch.bfloat16:
        pytest.skip("bf16 I/O at head_dim 128 runs the register-resident backward (test_linear_bwd_gpu.py)")
    print(f"case random tile kernels {cs} {dtype}", flush=True)
    K, ci = cs["K"], cs["ci"]
    c = linear_inputs(P, cs, dtype)
    c.pop("d_out", None)
    g = torch.Generator().manual_seed(cs["seed"] + 1)
    dO = torch.randn(cs["B"], cs["H"], cs["N"] * K, cs["d"], generator=g).to(dtype)
    d = to_dev(c)
    fw = P.ttt_linear_forward_raw(d["xq"], d["xk"], d["xv"], d["W0"], d["b0"], d["token_eta"], d["lr"], d["gamma"],
                                  d["beta"], K, 1e-6, ci, want_checkpoints=True)
    got = P.ttt_linear_backward_raw(d["xq"], d["xk"], d["xv"], d["W0"], d["b0"], d["token_eta"], d["lr"], d["gamma"],
                                    d["beta"], fw[3], fw[4], dO.to("cuda:0"), K, 1e-6, ci)
    torch.cuda.synchronize()
    n = np_inputs(c)
    ro, rW, rb = orc.linear_forward(n["W0"], n["b0"], n["xq"], n["xk"], n["xv"], n["token_eta"], n["lr"], n["gamma"],
                                    n["beta"], K=K)[:3]
    tol = TOL[dtype]
    frac = 0.99 if dtype == torch.bfloat16 else 0.999
    assert_close(fw[0], ro, tol, "out", min_frac=frac)
    assert_close(fw[1], rW, tol, "W", min_frac=frac)
    ref = oracle_bwd(c, dO, K)
    if dtype == torch.float32:
        compare(got, ref, tol)
    else:
        import numpy as np
        for gn, rn in NAMES:
            nel = np.asarray(ref[rn]).size
            assert_close(got[gn], ref[rn], tol, gn, min_frac=min(0.99, 1.0 - 1.5 / nel))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("cs", draw(5, 6, [32, 64, 96]), ids=lambda c: "B{B}H{H}d{d}K{K}N{N}{style}".format(**c))
def test_mlp_backward_random_shape(P, cs, dtype):
    """TTT-MLP backward: f32 I/O (f32 products) to 1e-4, bf16 I/O (register-resident sweep, bf16 operands in the scan)
    to the bf16 bar, max-norm per tensor.  The eight gradients that belong to a (batch, head) unit are compared on the
    whole call.  d_token_eta, d_gamma and d_beta are sums over units in which the units' contributions cancel (in one
    drawn case to a fiftieth of their size at one position), so the max-norm of the SUM is no measure of a kernel that
    computes every unit to the bar: they are compared unit by unit (calls on one unit each, same bar), and the whole
    call must return the sum of those calls (to the rounding of the f32 atomics that add them up)."""
    print(f"case random mlp bwd {cs} {dtype}", flush=True)
    import numpy as np
    K, B, H = cs["K"], cs["B"], cs["H"]
    c = mlp_case(P, cs["seed"], B, H, cs["N"] * K, cs["d"], K, dtype, cs["style"])
    g = torch.Generator().manual_seed(cs["seed"] + 2)
    c["d_out"] = torch.randn(B, H, cs["N"] * K, cs["d"], generator=g).to(dtype)
    d = to_dev(c)
    n = np_inputs(c)
    run = lambda x: P.ttt_mlp_backward_raw(x["xq"], x["xk"], x["xv"], x["W1"], x["b1"], x["W2"], x["b2"], x["token_eta"],
                                           x["lr"], x["gamma"], x["beta"], x["d_out"], K)
    ora = lambda x: orc.mlp_backward(x["W1"], x["b1"], x["W2"], x["b2"], x["xq"], x["xk"], x["xv"], x["token_eta"],
                                     x["lr"], x["gamma"], x["beta"], x["d_out"], K=K)
    per_bh, per_h = ("xq", "xk", "xv", "lr", "d_out"), ("W1", "b1", "W2", "b2", "gamma", "beta")
    unit = lambda x, b, h: {**{k: x[k][b:b + 1, h:h + 1] for k in per_bh}, **{k: x[k][h:h + 1] for k in per_h},
                            "token_eta": x["token_eta"]}
    got = run(d)
    torch.cuda.synchronize()
    ref = ora(n)

    def held(gv, rv, k, tol):
        gv, rv = gv.double().cpu().numpy() if torch.is_tensor(gv) else gv, np.asarray(rv)
        rel = np.abs(gv - rv).max() / max(np.abs(rv).max(), 1e-30)
        assert np.isfinite(gv).all() and rel <= tol, f"{k}: max-norm relative error {rel:.3e} > {tol}"

    for k in ("d_xq", "d_xk", "d_xv", "d_W1", "d_b1", "d_W2", "d_b2", "d_lr"):
        io_out = k in ("d_xq", "d_xk", "d_xv", "d_lr")
        held(got[k], ref[k], k, TOL[dtype] if (io_out or dtype == torch.bfloat16) else 1e-4)
    tol = TOL[dtype] if dtype == torch.bfloat16 else 1e-4
    sums = {k: np.zeros_like(np.asarray(ref[k])) for k in ("d_token_eta", "d_gamma", "d_beta")}
    for b in range(B):
        for h in range(H):
            gu = run({k: v.contiguous() for k, v in unit(d, b, h).items()})
            torch.cuda.synchronize()
            ru = ora(unit(n, b, h))
            for k in sums:
                held(gu[k], ru[k], f"{k} of unit ({b}, {h})", tol)
            sums["d_token_eta"] += gu["d_token_eta"].double().cpu().numpy()
            sums["d_gamma"][h] += gu["d_gamma"].double().cpu().numpy()[0]
            sums["d_beta"][h] += gu["d_beta"].double().cpu().numpy()[0]
    for k in sums:
        gv = got[k].double().cpu().numpy()
        scale = max(np.abs(sums[k]).max(), 1e-30)
        assert np.abs(gv - sums[k]).max() <= 1e-5 * scale * B * H, f"{k}: the whole call is not the sum of its units"
