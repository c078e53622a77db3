"""Benchmark of the fused TTT inner loop on one MI355X.

A step is one pass of the hot path over one batch of synthetic input that is already
resident in HBM.  Default workload = the TTT-Linear forward at the 125M shape
(B=32, H=12, d=64, seq=2048, mini-batch 16, bf16 I/O, f32 state).  Prints ONE JSON line.

Throughput follows the reference's definition: tokens/s = batch*seq / seconds of the inner
loop only, with Q/K/V, lr and token_eta precomputed (reference rust/cli/src/bench.rs:153-191,329).
Other workloads (--workload) cover the remaining benchmark configurations.
"""
from __future__ import annotations

import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E
F32_MFMA_PEAK_TF = 157.3   # MI355X dense fp32 matrix
BF16_MFMA_PEAK_TF = 2500.0

WORKLOADS = {
    # name: dict(cfg=config index, B, H, d, seq, K, io, kind)
    "linear_fwd_125m_bf16": dict(cfg=1, B=32, H=12, d=64, seq=2048, K=16, io="bf16", kind="linear_fwd"),
    "linear_fwd_cfg0_f32": dict(cfg=0, B=1, H=4, d=64, seq=256, K=16, io="f32", kind="linear_fwd"),
    "linear_fwd_125m_f32_b8": dict(cfg=2, B=8, H=12, d=64, seq=2048, K=16, io="f32", kind="linear_fwd"),
    "linear_fwd_bwd_125m_f32_b8": dict(cfg=2, B=8, H=12, d=64, seq=2048, K=16, io="f32", kind="linear_fwd_bwd"),
    "mlp_fwd_d96_bf16": dict(cfg=3, B=8, H=16, d=96, seq=2048, K=16, io="bf16", kind="mlp_fwd"),
    "mlp_fwd_bwd_d96_bf16": dict(cfg=3, B=8, H=16, d=96, seq=2048, K=16, io="bf16", kind="mlp_fwd_bwd"),
    "linear_fwd_bwd_125m_bf16_b32": dict(cfg=1, B=32, H=12, d=64, seq=2048, K=16, io="bf16", kind="linear_fwd_bwd"),
    # the elementwise passes either side of the inner loop at the 125M shape (hidden 768)
    "inner_inputs_125m_bf16": dict(cfg=1, B=32, H=12, d=64, seq=2048, K=16, io="bf16", kind="inner_inputs"),
    "layer_epilogue_125m_bf16": dict(cfg=1, B=32, H=12, d=64, seq=2048, K=16, io="bf16", kind="layer_epilogue"),
    "stack8_d128_seq8192_bf16": dict(cfg=4, B=4, H=16, d=128, seq=8192, K=16, io="bf16", kind="stack"),
}


def linear_fwd_bytes(B, H, seq, d, s):
    """Compulsory traffic of a forward: xq, xk, xv in, out written once, lr in."""
    return B * H * seq * (4 * d * s + s)


def linear_bwd_bytes(B, H, seq, d, s):
    """Backward: xq, xk, xv, d_out in; d_xq, d_xk, d_xv out; lr in, d_lr out."""
    return B * H * seq * (7 * d * s + 2 * s)


def cpu_baseline(c, K, kind, budget_s=20.0):
    """Times the C/OpenMP port of the reference CPU path (oracle/ttt_oracle.c) on the host cores
    on the same inputs (f32 arithmetic on the stored values), on a bounded batch slice."""
    import numpy as np
    from oracle import c_oracle
    cores = min(len(os.sched_getaffinity(0)), int(os.environ.get("OMP_NUM_THREADS", "9999")))
    n = {k: v.float().numpy() for k, v in c.items()}
    B, H, seq, d = n["xq"].shape
    if kind in ("mlp_fwd", "mlp_fwd_bwd"):
        fn = c_oracle.mlp_fwd
        keys = ("W1", "b1", "W2", "b2", "xq", "xk", "xv", "token_eta", "lr", "gamma", "beta")
    else:
        fn = c_oracle.linear_fwd
        keys = ("W0", "b0", "xq", "xk", "xv", "token_eta", "lr", "gamma", "beta")
    bsl = lambda nb: [n[k][:nb] if k in ("xq", "xk", "xv", "lr") else n[k] for k in keys]
    t0 = time.perf_counter()
    fn(*bsl(1), K=K, dtype=np.float32, nthreads=cores)
    t_one = time.perf_counter() - t0
    Bs = max(1, min(B, int(budget_s / 4 / max(t_one, 1e-4))))
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        fn(*bsl(Bs), K=K, dtype=np.float32, nthreads=cores)
        times.append(time.perf_counter() - t0)
    t = sum(times) / len(times)
    what = "forward" if kind not in ("linear_fwd_bwd", "mlp_fwd_bwd") else "forward only (the C port has no backward)"
    return {"value": Bs * seq / t, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"C/OpenMP f32 port of the reference CPU path, {what}, same inputs, batch {Bs} of "
                      f"{B} (tokens/s is batch-normalised), mean of 3 runs, {t:.3f} s per run"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="linear_fwd_125m_bf16", choices=sorted(WORKLOADS) + ["hbm_copy_calibration"])
    ap.add_argument("--checkpoint-interval", type=int, default=1)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; --gpus must be 1 (the path shards over "
                 "batch*heads with no communication inside the scan; only parameter gradients reduce)")

    import torch
    if a.workload == "hbm_copy_calibration":
        # plain device-to-device copy of known size: reference point for the FETCH_SIZE / WRITE_SIZE
        # counters (rocprofv3 --pmc) that the `traffic` figures are scaled by
        nbytes = 512 << 20
        src = torch.empty(nbytes, dtype=torch.uint8, device="cuda:0").random_(0, 255)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        for _ in range(a.steps):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"workload": a.workload, "copy_bytes": nbytes, "steps": a.steps}))
        return
    pkg = importlib.import_module("ttt-rs_amd")
    w = WORKLOADS[a.workload]
    B, H, d, seq, K, io, kind = w["B"], w["H"], w["d"], w["seq"], w["K"], w["io"], w["kind"]
    dtype = {"bf16": torch.bfloat16, "f32": torch.float32}[io]
    s = 2 if io == "bf16" else 4
    ci = a.checkpoint_interval
    dev = torch.device("cuda:0")
    th = B * H * seq  # token-heads

    if kind == "stack":
        # 8 layers (6 TTT-Linear then 2 TTT-MLP); layer input = previous output + fresh projections
        layers = []
        for li in range(8):
            c = pkg.synthetic.baseline_inputs(40 + li, B, H, seq, d, K, io_dtype=dtype, mlp=li >= 6)
            layers.append({k: v.to(dev) for k, v in c.items()})
        c = None

        def step():
            x = None
            for li, L in enumerate(layers):
                q, k, v = (L["xq"], L["xk"], L["xv"]) if x is None else (x + L["xq"], x + L["xk"], x + L["xv"])
                if li < 6:
                    x = pkg.ttt_linear_forward_raw(q, k, v, L["W0"], L["b0"], L["token_eta"], L["lr"],
                                                   L["gamma"], L["beta"], K)[0]
                else:
                    x = pkg.ttt_mlp_forward_raw(q, k, v, L["W1"], L["b1"], L["W2"], L["b2"], L["token_eta"],
                                                L["lr"], L["gamma"], L["beta"], K)[0]
            return (x,)
    elif kind in ("inner_inputs", "layer_epilogue"):
        c = None
        g = torch.Generator().manual_seed(1234 + w["cfg"])
        rn = lambda *sh: torch.randn(*sh, generator=g).to(dtype).to(dev)
        if kind == "inner_inputs":
            xq, xk, xv, lg = rn(B, seq, H, d), rn(B, seq, H, d), rn(B, seq, H, d), rn(B, seq, H)
            bias = torch.zeros(H, device=dev)
            tidx = (1.0 / torch.arange(1, K + 1, dtype=torch.float32)).to(dev)
            ltidx = torch.zeros(K, device=dev)
            rope = pkg.rope_cos_sin(K, 0, None, d, dev)

            def step():
                r = pkg.inner_loop_inputs_raw(xq, xk, xv, lg, bias, 1.0, tidx, ltidx, K, rope=rope, pos_wrap=K)
                return (r.qkv.xq, r.ttt_lr_eta)
        else:
            x, gate = rn(B, H, seq, d), rn(B, seq, H * d)
            gam, bet = torch.ones(H * d, device=dev), torch.zeros(H * d, device=dev)

            def step():
                return (pkg.layer_epilogue_raw(x, gam, bet, gate),)
    else:
        c = pkg.synthetic.baseline_inputs(w["cfg"], B, H, seq, d, K, io_dtype=dtype,
                                          with_dout=kind in ("linear_fwd_bwd", "mlp_fwd_bwd"),
                                          mlp=kind in ("mlp_fwd", "mlp_fwd_bwd"))
        dv = {k: v.to(dev) for k, v in c.items()}
        if kind == "linear_fwd":
            def step():
                return pkg.ttt_linear_forward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W0"], dv["b0"],
                                                  dv["token_eta"], dv["lr"], dv["gamma"], dv["beta"], K)
        elif kind == "mlp_fwd":
            def step():
                return pkg.ttt_mlp_forward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W1"], dv["b1"], dv["W2"],
                                               dv["b2"], dv["token_eta"], dv["lr"], dv["gamma"], dv["beta"], K)
        elif kind == "mlp_fwd_bwd":
            def step():
                fw = pkg.ttt_mlp_forward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W1"], dv["b1"], dv["W2"],
                                             dv["b2"], dv["token_eta"], dv["lr"], dv["gamma"], dv["beta"], K)
                g = pkg.ttt_mlp_backward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W1"], dv["b1"], dv["W2"],
                                             dv["b2"], dv["token_eta"], dv["lr"], dv["gamma"], dv["beta"],
                                             dv["d_out"], K)
                return (fw[0], g["d_xq"])
        else:
            # a checkpoint per mini-batch: checkpoints as operand fragments in kernel order (same gradients bit
            # for bit; bf16 I/O: half the checkpoint traffic); TTT_BENCH_CKPT=f32 keeps the reference's f32 matrices
            packed = ci == 1 and os.environ.get("TTT_BENCH_CKPT") != "f32"

            def step():
                out, W, b, Wc, bc = pkg.ttt_linear_forward_raw(
                    dv["xq"], dv["xk"], dv["xv"], dv["W0"], dv["b0"], dv["token_eta"], dv["lr"],
                    dv["gamma"], dv["beta"], K, 1e-6, ci, want_checkpoints=True, packed_checkpoints=packed)
                g = pkg.ttt_linear_backward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W0"], dv["b0"],
                                                dv["token_eta"], dv["lr"], dv["gamma"], dv["beta"], Wc, bc,
                                                dv["d_out"], K, 1e-6, ci, packed_checkpoints=packed)
                return (out, g["grad_xq"])

    for _ in range(a.warmup):
        step()
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
          for _ in range(a.steps)]
    t0 = time.perf_counter()
    for e0, e1 in ev:
        e0.record()          # events sit on the stream the kernels are launched on
        res = step()
        e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    dev_s = sum(e0.elapsed_time(e1) for e0, e1 in ev) / len(ev) / 1e3  # device time of one step
    assert all(torch.isfinite(r.float()).all() for r in res)

    pass_name = {"linear_fwd": "fwd", "linear_fwd_bwd": "fwd+bwd", "mlp_fwd": "fwd", "mlp_fwd_bwd": "fwd+bwd",
                 "stack": "fwd", "inner_inputs": "inner-loop inputs", "layer_epilogue": "layer epilogue"}[kind]
    out = {
        "metric": f"inner-loop tokens/sec ({pass_name}) at 125M shape" if d == 64 else
                  f"inner-loop tokens/sec ({pass_name})",
        "value": B * seq / (wall / a.steps),
        "unit": "tokens/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": wall / a.steps * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "data": "synthetic",
        "config": {"workload": a.workload, "batch": B, "heads": H, "head_dim": d, "seq_len": seq,
                   "mini_batch": K, "io_dtype": io, "pass": pass_name},
    }
    if kind == "linear_fwd":
        alg = linear_fwd_bytes(B, H, seq, d, s)
        out["dtype"] = "bf16" if io == "bf16" and d <= 64 else "f32"
        out["config"]["inner_model"] = "TTT-Linear"
        out["roofline"] = {"bound": "hbm", "achieved": alg / dev_s / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": alg / dev_s / 1e9 / HBM_PEAK_GBS, "traffic": None,
                           "kernel": "ttt_linear_fwd_sk_kernel", "kernel_avg_us": dev_s * 1e6,
                           "algorithmic_bytes": alg}
    elif kind in ("inner_inputs", "layer_epilogue"):
        # inner_inputs: xq, xk, xv read and written once, logits in, lr out; epilogue: inner_out and gate in, out written
        alg = th * (6 * d * s + 2 * s) if kind == "inner_inputs" else th * 3 * d * s
        out["dtype"] = "f32"
        out["roofline"] = {"bound": "hbm", "achieved": alg / dev_s / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": alg / dev_s / 1e9 / HBM_PEAK_GBS, "traffic": None,
                           "kernel": "ttt_inner_inputs_kernel" if kind == "inner_inputs" else "ttt_layer_epilogue_kernel",
                           "kernel_avg_us": dev_s * 1e6, "algorithmic_bytes": alg}
    elif kind == "linear_fwd_bwd" and io == "bf16" and ci == 1 and os.environ.get("TTT_LINEAR_BWD_KERNEL") != "lds":
        # register-resident backward (bf16 MFMA operands): the pair of passes is bound by HBM in the limit
        alg = linear_fwd_bytes(B, H, seq, d, s) + linear_bwd_bytes(B, H, seq, d, s)
        out["dtype"] = "bf16"
        out["config"].update(inner_model="TTT-Linear", checkpoint_interval=ci,
                             checkpoint_format="f32" if os.environ.get("TTT_BENCH_CKPT") == "f32" else "packed bf16")
        out["roofline"] = {"bound": "hbm", "achieved": alg / dev_s / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": alg / dev_s / 1e9 / HBM_PEAK_GBS, "traffic": None,
                           "kernel": "ttt_linear_fwd_sk_kernel + ttt_linear_bwd_mw_kernel (whole step)",
                           "kernel_avg_us": dev_s * 1e6, "algorithmic_bytes": alg,
                           "checkpoint_bytes": 2 * th * (d * d * (2 if os.environ.get("TTT_BENCH_CKPT") != "f32" else 4) + d * 4) // (ci * K),
                           "algorithmic_flops": th * (24 * d * d + 26 * K * d)}
    elif kind == "linear_fwd_bwd":
        # the backward kernel dominates; it computes in f32 MFMA: 18 d^2 + 22 K d flop per token-head
        flops = th * (24 * d * d + 26 * K * d)
        out["dtype"] = "f32"
        out["config"].update(inner_model="TTT-Linear", checkpoint_interval=ci,
                             checkpoint_format="f32 row-major" if (ci != 1 or os.environ.get("TTT_BENCH_CKPT") == "f32") else "packed")
        out["roofline"] = {"bound": "mfma", "achieved": flops / dev_s / 1e12, "peak": F32_MFMA_PEAK_TF,
                           "unit": "TFLOP/s", "frac": flops / dev_s / 1e12 / F32_MFMA_PEAK_TF, "traffic": None,
                           "kernel": ("ttt_linear_fwd_sk_kernel + ttt_linear_bwd_mw_kernel (whole step)"
                                      if ci == 1 and os.environ.get("TTT_LINEAR_BWD_KERNEL") != "lds" else
                                      "ttt_linear_fwd_sk_kernel + ttt_linear_bwd_kernel (whole step)"),
                           "kernel_avg_us": dev_s * 1e6, "algorithmic_flops": flops,
                           "algorithmic_bytes": linear_fwd_bytes(B, H, seq, d, s) + linear_bwd_bytes(B, H, seq, d, s)}
    elif kind == "mlp_fwd":
        flops = th * (56 * d * d + 20 * K * d)
        # bf16 I/O with d <= 96: register-resident kernel, bf16 MFMA operands with f32 accumulation and
        # state; otherwise the LDS-tile kernel with f32 MFMA
        rr = io == "bf16" and d <= 96 and os.environ.get("TTT_MLP_FWD_KERNEL") != "lds"
        peak = BF16_MFMA_PEAK_TF if rr else F32_MFMA_PEAK_TF
        out["dtype"] = "bf16" if rr else "f32"
        out["config"]["inner_model"] = "TTT-MLP"
        out["roofline"] = {"bound": "mfma", "achieved": flops / dev_s / 1e12, "peak": peak,
                           "unit": "TFLOP/s", "frac": flops / dev_s / 1e12 / peak, "traffic": None,
                           "kernel": "ttt_mlp_fwd_rr_kernel" if rr else "ttt_mlp_fwd_kernel",
                           "kernel_avg_us": dev_s * 1e6, "algorithmic_flops": flops}
    elif kind == "mlp_fwd_bwd":
        # forward (56 d^2 + 20 K d) plus the backward's own forward sweep (Z1, Z2, G1 and the two state updates:
        # 40 d^2; its output branch is not run) and the reverse scan's 14 state-sized and 7 rank-16 products:
        # (56 + 40 + 14*8 + 7*8) d^2 flop per token-head, K-sized terms aside
        flops = th * (264 * d * d)
        out["dtype"] = "f32"
        out["config"]["inner_model"] = "TTT-MLP"
        out["roofline"] = {"bound": "mfma", "achieved": flops / dev_s / 1e12, "peak": F32_MFMA_PEAK_TF,
                           "unit": "TFLOP/s", "frac": flops / dev_s / 1e12 / F32_MFMA_PEAK_TF, "traffic": None,
                           "kernel": "ttt_mlp_fwd_rr_kernel + ttt_mlp_fwd_kernel + ttt_mlp_bwd_kernel (whole step)",
                           "kernel_avg_us": dev_s * 1e6, "algorithmic_flops": flops}
    else:
        flops = th * (6 * (6 * d * d + 4 * K * d) + 2 * (56 * d * d + 20 * K * d))
        out["dtype"] = "bf16"   # register-resident kernels: bf16 MFMA operands, f32 accumulation and state
        out["config"]["inner_model"] = "6 x TTT-Linear + 2 x TTT-MLP"
        out["roofline"] = {"bound": "mfma", "achieved": flops / dev_s / 1e12, "peak": BF16_MFMA_PEAK_TF,
                           "unit": "TFLOP/s", "frac": flops / dev_s / 1e12 / BF16_MFMA_PEAK_TF, "traffic": None,
                           "kernel": "8 layer launches + input adds (whole step)",
                           "kernel_avg_us": dev_s * 1e6, "algorithmic_flops": flops}
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tpath):
        out["roofline"]["traffic"] = json.load(open(tpath)).get(a.workload)
    if not a.no_cpu_baseline and c is not None:
        out["cpu_baseline"] = cpu_baseline(c, K, kind)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
