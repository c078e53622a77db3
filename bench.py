"""Benchmark of the fused TTT inner loop on one MI355X.

A step is one pass of the hot path over one batch of synthetic input that is already
resident in HBM.  Default workload = the TTT-Linear forward at the 125M shape
(B=32, H=12, d=64, seq=2048, mini-batch 16, bf16 I/O, f32 state).  Prints ONE JSON line.

Throughput follows the reference's definition: tokens/s = batch*seq / seconds of the inner
loop only, with Q/K/V, lr and token_eta precomputed (reference rust/cli/src/bench.rs:153-191,329).
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

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E

WORKLOADS = {
    # name: (config_idx, B, H, d, seq, K, io dtype, kind)
    "linear_fwd_125m_bf16": (1, 32, 12, 64, 2048, 16, "bf16", "linear_fwd"),
    "linear_fwd_125m_f32_b8": (2, 8, 12, 64, 2048, 16, "f32", "linear_fwd"),
    "linear_fwd_cfg0_f32": (0, 1, 4, 64, 256, 16, "f32", "linear_fwd"),
}


def algorithmic_bytes(B, H, seq, d, s):
    """Compulsory traffic of the forward: xq, xk, xv in, out written once, lr in."""
    return B * H * seq * (4 * d * s + s)


def cpu_baseline(c, K, budget_s=20.0):
    """Times the C port of the reference CPU path (oracle/ttt_oracle.c) on the host cores, on
    the same inputs (f32 arithmetic on the stored values)."""
    import numpy as np
    from oracle import c_oracle
    cores = min(len(os.sched_getaffinity(0)), int(os.environ.get("OMP_NUM_THREADS", "9999")))
    n = {k: v.float().numpy() for k, v in c.items()}
    B, H, seq, d = n["xq"].shape
    args = (n["W0"], n["b0"], n["xq"], n["xk"], n["xv"], n["token_eta"], n["lr"], n["gamma"], n["beta"])
    # bounded sample: whole workload when it fits the time budget, else a batch slice
    t0 = time.perf_counter()
    c_oracle.linear_fwd(*[a[:1] if a.ndim >= 3 and a.shape[0] == B else a for a in args], K=K,
                        dtype=np.float32, nthreads=cores)
    t_one = time.perf_counter() - t0
    Bs = max(1, min(B, int(budget_s / 4 / max(t_one, 1e-4))))
    sl = [a[:Bs] if a.ndim >= 3 and a.shape[0] == B else a for a in args]
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        c_oracle.linear_fwd(*sl, K=K, dtype=np.float32, nthreads=cores)
        times.append(time.perf_counter() - t0)
    t = sum(times) / len(times)
    return {"value": Bs * seq / t, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"C/OpenMP f32 port of the reference CPU path, same inputs, batch {Bs} of {B} "
                      f"(tokens/s is batch-normalised), mean of 3 runs, {t:.3f} s per run"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="linear_fwd_125m_bf16", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; --gpus must be 1 (the path shards over "
                 "batch*heads with no communication, see DESIGN.md)")

    import torch
    pkg = importlib.import_module("ttt-rs_amd")
    cfg, B, H, d, seq, K, io, kind = WORKLOADS[a.workload]
    dtype = {"bf16": torch.bfloat16, "f32": torch.float32}[io]
    s = 2 if io == "bf16" else 4
    c = pkg.synthetic.baseline_inputs(cfg, B, H, seq, d, K, io_dtype=dtype)
    dev = torch.device("cuda:0")
    dv = {k: v.to(dev) for k, v in c.items()}

    def step():
        return pkg.ttt_linear_forward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W0"], dv["b0"],
                                          dv["token_eta"], dv["lr"], dv["gamma"], dv["beta"], K)

    for _ in range(a.warmup):
        step()
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
          for _ in range(a.steps)]
    t0 = time.perf_counter()
    for e0, e1 in ev:
        e0.record()          # events sit on the stream the kernel is launched on
        out = step()
        e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    kern_ms = [e0.elapsed_time(e1) for e0, e1 in ev]
    avg_kernel_s = sum(kern_ms) / len(kern_ms) / 1e3
    assert torch.isfinite(out[0].float()).all()

    ms_per_step = wall / a.steps * 1e3
    alg = algorithmic_bytes(B, H, seq, d, s)
    achieved = alg / avg_kernel_s / 1e9
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tpath):
        traffic = json.load(open(tpath)).get(a.workload)
    res = {
        "metric": "inner-loop tokens/sec (fwd) at 125M shape",
        "value": B * seq / (wall / a.steps),
        "unit": "tokens/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 I/O, f32 state and accumulation" if io == "bf16" else "f32",
        "data": "synthetic",
        "config": {"workload": a.workload, "batch": B, "heads": H, "head_dim": d, "seq_len": seq,
                   "mini_batch": K, "io_dtype": io, "inner_model": "TTT-Linear", "pass": "forward"},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                     "kernel": "ttt_linear_fwd_kernel", "kernel_avg_us": avg_kernel_s * 1e6,
                     "algorithmic_bytes": alg},
    }
    if not a.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline(c, K)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
