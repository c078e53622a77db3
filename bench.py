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
    # the forward on the projections as the GEMMs leave them: head split, RoPE, lr gate and token_eta formed inside the
    # inner kernel's tile loads (one kernel in place of ttt_inner_inputs followed by ttt_linear_fwd)
    "linear_fwd_fused_inputs_125m_bf16": dict(cfg=1, B=32, H=12, d=64, seq=2048, K=16, io="bf16", kind="linear_fwd_fused"),
    "stack8_d128_seq8192_bf16": dict(cfg=4, B=4, H=16, d=128, seq=8192, K=16, io="bf16", kind="stack"),
}


def linear_fwd_bytes(B, H, seq, d, s):
    """Compulsory traffic of a forward: xq, xk, xv in, out written once, lr in."""
    return B * H * seq * (4 * d * s + s)


def linear_bwd_bytes(B, H, seq, d, s):
    """Backward: xq, xk, xv, d_out in; d_xq, d_xk, d_xv out; lr in, d_lr out."""
    return B * H * seq * (7 * d * s + 2 * s)


def cpu_baseline(c, K, kind, budget_s=12.0):
    """Times the C/OpenMP port of the reference CPU path (oracle/ttt_oracle.c) on the host cores on the same inputs
    (f32 arithmetic on the stored values), on a bounded batch slice.  Forward workloads time the forward; the
    TTT-Linear forward+backward workloads time forward and backward (what a training step of the reference's CPU
    backend runs for this path); the C port has no TTT-MLP backward, so that workload times the forward only and
    says so."""
    import numpy as np
    from oracle import c_oracle
    cores = min(len(os.sched_getaffinity(0)), int(os.environ.get("OMP_NUM_THREADS", "9999")))
    n = {k: v.float().numpy() for k, v in c.items()}
    B, H, seq, d = n["xq"].shape
    sl = lambda keys, nb: [n[k][:nb] if k in ("xq", "xk", "xv", "lr", "d_out") else n[k] for k in keys]
    lin = ("W0", "b0", "xq", "xk", "xv", "token_eta", "lr", "gamma", "beta")
    if kind in ("mlp_fwd", "mlp_fwd_bwd"):
        keys = ("W1", "b1", "W2", "b2", "xq", "xk", "xv", "token_eta", "lr", "gamma", "beta")
        run = lambda nb: c_oracle.mlp_fwd(*sl(keys, nb), K=K, dtype=np.float32, nthreads=cores)
        what = "forward" if kind == "mlp_fwd" else "forward only (the C port has no TTT-MLP backward)"
    elif kind == "linear_fwd_bwd":
        def run(nb):
            c_oracle.linear_fwd(*sl(lin, nb), K=K, dtype=np.float32, nthreads=cores)
            c_oracle.linear_bwd(*sl(lin + ("d_out",), nb), K=K, dtype=np.float32, nthreads=cores)
        what = "forward + backward (all nine gradients)"
    else:
        run = lambda nb: c_oracle.linear_fwd(*sl(lin, nb), K=K, dtype=np.float32, nthreads=cores)
        what = "forward"
    t0 = time.perf_counter()
    run(1)
    t_one = time.perf_counter() - t0
    Bs = max(1, min(B, int(budget_s / 4 / max(t_one, 1e-4))))
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        run(Bs)
        times.append(time.perf_counter() - t0)
    t = sum(times) / len(times)
    return {"value": Bs * seq / t, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"C/OpenMP f32 port of the reference CPU path, {what}, same inputs, batch {Bs} of "
                      f"{B} (tokens/s is batch-normalised), mean of 3 runs, {t:.3f} s per run"}


def cpu_baseline_stack(layers_cpu, K, io_dtype, torch, B):
    """The long-context stack on the host cores: the C/OpenMP ports of the TTT-Linear and TTT-MLP forward chained
    layer by layer as the workload defines it (layer input = previous output + that layer's projections, sums rounded
    to the I/O type), on batch entry 0 of the same inputs (units are independent, tokens/s is batch-normalised)."""
    import numpy as np
    from oracle import c_oracle
    cores = min(len(os.sched_getaffinity(0)), int(os.environ.get("OMP_NUM_THREADS", "9999")))
    L1 = [{k: (v[:1] if k in ("xq", "xk", "xv", "lr") else v) for k, v in L.items()} for L in layers_cpu]
    seq = layers_cpu[0]["xq"].shape[2]
    f = lambda t: t.float().numpy()

    def run():
        x = None
        for L in L1:
            q, k, v = (L["xq"], L["xk"], L["xv"]) if x is None else \
                tuple((x + L[n].float()).to(io_dtype) for n in ("xq", "xk", "xv"))
            if "W2" in L:
                o = c_oracle.mlp_fwd(f(L["W1"]), f(L["b1"]), f(L["W2"]), f(L["b2"]), f(q), f(k), f(v), f(L["token_eta"]),
                                     f(L["lr"]), f(L["gamma"]), f(L["beta"]), K=K, dtype=np.float32, nthreads=cores)[0]
            else:
                o = c_oracle.linear_fwd(f(L["W0"]), f(L["b0"]), f(q), f(k), f(v), f(L["token_eta"]), f(L["lr"]),
                                        f(L["gamma"]), f(L["beta"]), K=K, dtype=np.float32, nthreads=cores)[0]
            x = torch.from_numpy(o).to(io_dtype).float()
        return x

    run()
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    t = sum(times) / len(times)
    return {"value": seq / t, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"C/OpenMP f32 ports of the reference CPU path (TTT-Linear and TTT-MLP forward) chained through the "
                      f"{len(L1)} layers, same inputs, batch 1 of {B} (tokens/s is batch-normalised), mean of 3 runs after "
                      f"one warm-up, {t:.3f} s per run"}


def cpu_baseline_fused(fused_cpu, K, base_lr, budget_s=12.0):
    """The forward from the projections on the host cores: the numpy restatement of the producers (head split, RoPE,
    lr gate, token_eta: oracle.inner_loop_inputs, float32) followed by the C/OpenMP port of the TTT-Linear forward, on
    a bounded batch slice of the same inputs."""
    import numpy as np
    from oracle import c_oracle, ttt_oracle as orc
    cores = min(len(os.sched_getaffinity(0)), int(os.environ.get("OMP_NUM_THREADS", "9999")))
    raw = {k: v.float().numpy() for k, v in fused_cpu["raw"].items()}
    par = {k: v.float().numpy() for k, v in fused_cpu["par"].items()}
    B, seq, H, d = raw["xq"].shape
    cos, sin = orc.rope_cos_sin(seq, 0, K, d)
    tidx = (1.0 / np.arange(1, K + 1)).astype(np.float32)

    def run(nb):
        q, k, v, lr, te = orc.inner_loop_inputs(raw["xq"][:nb], raw["xk"][:nb], raw["xv"][:nb], raw["lg"][:nb],
                                                np.zeros(H, np.float32), base_lr, tidx, np.zeros(K, np.float32), K,
                                                cos, sin, dtype=np.float32)
        c = np.ascontiguousarray
        c_oracle.linear_fwd(par["W0"], par["b0"], c(q), c(k), c(v), te[:K].astype(np.float32), c(lr), par["gamma"],
                            par["beta"], K=K, dtype=np.float32, nthreads=cores)

    t0 = time.perf_counter()
    run(1)
    t_one = time.perf_counter() - t0
    Bs = max(1, min(B, int(budget_s / 4 / max(t_one, 1e-4))))
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        run(Bs)
        times.append(time.perf_counter() - t0)
    t = sum(times) / len(times)
    return {"value": Bs * seq / t, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"numpy f32 restatement of the producers (one thread) + C/OpenMP f32 port of the TTT-Linear forward "
                      f"({cores} threads), same inputs, batch {Bs} of {B} (tokens/s is batch-normalised), mean of 3 runs "
                      f"after one probe, {t:.3f} s per run"}


class LinearCalls:
    """The TTT-Linear entry points on preallocated buffers: what a step of the benchmark issues is the C-ABI call
    and nothing else (no allocation, no copies), so the device time between the events around a call is the time of
    its kernels."""

    def __init__(self, pkg, dv, B, H, seq, d, K, dtype, ci, ckpt_format, with_bwd):
        import ctypes as C
        import torch
        self.pkg, self.C = pkg, C
        dev = dv["xq"].device
        f32 = dict(dtype=torch.float32, device=dev)
        self.desc = pkg.TttDesc(B, H, seq, d, K, 1e-6, ci, pkg.TTT_BF16 if dtype == torch.bfloat16 else pkg.TTT_F32,
                                0, 0, int(ckpt_format), 0)
        self.dv = dv
        self.out = torch.empty_like(dv["xq"])
        self.W, self.b = torch.empty((B, H, d, d), **f32), torch.empty((B, H, d), **f32)
        self.Wc = self.bc = None
        if with_bwd:
            n = pkg.lib().ttt_linear_num_checkpoints(C.byref(self.desc))
            self.Wc, self.bc = torch.empty((B, H, n, d, d), **f32), torch.empty((B, H, n, d), **f32)
            self.g = dict(xq=torch.empty_like(dv["xq"]), xk=torch.empty_like(dv["xq"]), xv=torch.empty_like(dv["xq"]),
                          W=torch.empty((B, H, d, d), **f32), b=torch.empty((B, H, d), **f32),
                          lr=torch.empty_like(dv["lr"]), te=torch.empty(seq, **f32), gam=torch.empty((H, d), **f32),
                          bet=torch.empty((H, d), **f32))
        self.stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
        # the backward takes a workspace where the library has a kernel that uses one (f32 I/O up to 128 units: two
        # workgroups per unit); allocated once, outside the timed region
        self.ws = None
        if with_bwd:
            nbytes = pkg.lib().ttt_linear_bwd_workspace_bytes(C.byref(self.desc))
            if nbytes > 0:
                self.ws = torch.empty((int(nbytes),), dtype=torch.uint8, device=dev)

    def _p(self, t):
        return None if t is None else self.C.c_void_p(t.data_ptr())

    def fwd(self):
        d, p = self.dv, self._p
        self.pkg._lib.check(self.pkg.lib().ttt_linear_fwd(
            self.C.byref(self.desc), p(d["xq"]), p(d["xk"]), p(d["xv"]), p(d["W0"]), p(d["b0"]), p(d["token_eta"]),
            p(d["lr"]), p(d["gamma"]), p(d["beta"]), p(self.out), p(self.W), p(self.b), p(self.Wc), p(self.bc),
            self.stream))

    def bwd(self):
        d, p, g = self.dv, self._p, self.g
        self.pkg._lib.check(self.pkg.lib().ttt_linear_bwd_ws(
            self.C.byref(self.desc), p(d["xq"]), p(d["xk"]), p(d["xv"]), p(d["W0"]), p(d["b0"]), p(d["token_eta"]),
            p(d["lr"]), p(d["gamma"]), p(d["beta"]), p(self.Wc), p(self.bc), p(d["d_out"]), None, None, p(g["xq"]),
            p(g["xk"]), p(g["xv"]), p(g["W"]), p(g["b"]), p(g["lr"]), p(g["te"]), p(g["gam"]), p(g["bet"]),
            p(self.ws), self.stream))


def fwd_kernel_name(io, units):
    """The TTT-Linear forward kernel the library picks at head_dim 64 and mini_batch 16: with f32 I/O and a CU per
    (batch, head) unit the variant with a control wave that copies the operands global -> LDS."""
    return "ttt_linear_fwd_dma_kernel" if io == "f32" and units <= 256 else "ttt_linear_fwd_sk_kernel"


def measured_counters(workload):
    """HBM bytes per launch and matrix-pipe utilisation of a workload's dominant kernel, as measured with rocprofv3
    counters and kept in profiles/traffic.json (not quantities of this run: counters cannot be read from inside it)."""
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if not os.path.exists(tpath):
        return None, None
    t = json.load(open(tpath))
    return t.get(workload), t.get("mfma_util", {}).get(workload)


def time_parts(parts, steps, torch):
    """Average device time (s) of each named call, measured with HIP events on the launch stream around that call
    alone, over `steps` repetitions of the whole sequence."""
    ev = [[(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in parts]
          for _ in range(steps)]
    for row in ev:
        for (e0, e1), (_, fn) in zip(row, parts):
            e0.record()
            fn()
            e1.record()
    torch.cuda.synchronize()
    return {name: sum(row[i][0].elapsed_time(row[i][1]) for row in ev) / steps / 1e3
            for i, (name, _) in enumerate(parts)}


def run_workload(name, a, pkg, torch):
    w = WORKLOADS[name]
    B, H, d, seq, K, io, kind = w["B"], w["H"], w["d"], w["seq"], w["K"], w["io"], w["kind"]
    dtype = {"bf16": torch.bfloat16, "f32": torch.float32}[io]
    s = 2 if io == "bf16" else 4
    ci = a.checkpoint_interval
    dev = torch.device("cuda:0")
    th = B * H * seq  # token-heads
    parts = None      # [(kernel name, call)] when a step is a sequence of separately timed calls
    c = None

    if kind == "stack":
        # 8 layers (6 TTT-Linear then 2 TTT-MLP); layer input = previous output + fresh projections
        layers, layers_cpu = [], []
        for li in range(8):
            cl = pkg.synthetic.baseline_inputs(40 + li, B, H, seq, d, K, io_dtype=dtype, mlp=li >= 6)
            layers.append({k: v.to(dev) for k, v in cl.items()})
            if not a.no_cpu_baseline:   # batch entry 0 is all the CPU leg reads
                layers_cpu.append({k: (v[:1].clone() if k in ("xq", "xk", "xv", "lr") else v) for k, v in cl.items()
                                   if k != "lr_logits"})
            del cl

        stack = [dict(L, pq=L["xq"], pk=L["xk"], pv=L["xv"]) for L in layers]
        # wavefront over sequence windows: layer l + 1 works on a window as soon as layer l has left it, windows
        # that are ready together share a launch, and with --stack-streams 2 the TTT-MLP launches run beside the
        # TTT-Linear ones (--stack-chunk 0: one launch per layer, one after the other)
        chunk = a.stack_chunk
        aux = torch.cuda.Stream(dev) if (chunk and a.stack_streams > 1) else None
        nws = pkg.ttt_stack_workspace_bytes(B, H, seq, d, K, dtype, [li >= 6 for li in range(8)], chunk)
        ws = torch.empty(nws, dtype=torch.uint8, device=dev)

        def step():
            # one call: per layer and window the input sums (x read once for xq, xk, xv) and the inner loop
            return (pkg.ttt_stack_forward_raw(stack, layers[0]["token_eta"], K, workspace=ws, chunk_tokens=chunk,
                                              aux_stream=aux, check_lost=False)[0],)
    elif kind == "linear_fwd_fused":
        import ctypes as C
        g = torch.Generator().manual_seed(1234 + w["cfg"])
        raw = {k: torch.randn(*sh, generator=g).to(dtype) for k, sh in
               (("xq", (B, seq, H, d)), ("xk", (B, seq, H, d)), ("xv", (B, seq, H, d)), ("lg", (B, seq, H)))}
        par = pkg.synthetic.baseline_inputs(w["cfg"], 1, H, K, d, K, io_dtype=dtype)   # W0, b0, gamma, beta of the shape
        fused_cpu = dict(raw=raw, par=par)
        rd = {k: v.to(dev) for k, v in raw.items()}
        pd = {k: par[k].to(dev) for k in ("W0", "b0", "gamma", "beta")}
        bias = torch.zeros(H, device=dev)
        tidx = (1.0 / torch.arange(1, K + 1, dtype=torch.float32)).to(dev)
        ltidx = torch.zeros(K, device=dev)
        rope = pkg.rope_cos_sin(K, 0, None, d, dev)
        f32 = dict(dtype=torch.float32, device=dev)
        fo = dict(out=torch.empty((B, H, seq, d), dtype=dtype, device=dev), W=torch.empty((B, H, d, d), **f32),
                  b=torch.empty((B, H, d), **f32))
        desc = pkg.TttDesc(B, H, seq, d, K, 1e-6, 1, pkg.TTT_BF16, 0, 0, 0, 0)
        ptr = lambda t: C.c_void_p(t.data_ptr())
        stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)

        def fused_call():
            pkg._lib.check(pkg.lib().ttt_linear_fwd_fused_inputs(
                C.byref(desc), ptr(rd["xq"]), ptr(rd["xk"]), ptr(rd["xv"]), ptr(rd["lg"]), ptr(bias), C.c_float(1.0),
                ptr(tidx), ptr(ltidx), ptr(rope[0]), ptr(rope[1]), 0, K, ptr(pd["W0"]), ptr(pd["b0"]), ptr(pd["gamma"]),
                ptr(pd["beta"]), ptr(fo["out"]), ptr(fo["W"]), ptr(fo["b"]), None, None, None, None, None, None, None,
                stream))

        def two_pass():
            i = pkg.inner_loop_inputs_raw(rd["xq"], rd["xk"], rd["xv"], rd["lg"], bias, 1.0, tidx, ltidx, K, rope=rope,
                                          pos_wrap=K)
            return pkg.ttt_linear_forward_raw(i.qkv.xq, i.qkv.xk, i.qkv.xv, pd["W0"], pd["b0"], i.token_eta,
                                              i.ttt_lr_eta, pd["gamma"], pd["beta"], K)

        parts = [("ttt_linear_fwd_fused_inputs", fused_call), ("ttt_inner_inputs + ttt_linear_fwd", two_pass)]

        def step():
            fused_call()
            return (fo["out"], fo["W"])
    elif kind in ("inner_inputs", "layer_epilogue"):
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
        if kind in ("linear_fwd", "linear_fwd_bwd"):
            # a checkpoint per mini-batch: what is saved for the backward is the form the library names as the cheapest
            # for the shape ("auto", ttt_linear_best_checkpoint_format): bf16 I/O up to 512 units and head_dim 96, the
            # update factors and the final state (a quarter of the packed bytes; the feature-split backward walks the
            # states back); otherwise the states as operand fragments in kernel order ("packed").
            # --checkpoint-format f32 keeps the reference's f32 matrices.
            ckfmt = 0
            if kind == "linear_fwd_bwd" and ci == 1:
                import ctypes as C
                probe = pkg.TttDesc(B, H, seq, d, K, 1e-6, ci, pkg.TTT_BF16 if dtype == torch.bfloat16 else pkg.TTT_F32,
                                    0, 0, 0, 0)
                best = pkg.lib().ttt_linear_best_checkpoint_format(C.byref(probe))
                ckfmt = {"f32": 0, "packed": 1, "factors": 2, "auto": best}[a.checkpoint_format]
            calls = LinearCalls(pkg, dv, B, H, seq, d, K, dtype, ci, ckfmt, kind == "linear_fwd_bwd")
            if kind == "linear_fwd":
                parts = [("ttt_linear_fwd", calls.fwd)]

                def step():
                    calls.fwd()
                    return (calls.out, calls.W)
            else:
                parts = [("ttt_linear_fwd (writes checkpoints)", calls.fwd), ("ttt_linear_bwd", calls.bwd)]

                def step():
                    calls.fwd()
                    calls.bwd()
                    return (calls.out, calls.g["xq"], calls.g["W"])
        elif kind == "mlp_fwd":
            def step():
                return pkg.ttt_mlp_forward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W1"], dv["b1"], dv["W2"],
                                               dv["b2"], dv["token_eta"], dv["lr"], dv["gamma"], dv["beta"], K)
        else:
            # the forward saves the update factors for the backward (ttt_mlp_fwd_saving + ttt_mlp_bwd_saved), as a
            # training step does: the backward then runs no forward sweep of its own
            def step():
                fw = pkg.ttt_mlp_forward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W1"], dv["b1"], dv["W2"],
                                             dv["b2"], dv["token_eta"], dv["lr"], dv["gamma"], dv["beta"], K,
                                             save_for_backward=True)
                g = pkg.ttt_mlp_backward_raw(dv["xq"], dv["xk"], dv["xv"], dv["W1"], dv["b1"], dv["W2"],
                                             dv["b2"], dv["token_eta"], dv["lr"], dv["gamma"], dv["beta"],
                                             dv["d_out"], K, saved=fw[5])
                return (fw[0], g["d_xq"])

    # status word of the two-CU TTT-MLP kernel (head_dim 128): it must not move while this workload runs
    lost0 = pkg.mlp_fwd_lost_workgroups()
    for _ in range(a.warmup):
        step()
    torch.cuda.synchronize()
    # the timed region: exactly `steps` steps between two synchronisations, nothing else on the stream
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for _ in range(a.steps):
        res = step()
    ev1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    # device time of the timed region itself (HIP events on the launch stream around the K steps): for a workload
    # whose step is one kernel this is K launches back to back, i.e. the kernel's average duration in the timed run
    region_s = ev0.elapsed_time(ev1) / 1e3 / a.steps
    assert all(torch.isfinite(r.float()).all() for r in res)
    # device times, in passes of their own: HIP events on the launch stream around a whole step, and around each
    # call of a step that consists of several
    dev_s = time_parts([("step", step)], a.steps, torch)["step"]
    part_s = time_parts(parts, a.steps, torch) if parts else None
    lost = pkg.mlp_fwd_lost_workgroups() - lost0
    assert lost == 0, f"{lost} workgroups of the two-CU TTT-MLP kernel waited for their partner in vain"

    pass_name = {"linear_fwd": "fwd", "linear_fwd_bwd": "fwd+bwd", "mlp_fwd": "fwd", "mlp_fwd_bwd": "fwd+bwd",
                 "stack": "fwd", "inner_inputs": "inner-loop inputs", "layer_epilogue": "layer epilogue",
                 "linear_fwd_fused": "fwd from the projections"}[kind]
    out = {
        "metric": f"inner-loop tokens/sec ({pass_name}) at 125M shape" if d == 64 else
                  f"inner-loop tokens/sec ({pass_name})",
        "value": B * seq / (wall / a.steps),
        "unit": "tokens/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": wall / a.steps * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "data": "synthetic",
        "config": {"workload": name, "batch": B, "heads": H, "head_dim": d, "seq_len": seq,
                   "mini_batch": K, "io_dtype": io, "pass": pass_name},
    }
    traffic, mfma_util = measured_counters(name)
    counters = {"traffic": traffic, "traffic_source": "profiles/traffic.json (rocprofv3 FETCH_SIZE/WRITE_SIZE runs)"
                if traffic is not None else None}
    if mfma_util is not None:
        counters.update(mfma_util=mfma_util, mfma_util_source="profiles/traffic.json (rocprofv3 SQ_VALU_MFMA_BUSY_CYCLES "
                        "of the dominant kernel over its traced duration x 2.4 GHz x 1024 SIMDs)")
    if kind == "linear_fwd":
        alg = linear_fwd_bytes(B, H, seq, d, s)
        k_s = region_s
        out["dtype"] = "bf16" if io == "bf16" else "f32"
        out["config"]["inner_model"] = "TTT-Linear"
        out["roofline"] = {"bound": "hbm", "achieved": alg / k_s / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": alg / k_s / 1e9 / HBM_PEAK_GBS, **counters,
                           "kernel": fwd_kernel_name(io, B * H), "kernel_avg_us": k_s * 1e6,
                           "kernel_avg_source": "HIP events around the timed region / steps (launches back to back)",
                           "single_call_event_us": part_s["ttt_linear_fwd"] * 1e6,
                           "step_avg_us": dev_s * 1e6, "algorithmic_bytes": alg}
    elif kind == "linear_fwd_fused":
        # the projections and the logits in, out written once: the bytes of the inner loop itself; the two-pass path
        # moves 6 d s + 2 s more per token-head (the [B,H,seq,d] copies written and read back)
        alg = linear_fwd_bytes(B, H, seq, d, s)
        k_s, two_s = region_s, part_s["ttt_inner_inputs + ttt_linear_fwd"]
        out["dtype"] = "bf16"
        out["config"]["inner_model"] = "TTT-Linear"
        out["roofline"] = {"bound": "hbm", "achieved": alg / k_s / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": alg / k_s / 1e9 / HBM_PEAK_GBS, **counters,
                           "kernel": "ttt_linear_fwd_fi_kernel", "kernel_avg_us": k_s * 1e6,
                           "kernel_avg_source": "HIP events around the timed region / steps (launches back to back)",
                           "single_call_event_us": part_s["ttt_linear_fwd_fused_inputs"] * 1e6,
                           "step_avg_us": dev_s * 1e6, "algorithmic_bytes": alg,
                           "other_kernels": [{"kernel": "ttt_inner_inputs_kernel + ttt_linear_fwd_sk_kernel (the two "
                                                        "passes this kernel replaces, same inputs, same run)",
                                              "kernel_avg_us": two_s * 1e6,
                                              "algorithmic_bytes": alg + th * (6 * d * s + 2 * s)}]}
    elif kind in ("inner_inputs", "layer_epilogue"):
        # inner_inputs: xq, xk, xv read and written once, logits in, lr out; epilogue: inner_out and gate in, out written
        alg = th * (6 * d * s + 2 * s) if kind == "inner_inputs" else th * 3 * d * s
        out["dtype"] = "f32"
        out["roofline"] = {"bound": "hbm", "achieved": alg / dev_s / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": alg / dev_s / 1e9 / HBM_PEAK_GBS, **counters,
                           "kernel": "ttt_inner_inputs_kernel" if kind == "inner_inputs" else "ttt_layer_epilogue_kernel",
                           "kernel_avg_us": dev_s * 1e6, "algorithmic_bytes": alg}
    elif kind == "linear_fwd_bwd":
        # dominant kernel: the backward.  bf16 I/O: bf16 matrix operands, the pair of passes is bound by HBM in the
        # limit (7 d s + 2 s bytes per token-head for the backward); f32 I/O: true-f32 matrix products,
        # 18 d^2 + 22 K d flop per token-head, bound by the f32 matrix pipe.
        lds = ci != 1
        bwd_s, fwd_s = part_s["ttt_linear_bwd"], part_s["ttt_linear_fwd (writes checkpoints)"]
        if ckfmt == 2:  # a [16 x d] bf16 factor per mini-batch and the final state per unit
            ck_bytes = th * (16 * d * 2) // K + B * H * (d * d + d) * 4
        else:
            ck_bytes = th * (d * d * (2 if (ckfmt == 1 and io == "bf16") else 4) + d * 4) // (ci * K)  # written once, read once
        out["dtype"] = io
        out["config"].update(inner_model="TTT-Linear", checkpoint_interval=ci,
                             checkpoint_format=("f32 row-major", "packed", "update factors")[ckfmt])
        kname = ("ttt_linear_bwd_kernel" if lds else
                 "ttt_linear_bwd_pair_kernel (two workgroups per unit)" if calls.ws is not None else "ttt_linear_bwd_mw_kernel")
        if io == "bf16" and not lds:
            alg = linear_bwd_bytes(B, H, seq, d, s)
            roof = {"bound": "hbm", "achieved": alg / bwd_s / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": alg / bwd_s / 1e9 / HBM_PEAK_GBS, "algorithmic_bytes": alg}
        else:
            flops = th * (18 * d * d + 22 * K * d)
            roof = {"bound": "mfma", "achieved": flops / bwd_s / 1e12, "peak": F32_MFMA_PEAK_TF, "unit": "TFLOP/s",
                    "frac": flops / bwd_s / 1e12 / F32_MFMA_PEAK_TF, "algorithmic_flops": flops,
                    "algorithmic_bytes": linear_bwd_bytes(B, H, seq, d, s)}
        out["roofline"] = {**roof, **counters, "kernel": kname, "kernel_avg_us": bwd_s * 1e6,
                           "step_avg_us": dev_s * 1e6, "checkpoint_bytes_each_way": ck_bytes,
                           "other_kernels": [{"kernel": fwd_kernel_name(io, B * H) + " (writes checkpoints)",
                                              "kernel_avg_us": fwd_s * 1e6,
                                              "algorithmic_bytes": linear_fwd_bytes(B, H, seq, d, s)}],
                           "step_algorithmic_bytes": linear_fwd_bytes(B, H, seq, d, s) + linear_bwd_bytes(B, H, seq, d, s),
                           "step_algorithmic_flops": th * (24 * d * d + 26 * K * d)}
    elif kind == "mlp_fwd":
        flops = th * (56 * d * d + 20 * K * d)
        # bf16 I/O: register-resident kernels, bf16 matrix operands with f32 accumulation and state; f32 I/O: the
        # LDS-tile kernel with f32 products
        rr = io == "bf16"
        peak = BF16_MFMA_PEAK_TF if rr else F32_MFMA_PEAK_TF
        out["dtype"] = "bf16" if rr else "f32"
        out["config"]["inner_model"] = "TTT-MLP"
        out["roofline"] = {"bound": "mfma", "achieved": flops / dev_s / 1e12, "peak": peak,
                           "unit": "TFLOP/s", "frac": flops / dev_s / 1e12 / peak, **counters,
                           "kernel": ("ttt_mlp_fwd_rr_kernel" if d <= 96 else "ttt_mlp_fwd_cl2_kernel") if rr else "ttt_mlp_fwd_kernel",
                           "kernel_avg_us": dev_s * 1e6, "algorithmic_flops": flops}
    elif kind == "mlp_fwd_bwd":
        # forward (56 d^2 + 20 K d) and the reverse scan's 14 state-sized and 7 rank-16 products:
        # (56 + 14*8 + 7*8) d^2 flop per token-head, K-sized terms aside.  The forward saves the update factors, so the
        # backward runs no forward sweep of its own.
        flops = th * (224 * d * d)
        # bf16 I/O up to head_dim 96: every product of the scan takes bf16 operands (f32 accumulation, f32 state and
        # gradient accumulators in memory); otherwise true-f32 products
        bf = io == "bf16" and d <= 96
        peak = BF16_MFMA_PEAK_TF if bf else F32_MFMA_PEAK_TF
        out["dtype"] = "bf16" if bf else "f32"
        out["config"]["inner_model"] = "TTT-MLP"
        out["roofline"] = {"bound": "mfma", "achieved": flops / dev_s / 1e12, "peak": peak,
                           "unit": "TFLOP/s", "frac": flops / dev_s / 1e12 / peak, **counters,
                           "kernel": "ttt_mlp_fwd_rr_kernel (forward, saving the update factors) + ttt_mlp_bwd_kernel (whole step)",
                           "kernel_avg_us": dev_s * 1e6, "algorithmic_flops": flops}
    else:
        flops = th * (6 * (6 * d * d + 4 * K * d) + 2 * (56 * d * d + 20 * K * d))
        out["dtype"] = "bf16"   # register-resident kernels: bf16 MFMA operands, f32 accumulation and state
        out["config"]["inner_model"] = "6 x TTT-Linear + 2 x TTT-MLP"
        out["roofline"] = {"bound": "mfma", "achieved": flops / dev_s / 1e12, "peak": BF16_MFMA_PEAK_TF,
                           "unit": "TFLOP/s", "frac": flops / dev_s / 1e12 / BF16_MFMA_PEAK_TF, **counters,
                           "kernel": "ttt_stack_fwd: 8 layers x %d sequence windows, windows of a diagonal in one launch per kind, %d stream(s) (whole step)"
                                     % (seq // a.stack_chunk if a.stack_chunk else 1, 2 if (a.stack_chunk and a.stack_streams > 1) else 1),
                           "kernel_avg_us": dev_s * 1e6, "algorithmic_flops": flops}
        out["config"]["stack_chunk_tokens"] = a.stack_chunk
        out["config"]["stack_streams"] = 2 if (a.stack_chunk and a.stack_streams > 1) else 1
    if not a.no_cpu_baseline and c is not None:
        out["cpu_baseline"] = cpu_baseline(c, K, kind)
    elif not a.no_cpu_baseline and kind == "stack":
        out["cpu_baseline"] = cpu_baseline_stack(layers_cpu, K, dtype, torch, B)
    elif not a.no_cpu_baseline and kind == "linear_fwd_fused":
        out["cpu_baseline"] = cpu_baseline_fused(fused_cpu, K, 1.0)
    return out


# the headline metric names the forward AND the forward+backward at the 125M shape: the default run measures the
# forward (BASELINE config 1) as the line's own value and, as `extra` entries, the two forward+backward workloads
# (bf16 at the config-1 shape, f32 = BASELINE config 2), the TTT-MLP forward (config 3) with its forward+backward,
# the 8-layer long-context stack (config 4), and the forward of config 1 on the projections (producers fused in)
DEFAULT_EXTRA = ("linear_fwd_bwd_125m_bf16_b32", "linear_fwd_bwd_125m_f32_b8", "mlp_fwd_d96_bf16",
                 "mlp_fwd_bwd_d96_bf16", "stack8_d128_seq8192_bf16", "linear_fwd_fused_inputs_125m_bf16")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default=None, choices=sorted(WORKLOADS) + ["hbm_copy_calibration"])
    ap.add_argument("--checkpoint-interval", type=int, default=1)
    ap.add_argument("--checkpoint-format", default="auto", choices=["auto", "factors", "packed", "f32"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--stack-chunk", type=int, default=2048, help="stack workload: tokens per wavefront window (0: none)")
    ap.add_argument("--stack-streams", type=int, default=2, choices=[1, 2], help="stack workload: 2 = TTT-MLP launches on a second stream")
    ap.add_argument("--no-extra", action="store_true", help="default run: only the forward, not the fwd+bwd entries")
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
    default_run = a.workload is None
    out = run_workload(a.workload or "linear_fwd_125m_bf16", a, pkg, torch)
    if default_run and not a.no_extra:
        out["extra"] = [run_workload(name, a, pkg, torch) for name in DEFAULT_EXTRA]
    print(json.dumps(out))


if __name__ == "__main__":
    main()
