"""Writes the golden fixtures of this folder:  python tests/golden/make_fixtures.py

Each .npz holds the inputs of one small case of the fused TTT inner loop (float32, so the stored values are
exactly what every implementation is given) and the float64 results of the numpy oracle for it: forward outputs,
final state, checkpoints, and all gradients for a stored upstream gradient.

Provenance.  The reference commits no input/output vectors for this path: its Rust tests draw random inputs and
compare the fused kernels with its own Burn-op model at run time (rust/core/src/test_utils.rs:613-743), and its
PyTorch script generates fixtures when run (reference/validate.py:40-54).  Neither was run here.  The vectors
therefore come from this repository's oracle, whose functions are pinned by independent mathematics in
tests/test_oracle_pins.py; the fixtures freeze those results, so that a later change to the oracle, to the C port
or to a kernel is measured against numbers that no longer move with the code under test.

Shapes follow the reference's own test shapes (rust/fused/src/linear_fused_tile/tests.rs:23-89: (B,H,d,K,stages,ci)
= (2,2,32,8,4,2), (1,4,32,16,2,1)) plus a d = 64 case and two TTT-MLP cases; inputs are drawn as the reference's test
harness draws them (test_utils.rs:126-156).
"""
import importlib
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
orc = importlib.import_module("oracle.ttt_oracle")
synthetic = importlib.import_module("ttt-rs_amd.synthetic")

# name -> (B, H, d, K, stages, checkpoint_interval)
LINEAR = {"linear_b2_h2_d32_k8_n4_ci2": (2, 2, 32, 8, 4, 2),
          "linear_b1_h4_d32_k16_n2_ci1": (1, 4, 32, 16, 2, 1),
          "linear_b1_h2_d64_k16_n3_ci1": (1, 2, 64, 16, 3, 1)}
# name -> (B, H, d, K, stages)
MLP = {"mlp_b1_h2_d32_k8_n3": (1, 2, 32, 8, 3),
       "mlp_b1_h1_d64_k16_n2": (1, 1, 64, 16, 2)}


def f64(t):
    return t.double().numpy()


def linear_case(name, B, H, d, K, N, ci, seed):
    seq = N * K
    c = synthetic.reference_test_inputs(seed, B, H, seq, d, K)
    g = torch.Generator().manual_seed(seed + 1)
    d_out = torch.randn(B, H, seq, d, generator=g)
    d_W = torch.randn(B, H, d, d, generator=g) * 0.1
    d_b = torch.randn(B, H, d, generator=g) * 0.1
    a = [f64(c[k]) for k in ("W0", "b0", "xq", "xk", "xv", "token_eta", "lr", "gamma", "beta")]
    out, W, b, Wc, bc = orc.linear_forward(*a, K=K, checkpoint_interval=ci)
    gr = orc.linear_backward(*a, f64(d_out), K=K, d_W_out=f64(d_W), d_b_out=f64(d_b))
    data = {"in_" + k: v.numpy() for k, v in c.items()}
    data.update(in_d_out=d_out.numpy(), in_d_W_out=d_W.numpy(), in_d_b_out=d_b.numpy(),
                meta=np.array([B, H, d, K, N, ci], dtype=np.int64),
                out=out, W_out=W, b_out=b, W_ckpt=Wc, b_ckpt=bc)
    data.update({"grad_" + k: v for k, v in gr.items()})
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **data)


def mlp_case(name, B, H, d, K, N, seed):
    seq, m = N * K, 4 * d
    c = synthetic.reference_test_inputs(seed, B, H, seq, d, K)
    g = torch.Generator().manual_seed(seed + 1)
    n = lambda *s: torch.randn(*s, generator=g)
    c.pop("W0"), c.pop("b0")
    c.update(W1=n(H, d, m) * 0.02, b1=n(H, m) * 0.02, W2=n(H, m, d) * 0.02, b2=n(H, d) * 0.02)
    d_out = n(B, H, seq, d)
    dst = [n(B, H, d, m) * 0.1, n(B, H, m) * 0.1, n(B, H, m, d) * 0.1, n(B, H, d) * 0.1]
    a = [f64(c[k]) for k in ("W1", "b1", "W2", "b2", "xq", "xk", "xv", "token_eta", "lr", "gamma", "beta")]
    fw = orc.mlp_forward(*a, K=K)
    gr = orc.mlp_backward(*a, f64(d_out), K=K, d_state_out=[f64(x) for x in dst])
    data = {"in_" + k: v.numpy() for k, v in c.items()}
    data.update(in_d_out=d_out.numpy(), meta=np.array([B, H, d, K, N], dtype=np.int64))
    data.update({"in_d_state_%d" % i: x.numpy() for i, x in enumerate(dst)})
    data.update({"fwd_%d" % i: x for i, x in enumerate(fw)})
    data.update({"grad_" + k: v for k, v in gr.items()})
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **data)


if __name__ == "__main__":
    for i, (name, (B, H, d, K, N, ci)) in enumerate(LINEAR.items()):
        linear_case(name, B, H, d, K, N, ci, 9000 + 10 * i)
    for i, (name, (B, H, d, K, N)) in enumerate(MLP.items()):
        mlp_case(name, B, H, d, K, N, 9500 + 10 * i)
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
