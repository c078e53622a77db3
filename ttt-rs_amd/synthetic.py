"""Seeded synthetic inputs for the inner loop.

`baseline_inputs` draws what the benchmark configurations describe: N(0,1) activations,
W0 ~ N(0, 0.02^2), b0 = 0, LayerNorm gamma = 1 / beta = 0, lr = (base_lr/d)*sigmoid(N(0,1))
(get_lr, reference rust/layer/src/ttt.rs:205-227) and token_eta[i] = 1/(i+1) inside the
mini-batch (rust/layer/src/ttt.rs:106-110).  `reference_test_inputs` follows the reference's
own test generator (rust/core/src/test_utils.rs:126-156).
Everything is drawn on the CPU in f32 in a fixed order so the same seed gives the same
tensors everywhere; bf16 configurations round activations and lr to bf16 once, here.
"""
from __future__ import annotations

import torch


def _round(t: torch.Tensor, io_dtype: torch.dtype) -> torch.Tensor:
    return t.to(io_dtype)


def baseline_inputs(config_idx: int, B: int, H: int, seq: int, d: int, K: int = 16,
                    io_dtype: torch.dtype = torch.float32, base_lr: float = 1.0,
                    with_dout: bool = False, mlp: bool = False):
    g = torch.Generator(device="cpu")
    g.manual_seed(1234 + config_idx)
    n = lambda *s: torch.randn(*s, generator=g, dtype=torch.float32)
    c = {}
    c["xq"], c["xk"], c["xv"] = n(B, H, seq, d), n(B, H, seq, d), n(B, H, seq, d)
    if mlp:
        c["W1"], c["W2"] = n(H, d, 4 * d) * 0.02, n(H, 4 * d, d) * 0.02
        c["b1"], c["b2"] = torch.zeros(H, 4 * d, dtype=torch.float32), torch.zeros(H, d, dtype=torch.float32)
    else:
        c["W0"] = n(H, d, d) * 0.02
        c["b0"] = torch.zeros(H, d, dtype=torch.float32)
    c["gamma"], c["beta"] = torch.ones(H, d, dtype=torch.float32), torch.zeros(H, d, dtype=torch.float32)
    c["lr_logits"] = n(B, H, seq)  # kept for the chain d lr -> d logits (f32; not an input of the inner loop)
    c["lr"] = (base_lr / d) * torch.sigmoid(c["lr_logits"])
    c["token_eta"] = 1.0 / torch.arange(1, K + 1, dtype=torch.float32)
    if with_dout:
        c["d_out"] = n(B, H, seq, d)
    for k in ("xq", "xk", "xv", "lr", "d_out"):
        if k in c:
            c[k] = _round(c[k], io_dtype)
    return c


def reference_test_inputs(seed: int, B: int, H: int, seq: int, d: int, K: int,
                          io_dtype: torch.dtype = torch.float32, trained_params: bool = True):
    """test_utils.rs:126-156: activations N(0,0.1), lr U(0.01,0.05), token_eta 1/(i+1) tiled;
    parameters N(0,0.02) incl. bias and LayerNorm weight/bias (linear.rs:54-78)."""
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    n = lambda *s: torch.randn(*s, generator=g, dtype=torch.float32)
    c = {}
    c["xq"], c["xk"], c["xv"] = n(B, H, seq, d) * 0.1, n(B, H, seq, d) * 0.1, n(B, H, seq, d) * 0.1
    c["W0"], c["b0"] = n(H, d, d) * 0.02, n(H, d) * 0.02
    if trained_params:
        c["gamma"], c["beta"] = n(H, d) * 0.02, n(H, d) * 0.02
    else:
        c["gamma"], c["beta"] = torch.ones(H, d, dtype=torch.float32), torch.zeros(H, d, dtype=torch.float32)
    c["lr"] = 0.01 + 0.04 * torch.rand(B, H, seq, generator=g, dtype=torch.float32)
    c["token_eta"] = 1.0 / torch.arange(1, K + 1, dtype=torch.float32)
    for k in ("xq", "xk", "xv", "lr"):
        c[k] = _round(c[k], io_dtype)
    return c
