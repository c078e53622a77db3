"""Shared helpers for the parity tests."""
import numpy as np
import torch

# Tolerances: f32 rel <= 1e-4, bf16 rel <= 2e-2 (max-norm relative per tensor), plus an
# elementwise bound |x-ref| <= tol*|ref| + 0.1*tol*max|ref| on at least 99.9 % of elements.
TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2}


def to_np(t):
    if isinstance(t, torch.Tensor):
        return t.detach().to("cpu", torch.float64).numpy()
    return np.asarray(t, dtype=np.float64)


def assert_close(got, ref, tol, name="", min_frac=0.999):
    got, ref = to_np(got), to_np(ref)
    assert got.shape == ref.shape, (name, got.shape, ref.shape)
    assert np.isfinite(got).all(), f"{name}: non-finite values"
    scale = np.abs(ref).max()
    err = np.abs(got - ref)
    rel = err.max() / max(scale, 1e-30)
    assert rel <= tol, f"{name}: max-norm relative error {rel:.3e} > {tol:g}"
    ok = err <= tol * np.abs(ref) + 0.1 * tol * scale
    frac = ok.mean()
    assert frac >= min_frac, f"{name}: only {frac:.5f} of elements within elementwise bound"
    return rel


def np_inputs(c):
    """dict of torch tensors (possibly bf16) -> float64 numpy (exact values of the stored inputs)."""
    return {k: to_np(v) for k, v in c.items()}


def to_dev(c, dev="cuda:0"):
    return {k: v.to(dev) for k, v in c.items()}
