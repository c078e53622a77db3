"""The C oracle (the timed CPU baseline) against the pinned numpy oracle."""
import numpy as np
import pytest

from oracle import c_oracle, ttt_oracle as orc


def case(seed, B, H, seq, d, K, m=None):
    rng = np.random.default_rng(seed)
    r = lambda *s, sc=1.0: rng.standard_normal(s) * sc
    c = dict(xq=r(B, H, seq, d), xk=r(B, H, seq, d), xv=r(B, H, seq, d),
             gamma=1 + r(H, d, sc=0.1), beta=r(H, d, sc=0.1),
             lr=rng.uniform(0.001, 0.02, (B, H, seq)), te=1.0 / np.arange(1, K + 1))
    if m:
        c.update(W1=r(H, d, m, sc=0.05), b1=r(H, m, sc=0.05), W2=r(H, m, d, sc=0.05), b2=r(H, d, sc=0.05))
    else:
        c.update(W0=r(H, d, d, sc=0.05), b0=r(H, d, sc=0.05))
    return c


@pytest.mark.parametrize("B,H,seq,d,K", [(2, 3, 64, 64, 16), (1, 2, 37, 32, 8)])
def test_c_linear_fwd_matches_numpy_oracle(B, H, seq, d, K):
    c = case(1, B, H, seq, d, K)
    ref = orc.linear_forward(c["W0"], c["b0"], c["xq"], c["xk"], c["xv"], c["te"], c["lr"],
                             c["gamma"], c["beta"], K=K)
    for dtype, tol in ((np.float64, 1e-11), (np.float32, 2e-4)):
        got = c_oracle.linear_fwd(c["W0"], c["b0"], c["xq"], c["xk"], c["xv"], c["te"], c["lr"],
                                  c["gamma"], c["beta"], K=K, dtype=dtype, nthreads=2)
        for g, r in zip(got, ref):
            assert np.abs(g - r).max() <= tol * np.abs(r).max()


@pytest.mark.parametrize("B,H,seq,d,K", [(2, 2, 48, 32, 16), (1, 2, 21, 16, 8)])
def test_c_mlp_fwd_matches_numpy_oracle(B, H, seq, d, K):
    c = case(2, B, H, seq, d, K, m=4 * d)
    ref = orc.mlp_forward(c["W1"], c["b1"], c["W2"], c["b2"], c["xq"], c["xk"], c["xv"], c["te"],
                          c["lr"], c["gamma"], c["beta"], K=K)
    for dtype, tol in ((np.float64, 1e-11), (np.float32, 2e-4)):
        got = c_oracle.mlp_fwd(c["W1"], c["b1"], c["W2"], c["b2"], c["xq"], c["xk"], c["xv"], c["te"],
                               c["lr"], c["gamma"], c["beta"], K=K, dtype=dtype, nthreads=2)
        for g, r in zip(got, ref):
            assert np.abs(g - r).max() <= tol * np.abs(r).max()


@pytest.mark.parametrize("B,H,N,d,K", [(2, 3, 4, 64, 16), (1, 2, 3, 32, 8), (1, 1, 1, 16, 4)])
def test_c_linear_bwd_matches_numpy_oracle(B, H, N, d, K):
    """The C backward (the timed CPU baseline of the forward+backward workloads) against the numpy oracle, which is
    itself pinned to torch autograd through the primal per-token formulation (test_oracle_pins.py): all nine
    gradients, float64 to rounding and float32 to 5e-4."""
    seq = N * K
    c = case(3, B, H, seq, d, K)
    rng = np.random.default_rng(30)
    d_out = rng.standard_normal((B, H, seq, d))
    args = (c["W0"], c["b0"], c["xq"], c["xk"], c["xv"], c["te"], c["lr"], c["gamma"], c["beta"], d_out)
    ref = orc.linear_backward(*args, K=K)
    for dtype, tol in ((np.float64, 1e-10), (np.float32, 5e-4)):
        got = c_oracle.linear_bwd(*args, K=K, dtype=dtype, nthreads=2)
        assert set(got) == set(ref)
        for k in ref:
            assert np.abs(got[k] - ref[k]).max() <= tol * np.abs(ref[k]).max(), (k, dtype)
