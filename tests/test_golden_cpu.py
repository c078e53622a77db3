"""The committed fixtures of tests/golden against the two CPU restatements.

The fixtures were written by tests/golden/make_fixtures.py from the numpy oracle (the reference commits no
vectors for this path); they freeze its results.  Here the numpy oracle must still reproduce them to rounding
(an edit that changes its results fails), and the C port, the timed CPU baseline, must agree in f32.
"""
import glob
import os

import numpy as np
import pytest

from oracle import c_oracle, ttt_oracle as orc

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
LINEAR = sorted(glob.glob(os.path.join(GOLDEN, "linear_*.npz")))
MLP = sorted(glob.glob(os.path.join(GOLDEN, "mlp_*.npz")))
LIN_IN = ("W0", "b0", "xq", "xk", "xv", "token_eta", "lr", "gamma", "beta")
MLP_IN = ("W1", "b1", "W2", "b2", "xq", "xk", "xv", "token_eta", "lr", "gamma", "beta")


def rel(a, b):
    return np.abs(np.asarray(a) - b).max() / max(np.abs(b).max(), 1e-300)


def test_fixtures_are_present():
    assert len(LINEAR) == 3 and len(MLP) == 2


@pytest.mark.parametrize("path", LINEAR, ids=[os.path.basename(p)[:-4] for p in LINEAR])
def test_numpy_oracle_reproduces_linear_fixture(path):
    f = np.load(path)
    B, H, d, K, N, ci = f["meta"]
    a = [f["in_" + k].astype(np.float64) for k in LIN_IN]
    got = orc.linear_forward(*a, K=int(K), checkpoint_interval=int(ci))
    for g, k in zip(got, ("out", "W_out", "b_out", "W_ckpt", "b_ckpt")):
        assert rel(g, f[k]) <= 1e-12, k
    gr = orc.linear_backward(*a, f["in_d_out"].astype(np.float64), K=int(K),
                             d_W_out=f["in_d_W_out"].astype(np.float64), d_b_out=f["in_d_b_out"].astype(np.float64))
    for k, v in gr.items():
        assert rel(v, f["grad_" + k]) <= 1e-12, k


@pytest.mark.parametrize("path", MLP, ids=[os.path.basename(p)[:-4] for p in MLP])
def test_numpy_oracle_reproduces_mlp_fixture(path):
    f = np.load(path)
    K = int(f["meta"][3])
    a = [f["in_" + k].astype(np.float64) for k in MLP_IN]
    for i, g in enumerate(orc.mlp_forward(*a, K=K)):
        assert rel(g, f["fwd_%d" % i]) <= 1e-12, i
    dst = [f["in_d_state_%d" % i].astype(np.float64) for i in range(4)]
    gr = orc.mlp_backward(*a, f["in_d_out"].astype(np.float64), K=K, d_state_out=dst)
    for k, v in gr.items():
        assert rel(v, f["grad_" + k]) <= 1e-12, k


@pytest.mark.parametrize("path", LINEAR, ids=[os.path.basename(p)[:-4] for p in LINEAR])
def test_c_port_matches_linear_fixture(path):
    f = np.load(path)
    K = int(f["meta"][3])
    a = [f["in_" + k].astype(np.float64) for k in LIN_IN]
    got = c_oracle.linear_fwd(*a, K=K, dtype=np.float32, nthreads=2)
    for g, k in zip(got, ("out", "W_out", "b_out")):
        assert rel(g, f[k]) <= 2e-4, k


@pytest.mark.parametrize("path", LINEAR, ids=[os.path.basename(p)[:-4] for p in LINEAR])
def test_c_port_backward_matches_linear_fixture(path):
    """The C backward (f32) on the frozen cases, upstream state gradients included."""
    f = np.load(path)
    K = int(f["meta"][3])
    a = [f["in_" + k].astype(np.float64) for k in LIN_IN]
    got = c_oracle.linear_bwd(*a, f["in_d_out"], K=K, dtype=np.float32, nthreads=2, d_W_out=f["in_d_W_out"],
                              d_b_out=f["in_d_b_out"])
    for k, v in got.items():
        assert rel(v, f["grad_" + k]) <= 5e-4, k


@pytest.mark.parametrize("path", MLP, ids=[os.path.basename(p)[:-4] for p in MLP])
def test_c_port_matches_mlp_fixture(path):
    f = np.load(path)
    K = int(f["meta"][3])
    a = [f["in_" + k].astype(np.float64) for k in MLP_IN]
    got = c_oracle.mlp_fwd(*a, K=K, dtype=np.float32, nthreads=2)
    for i, g in enumerate(got):
        assert rel(g, f["fwd_%d" % i]) <= 2e-4, i
