"""GPU parity against the committed fixtures of tests/golden (written once by tests/golden/make_fixtures.py from
the numpy oracle; the reference commits no vectors for this path).  Inputs are the stored float32 arrays, results
are compared with the stored float64 ones: forward, final state, checkpoints and every gradient, through the C ABI.
Tolerance: 1e-4 (f32 I/O), as in tests/helpers.py.
"""
import glob
import importlib
import os

import numpy as np
import pytest
import torch

from helpers import assert_close

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
LINEAR = sorted(glob.glob(os.path.join(GOLDEN, "linear_*.npz")))
MLP = sorted(glob.glob(os.path.join(GOLDEN, "mlp_*.npz")))
LIN_IN = ("xq", "xk", "xv", "W0", "b0", "token_eta", "lr", "gamma", "beta")
MLP_IN = ("xq", "xk", "xv", "W1", "b1", "W2", "b2", "token_eta", "lr", "gamma", "beta")
LIN_GRADS = [("grad_xq", "d_xq"), ("grad_xk", "d_xk"), ("grad_xv", "d_xv"), ("grad_weight", "d_W0"),
             ("grad_bias", "d_b0"), ("grad_ttt_lr_eta", "d_lr"), ("grad_token_eta", "d_token_eta"),
             ("grad_ln_weight", "d_gamma"), ("grad_ln_bias", "d_beta")]
MLP_GRADS = ("d_xq", "d_xk", "d_xv", "d_W1", "d_b1", "d_W2", "d_b2", "d_lr", "d_token_eta", "d_gamma", "d_beta")
TOL = 1e-4


@pytest.fixture(scope="module")
def P():
    return importlib.import_module("ttt-rs_amd")


def dev(f, k):
    return torch.from_numpy(f["in_" + k]).to("cuda:0")


def test_fixtures_are_present():
    assert len(LINEAR) == 3 and len(MLP) == 2


@pytest.mark.parametrize("path", LINEAR, ids=[os.path.basename(p)[:-4] for p in LINEAR])
def test_linear_forward_and_backward_match_fixture(P, path):
    print("case golden", os.path.basename(path), flush=True)
    f = np.load(path)
    K, ci = int(f["meta"][3]), int(f["meta"][5])
    a = [dev(f, k) for k in LIN_IN]
    out, W, b, Wc, bc = P.ttt_linear_forward_raw(*a, K, 1e-6, ci, want_checkpoints=True)
    for g, k in zip((out, W, b, Wc, bc), ("out", "W_out", "b_out", "W_ckpt", "b_ckpt")):
        assert_close(g, f[k], TOL, k)
    g = P.ttt_linear_backward_raw(*a, Wc, bc, dev(f, "d_out"), K, 1e-6, ci, dev(f, "d_W_out"), dev(f, "d_b_out"))
    torch.cuda.synchronize()
    for gn, rn in LIN_GRADS:
        assert_close(g[gn], f["grad_" + rn], TOL, gn)


@pytest.mark.parametrize("path", MLP, ids=[os.path.basename(p)[:-4] for p in MLP])
def test_mlp_forward_and_backward_match_fixture(P, path):
    print("case golden", os.path.basename(path), flush=True)
    f = np.load(path)
    K = int(f["meta"][3])
    a = [dev(f, k) for k in MLP_IN]
    fw = P.ttt_mlp_forward_raw(*a, K)
    for i, g in enumerate(fw):
        assert_close(g, f["fwd_%d" % i], TOL, "fwd_%d" % i)
    got = P.ttt_mlp_backward_raw(*a, dev(f, "d_out"), K, d_state_out=[dev(f, "d_state_%d" % i) for i in range(4)])
    torch.cuda.synchronize()
    for k in MLP_GRADS:
        assert_close(got[k], f["grad_" + k], TOL, k)
