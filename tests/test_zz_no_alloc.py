"""GPU test of ttt_mlp_bwd_static, the entry point that allocates nothing: its workspace is a buffer
inside the library's device image.  Through the C ABI, against ttt_mlp_bwd (caller-owned workspace) on
the same inputs: three calls in a row, the second with a smaller input and the third with the first shape again,
so each later call runs on whatever the earlier ones left in the shared buffer, shrinking and growing.

Outputs written by plain stores must agree bit for bit (same kernels, same order of operations); the three
outputs accumulated with floating-point atomics over (batch, head) units (d_token_eta, d_gamma, d_beta)
are compared to the f32 parity bar of the other MLP backward tests (max-norm relative error 1e-4)."""
import ctypes as C
import importlib

import pytest
import torch

from helpers import assert_close, to_dev
from test_mlp_fwd_gpu import mlp_case

pytestmark = pytest.mark.gpu

PLAIN = ("d_xq", "d_xk", "d_xv", "d_W1", "d_b1", "d_W2", "d_b2", "d_lr")
ATOMIC = ("d_token_eta", "d_gamma", "d_beta")


@pytest.fixture(scope="module")
def P():
    return importlib.import_module("ttt-rs_amd")


def both(P, B, H, d, K, N, dtype, seed, state_grads):
    seq = N * K
    c = to_dev(mlp_case(P, seed, B, H, seq, d, K, dtype, "ref"))
    g = torch.Generator().manual_seed(seed + 1)
    d_out = torch.randn(B, H, seq, d, generator=g).to(dtype).to("cuda:0")
    dst = None
    if state_grads:
        m = 4 * d
        dst = [(torch.randn(*s, generator=g) * 0.1).to("cuda:0")
               for s in ((B, H, d, m), (B, H, m), (B, H, m, d), (B, H, d))]
    args = (c["xq"], c["xk"], c["xv"], c["W1"], c["b1"], c["W2"], c["b2"], c["token_eta"], c["lr"], c["gamma"],
            c["beta"], d_out, K)
    ref = P.ttt_mlp_backward_raw(*args, d_state_out=dst)
    torch.cuda.synchronize()
    # output tensors allocated up front: the call under test then allocates nothing at all
    into = {k: torch.full_like(v, float("nan")) for k, v in ref.items()}
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    # free device memory as the driver sees it: an allocation made behind torch's back (hipMalloc, a memory pool,
    # a runtime object that takes device memory) would lower it
    free_before = torch.cuda.mem_get_info()[0]
    got = P.ttt_mlp_backward_raw(*args, d_state_out=dst, static_scratch=True, into=into)
    after = torch.cuda.memory_stats()["allocation.all.allocated"]
    torch.cuda.synchronize()
    free_after = torch.cuda.mem_get_info()[0]
    assert after == before, "the static-scratch call allocated device memory through torch"
    assert free_after == free_before, f"free device memory changed by {free_before - free_after} bytes over the static-scratch call"
    return got, ref


def check(got, ref):
    for k in PLAIN:
        assert torch.equal(got[k], ref[k]), f"{k}: differs from ttt_mlp_bwd"
    for k in ATOMIC:
        assert_close(got[k], ref[k].double().cpu().numpy(), 1e-4, k)


def test_static_scratch_matches_workspace_call_twice(P):
    print("case no-alloc: B2 H2 d64 K16 N4 f32, then B1 H2 d32 K8 N2 bf16", flush=True)
    got, ref = both(P, 2, 2, 64, 16, 4, torch.float32, 901, True)
    check(got, ref)
    got, ref = both(P, 1, 2, 32, 8, 2, torch.bfloat16, 902, False)
    check(got, ref)
    # and back to the first shape: the buffer now holds the smaller call's leftovers inside the larger call's extent
    print("case no-alloc: B2 H2 d64 K16 N4 f32 again", flush=True)
    got, ref = both(P, 2, 2, 64, 16, 4, torch.float32, 903, True)
    check(got, ref)


def test_static_scratch_refuses_what_does_not_fit(P):
    print("case no-alloc: oversize refused", flush=True)
    L = P.lib()
    desc = P.TttDesc(8, 16, 2048, 96, 16, 1e-6, 1, P.TTT_BF16, 0, 0, 0)
    assert L.ttt_mlp_bwd_workspace_bytes(C.byref(desc)) > (32 << 20)
    one = torch.zeros(64, device="cuda:0")
    p = C.c_void_p(one.data_ptr())
    rc = L.ttt_mlp_bwd_static(C.byref(desc), *([p] * 12), *([None] * 4), *([p] * 11), None)
    assert rc == P.TTT_ERR_SHAPE
    assert b"ttt_mlp_bwd_static" in L.ttt_last_error() and b"scratch" in L.ttt_last_error()
