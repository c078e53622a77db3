"""CPU-side checks of the C ABI: the library loads, exports every declared symbol, and argument
validation answers without touching a GPU."""
import ctypes as C
import importlib
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def P():
    return importlib.import_module("ttt-rs_amd")


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "ttt_mi355x.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ttt_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(P):
    L = C.CDLL(P.LIB_PATH)
    syms = declared_symbols()
    assert set(syms) == set(P.EXPORTS)
    for s in syms:
        assert getattr(L, s) is not None


def test_version_and_error_strings(P):
    assert b"gfx950" in P.lib().ttt_version()


def desc(P, **kw):
    base = dict(batch=2, heads=2, seq=32, head_dim=64, mini_batch=16, eps=1e-6,
                checkpoint_interval=1, io_dtype=P.TTT_F32, state_per_batch=0)
    base.update(kw)
    return P.TttDesc(**base)


def test_shape_validation(P):
    L = P.lib()
    assert L.ttt_linear_supported(C.byref(desc(P))) == P.TTT_OK
    # seq must be a multiple of mini_batch (forward/launch.rs:209-213 asserts the same)
    assert L.ttt_linear_supported(C.byref(desc(P, seq=33))) == P.TTT_ERR_SHAPE
    assert b"multiple" in L.ttt_last_error()
    assert L.ttt_linear_supported(C.byref(desc(P, head_dim=48))) == P.TTT_ERR_UNSUPPORTED
    # mini-batches beyond 16 tokens: up to 32 at head_dim 32, as the reference's tile table
    # (rust/fused/src/linear_fused_tile/mod.rs:31-38: (8,32) (8,64) (16,32) (16,64) (32,32))
    assert L.ttt_linear_supported(C.byref(desc(P, mini_batch=32, seq=64))) == P.TTT_ERR_UNSUPPORTED   # head_dim 64
    assert b"head_dim 32" in L.ttt_last_error()
    for K, d, want in ((8, 32, P.TTT_OK), (8, 64, P.TTT_OK), (16, 32, P.TTT_OK), (16, 64, P.TTT_OK),
                       (32, 32, P.TTT_OK), (24, 32, P.TTT_OK), (33, 32, P.TTT_ERR_UNSUPPORTED),
                       (32, 96, P.TTT_ERR_UNSUPPORTED)):
        assert L.ttt_linear_supported(C.byref(desc(P, mini_batch=K, head_dim=d, seq=4 * K))) == want, (K, d)
    big = lambda **kw: desc(P, mini_batch=32, head_dim=32, seq=128, **kw)
    assert L.ttt_linear_bwd_supported(C.byref(big())) == P.TTT_OK
    assert L.ttt_linear_bwd_supported(C.byref(big(checkpoint_interval=2, io_dtype=P.TTT_BF16))) == P.TTT_OK
    assert L.ttt_linear_bwd_supported(C.byref(big(checkpoint_format=1))) == P.TTT_ERR_UNSUPPORTED
    assert L.ttt_linear_bwd_supported(C.byref(big(checkpoint_format=2, io_dtype=P.TTT_BF16))) == P.TTT_ERR_UNSUPPORTED
    assert L.ttt_linear_best_checkpoint_format(C.byref(big(io_dtype=P.TTT_BF16))) == 0
    assert L.ttt_mlp_supported(C.byref(big())) == P.TTT_ERR_UNSUPPORTED
    assert L.ttt_linear_adam_supported(C.byref(big())) == P.TTT_ERR_UNSUPPORTED
    assert L.ttt_linear_fwd_fused_inputs_supported(C.byref(big(io_dtype=P.TTT_BF16)), 0, 0) == P.TTT_ERR_UNSUPPORTED
    assert L.ttt_linear_supported(C.byref(desc(P, checkpoint_interval=0))) == P.TTT_ERR_SHAPE
    assert L.ttt_linear_supported(C.byref(desc(P, io_dtype=7))) == P.TTT_ERR_UNSUPPORTED
    assert L.ttt_linear_supported(None) == P.TTT_ERR_NULL
    # checkpoint formats: 0 (f32 row-major), 1 (packed) and 2 (update factors) exist
    assert L.ttt_linear_supported(C.byref(desc(P, checkpoint_format=1))) == P.TTT_OK
    assert L.ttt_linear_supported(C.byref(desc(P, checkpoint_format=2))) == P.TTT_OK
    assert L.ttt_linear_supported(C.byref(desc(P, checkpoint_format=3))) == P.TTT_ERR_SHAPE
    assert b"checkpoint_format" in L.ttt_last_error()


def test_best_checkpoint_format(P):
    L = P.lib()
    best = lambda **kw: L.ttt_linear_best_checkpoint_format(C.byref(desc(P, **kw)))
    assert best(io_dtype=P.TTT_BF16) == 2                            # update factors
    assert best(io_dtype=P.TTT_BF16, head_dim=96) == 2
    assert best(io_dtype=P.TTT_BF16, checkpoint_format=0) == 2       # the desc's own format field is not read
    assert best(io_dtype=P.TTT_BF16, head_dim=128) == 1              # packed states
    assert best(io_dtype=P.TTT_BF16, seq=16) == 1                    # one mini-batch
    assert best(io_dtype=P.TTT_BF16, batch=64, heads=12) == 1        # more than 512 units: single-wave backward
    assert best(io_dtype=P.TTT_F32) == 1
    assert best(checkpoint_interval=2) == 0 and best(io_dtype=P.TTT_BF16, checkpoint_interval=4) == 0
    assert best(seq=33) < 0
    # the hint is part of the question: the LDS-tile backward reads f32 matrices only
    assert best(io_dtype=P.TTT_BF16, kernel_hint=P.TTT_HINT_LDS_TILES) == 0
    assert best(io_dtype=P.TTT_F32, kernel_hint=P.TTT_HINT_LDS_TILES) == 0
    # f32 I/O at head_dim 128: the LDS-tile backward that reads the row-major checkpoints in place
    assert best(io_dtype=P.TTT_F32, head_dim=128) == 0
    assert best(head_dim=96, checkpoint_interval=2) == 0
    # no backward kernel at all: the backward's status, no format
    assert best(head_dim=128, checkpoint_interval=2) == P.TTT_ERR_UNSUPPORTED
    assert best(head_dim=48) == P.TTT_ERR_UNSUPPORTED
    # what it names is accepted by the backward
    for kw in (dict(io_dtype=P.TTT_BF16), dict(io_dtype=P.TTT_F32), dict(io_dtype=P.TTT_BF16, head_dim=128),
               dict(checkpoint_interval=2), dict(io_dtype=P.TTT_BF16, kernel_hint=P.TTT_HINT_LDS_TILES)):
        fmt = best(**kw)
        assert L.ttt_linear_bwd_supported(C.byref(desc(P, checkpoint_format=fmt, **kw))) == P.TTT_OK


def test_num_checkpoints(P):
    L = P.lib()
    assert L.ttt_linear_num_checkpoints(C.byref(desc(P, seq=16 * 9, checkpoint_interval=4))) == 3
    assert L.ttt_linear_num_checkpoints(C.byref(desc(P, seq=16 * 8, checkpoint_interval=1))) == 8


def test_backward_support_query_and_kernel_hints(P):
    """ttt_linear_bwd_supported answers what ttt_linear_bwd would (fewer combinations than the forward), and
    desc.kernel_hint is part of the descriptor: the library reads no environment variable."""
    L = P.lib()
    ok = lambda **kw: L.ttt_linear_bwd_supported(C.byref(desc(P, **kw)))
    assert ok() == P.TTT_OK
    assert ok(head_dim=128, io_dtype=P.TTT_BF16) == P.TTT_OK
    assert ok(head_dim=128, io_dtype=P.TTT_F32) == P.TTT_OK
    assert ok(head_dim=128, io_dtype=P.TTT_F32, checkpoint_format=1) == P.TTT_ERR_UNSUPPORTED
    assert L.ttt_linear_supported(C.byref(desc(P, head_dim=128))) == P.TTT_OK
    assert ok(head_dim=96, checkpoint_interval=2) == P.TTT_OK
    assert ok(head_dim=128, checkpoint_interval=2) == P.TTT_ERR_UNSUPPORTED
    assert b"checkpoint_interval 1" in L.ttt_last_error()
    assert ok(head_dim=64, checkpoint_interval=2) == P.TTT_OK
    assert ok(checkpoint_format=1, checkpoint_interval=2) == P.TTT_ERR_UNSUPPORTED
    # packed checkpoints exist for the register-resident kernels only
    assert ok(checkpoint_format=1, kernel_hint=P.TTT_HINT_LDS_TILES) == P.TTT_ERR_UNSUPPORTED
    # update factors: bf16 I/O, a checkpoint per mini-batch, head_dim <= 96, the register-resident kernels
    fac = lambda **kw: ok(checkpoint_format=2, **{"io_dtype": P.TTT_BF16, **kw})
    assert fac() == P.TTT_OK and fac(head_dim=96) == P.TTT_OK and fac(seq=16) == P.TTT_OK
    for bad in (dict(io_dtype=P.TTT_F32), dict(head_dim=128), dict(checkpoint_interval=2),
                dict(kernel_hint=P.TTT_HINT_LDS_TILES)):
        assert fac(**bad) == P.TTT_ERR_UNSUPPORTED, bad
        assert b"update-factor checkpoints" in L.ttt_last_error()
    assert ok(kernel_hint=P.TTT_HINT_LDS_TILES) == P.TTT_OK
    assert ok(kernel_hint=4) == P.TTT_OK and ok(kernel_hint=1, io_dtype=P.TTT_BF16) == P.TTT_OK
    # a hint that names no kernel for the desc is ignored (no LDS-tile backward at head_dim 96)
    assert ok(head_dim=96, kernel_hint=P.TTT_HINT_LDS_TILES) == P.TTT_OK
    assert ok(seq=33) == P.TTT_ERR_SHAPE
    # the struct the binding declares is the struct the header declares (field order and count)
    text = open(os.path.join(ROOT, "include", "ttt_mi355x.h")).read()
    body = re.sub(r"/\*.*?\*/", "", text[text.index("typedef struct ttt_desc {"):text.index("} ttt_desc;")], flags=re.S)
    fields = re.findall(r"\b(?:int32_t|float)\s+(\w+)\s*;", body)
    assert fields == [f[0] for f in P.TttDesc._fields_]
    src = open(os.path.join(ROOT, "ttt-rs_amd", "csrc", "ttt_api.hip")).read()
    assert "getenv" not in src


def test_null_pointers_are_rejected_before_any_launch(P):
    L = P.lib()
    rc = L.ttt_linear_fwd(C.byref(desc(P)), *([None] * 15))
    assert rc == P.TTT_ERR_NULL


def test_stack_plan_is_validated_without_a_gpu(P):
    """ttt_stack_fwd_workspace_bytes / ttt_stack_fwd check the plan (layer kinds, window length, pointers) before any
    HIP call: wrong plans answer with an error code here, on a machine without a GPU."""
    L = P.lib()
    d = desc(P, batch=1, heads=2, seq=64, head_dim=64, io_dtype=P.TTT_BF16)
    layers = (P.TttStackLayer * 2)()
    layers[0].kind, layers[1].kind = 0, 1
    U, D, M, seq = 2, 64, 256, 64
    tensor = (U * seq * D * 2 + 255) // 256 * 256
    assert L.ttt_stack_fwd_workspace_bytes(C.byref(d), 2, layers, 0) == 3 * tensor
    # with windows: one spare copy of every layer's state as well
    up = lambda n: (n + 255) // 256 * 256
    spare = up(U * (D * D + D) * 4) + up(U * (2 * D * M + M + D) * 4)
    assert L.ttt_stack_fwd_workspace_bytes(C.byref(d), 2, layers, 32) == 3 * tensor + spare
    for bad in (24, 48, 128, -16):      # not a multiple of mini_batch; not a divisor of seq; longer than seq; negative
        assert L.ttt_stack_fwd_workspace_bytes(C.byref(d), 2, layers, bad) == -1
        assert b"chunk_tokens" in L.ttt_last_error()
    layers[1].kind = 7
    assert L.ttt_stack_fwd_workspace_bytes(C.byref(d), 2, layers, 0) == -1
    layers[1].kind = 1
    assert L.ttt_stack_fwd_workspace_bytes(C.byref(d), 0, layers, 0) == -1
    # NULL token_eta / out / workspace, then NULL layer tensors: refused before anything is enqueued
    assert L.ttt_stack_fwd(C.byref(d), 2, layers, None, None, None, 0, None, None) == P.TTT_ERR_NULL
    dummy = C.create_string_buffer(64)
    ptr = C.c_void_p((C.addressof(dummy) + 15) // 16 * 16)
    assert L.ttt_stack_fwd(C.byref(d), 2, layers, ptr, ptr, ptr, 0, None, None) == P.TTT_ERR_NULL
    assert b"layer 0" in L.ttt_last_error()
    # the second stream must be a different one
    assert L.ttt_stack_fwd(C.byref(d), 2, layers, ptr, ptr, ptr, 32, ptr, ptr) == P.TTT_ERR_SHAPE


def test_eta_logit_gradient_helper_matches_the_oracle_chain(P):
    """Host logic, no GPU: the chain from grad_ttt_lr_eta to the lr-gate logits (rust/layer/src/ttt.rs:205-227)."""
    import numpy as np
    import torch
    from oracle import ttt_oracle as orc
    g = torch.Generator().manual_seed(3)
    d_lr, z = torch.randn(2, 3, 32, generator=g), torch.randn(2, 3, 32, generator=g)
    got = P.ttt_lr_eta_logit_grad(d_lr, z, 1.5, 64).double().numpy()
    ref = orc.lr_logit_grad(d_lr.double().numpy(), z.double().numpy(), 1.5, 64)
    assert np.abs(got - ref).max() <= 1e-6 * np.abs(ref).max()
