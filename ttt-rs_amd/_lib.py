"""ctypes binding of include/ttt_mi355x.h.  Loading fails loudly when the HIP library has not
been built: there is no CPU fallback anywhere in this package."""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libttt_mi355x.so")

TTT_OK, TTT_ERR_SHAPE, TTT_ERR_UNSUPPORTED, TTT_ERR_HIP, TTT_ERR_NULL = 0, -1, -2, -3, -4
TTT_F32, TTT_BF16 = 0, 1
TTT_HINT_AUTO, TTT_HINT_LDS_TILES = 0, 0x100  # kernel_hint: low byte = waves per unit (1, 2, 4)
TTT_HINT_TEST_LOST_PARTNER = 0x200
TTT_HINT_TWO_CU = 0x400
TTT_HINT_OWN_LOADS = 0x1000
TTT_HINT_ALL_LOADS = 0x2000
TTT_HINT_TEST_OTHER_XCD = 0x800
TTT_HINT_F32_PRODUCTS = 0x4000
TTT_HINT_ONE_WORKGROUP = 0x8000

EXPORTS = (
    "ttt_version", "ttt_last_error", "ttt_linear_supported", "ttt_linear_bwd_supported",
    "ttt_linear_best_checkpoint_format",
    "ttt_linear_num_checkpoints",
    "ttt_linear_fwd", "ttt_linear_bwd", "ttt_linear_bwd_workspace_bytes", "ttt_linear_bwd_ws", "ttt_mlp_supported", "ttt_mlp_fwd",
    "ttt_mlp_fwd_lost_workgroups", "ttt_mlp_bwd_workspace_bytes", "ttt_mlp_bwd", "ttt_mlp_bwd_static", "ttt_mlp_fwd_saving_supported", "ttt_mlp_fwd_saving", "ttt_mlp_bwd_saved", "ttt_stack_fwd_workspace_bytes", "ttt_stack_fwd", "ttt_inner_inputs", "ttt_layer_epilogue", "ttt_linear_fwd_fused_inputs_supported", "ttt_linear_fwd_fused_inputs", "ttt_linear_adam_supported", "ttt_linear_adam_fwd", "ttt_mlpn_supported", "ttt_mlpn_fwd", "ttt_selftest_mfma_mixed",
)


class TttDesc(C.Structure):
    _fields_ = [
        ("batch", C.c_int32), ("heads", C.c_int32), ("seq", C.c_int32), ("head_dim", C.c_int32),
        ("mini_batch", C.c_int32), ("eps", C.c_float), ("checkpoint_interval", C.c_int32),
        ("io_dtype", C.c_int32), ("state_per_batch", C.c_int32), ("seq_stride", C.c_int32),
        ("checkpoint_format", C.c_int32), ("kernel_hint", C.c_int32),
    ]


class TttStackLayer(C.Structure):
    """ttt_stack_layer of include/ttt_mi355x.h."""
    _fields_ = [("kind", C.c_int32)] + [(n, C.c_void_p) for n in (
        "pq", "pk", "pv", "W1", "b1", "W2", "b2", "lr", "gamma", "beta", "W1_out", "b1_out", "W2_out", "b2_out")]


class TttError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"ttt status {code}: {msg}")
        self.code = code


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it first (python ttt-rs_amd/build.py); "
                "this package has no fallback path")
        L = C.CDLL(LIB_PATH)
        vp = C.c_void_p
        dp = C.POINTER(TttDesc)
        for name in EXPORTS:
            getattr(L, name).restype = C.c_int
        L.ttt_version.restype = C.c_char_p
        L.ttt_last_error.restype = C.c_char_p
        L.ttt_linear_supported.argtypes = [dp]
        L.ttt_linear_bwd_supported.argtypes = [dp]
        L.ttt_linear_best_checkpoint_format.argtypes = [dp]
        L.ttt_linear_best_checkpoint_format.restype = C.c_int
        L.ttt_linear_num_checkpoints.argtypes = [dp]
        L.ttt_linear_num_checkpoints.restype = C.c_int64
        L.ttt_linear_fwd.argtypes = [dp] + [vp] * 15
        L.ttt_linear_bwd.argtypes = [dp] + [vp] * 24
        L.ttt_linear_bwd_workspace_bytes.argtypes = [dp]
        L.ttt_linear_bwd_workspace_bytes.restype = C.c_int64
        L.ttt_linear_bwd_ws.argtypes = [dp] + [vp] * 25
        L.ttt_mlp_supported.argtypes = [dp]
        L.ttt_mlp_fwd.argtypes = [dp] + [vp] * 17
        L.ttt_mlp_bwd_workspace_bytes.argtypes = [dp]
        L.ttt_mlp_bwd_workspace_bytes.restype = C.c_int64
        L.ttt_mlp_bwd.argtypes = [dp] + [vp] * 29
        L.ttt_mlp_bwd_static.argtypes = [dp] + [vp] * 28
        L.ttt_mlp_fwd_saving_supported.argtypes = [dp]
        L.ttt_mlp_fwd_saving.argtypes = [dp] + [vp] * 18
        L.ttt_mlp_bwd_saved.argtypes = [dp] + [vp] * 29
        L.ttt_mlp_fwd_lost_workgroups.argtypes = [C.POINTER(C.c_int64)]
        L.ttt_stack_fwd_workspace_bytes.argtypes = [dp, C.c_int32, C.POINTER(TttStackLayer), C.c_int32]
        L.ttt_stack_fwd_workspace_bytes.restype = C.c_int64
        L.ttt_stack_fwd.argtypes = [dp, C.c_int32, C.POINTER(TttStackLayer), vp, vp, vp, C.c_int32, vp, vp]
        L.ttt_inner_inputs.argtypes = [dp] + [vp] * 5 + [C.c_float] + [vp] * 4 + [C.c_int, C.c_int] + [vp] * 6
        L.ttt_layer_epilogue.argtypes = [dp] + [vp] * 3 + [C.c_float] + [vp] * 3
        L.ttt_mlpn_supported.argtypes = [dp, C.c_int]
        L.ttt_mlpn_fwd.argtypes = [dp, C.c_int] + [vp] * 13
        L.ttt_linear_adam_supported.argtypes = [dp]
        L.ttt_linear_adam_fwd.argtypes = [dp] + [vp] * 9 + [C.c_int] + [C.c_float] * 4 + [vp] * 12
        L.ttt_linear_fwd_fused_inputs_supported.argtypes = [dp, C.c_int, C.c_int]
        L.ttt_linear_fwd_fused_inputs.argtypes = ([dp] + [vp] * 5 + [C.c_float] + [vp] * 4 + [C.c_int, C.c_int] +
                                                  [vp] * 15)
        L.ttt_selftest_mfma_mixed.argtypes = [C.c_int, C.c_int, vp, vp]
        _lib = L
    return _lib


def check(rc: int):
    if rc != TTT_OK:
        raise TttError(rc, lib().ttt_last_error().decode())
