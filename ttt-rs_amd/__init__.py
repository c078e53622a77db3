"""MI355X-native fused TTT inner loop (TTT-Linear / TTT-MLP mini-batch dual form).

Host-side mirror of the reference's inner-model surface (rust/core/src/inner.rs:13-58,
rust/fused/src/linear_fused_tile/wrapper.rs:81-211) over the C ABI in include/ttt_mi355x.h.
torch is used only to hold device memory and streams.
"""
from ._lib import (TTT_BF16, TTT_ERR_HIP, TTT_ERR_NULL, TTT_ERR_SHAPE, TTT_ERR_UNSUPPORTED,
                   TTT_F32, TTT_OK, TTT_HINT_AUTO, TTT_HINT_LDS_TILES, TTT_HINT_TEST_LOST_PARTNER, TTT_HINT_TWO_CU, TTT_HINT_OWN_LOADS, TTT_HINT_ALL_LOADS, TTT_HINT_TEST_OTHER_XCD, TTT_HINT_F32_PRODUCTS, TTT_HINT_ONE_WORKGROUP, EXPORTS, LIB_PATH, TttDesc, TttError, TttStackLayer, check, lib)
from .inner import (FusedMlp, FusedTileMulti, TTTMLPState, ttt_mlp_forward_raw, ttt_mlp_backward_raw, ModelConfig, Qkv, TTTConfig, TTTInputsInner, TTTLinearState,
                    ttt_linear_backward_raw, ttt_linear_forward_raw, inner_loop_inputs_raw, layer_epilogue_raw, ttt_linear_forward_fused_inputs_raw, ttt_linear_adam_forward_raw, ttt_mlpn_forward_raw, FusedLinearAdam, TTTLinearAdamConfig, TTTLinearAdamState, FusedMlpN, TTTMLPNState,
                    rope_cos_sin, ttt_lr_eta_logit_grad, ttt_stack_forward_raw, mlp_fwd_lost_workgroups,
                    ttt_stack_workspace_bytes)
from . import synthetic

__all__ = [
    "FusedTileMulti", "FusedMlp", "TTTMLPState", "ttt_mlp_forward_raw", "ttt_mlp_backward_raw", "ModelConfig", "Qkv", "TTTConfig", "TTTInputsInner", "TTTLinearState",
    "ttt_linear_forward_raw", "ttt_linear_backward_raw", "inner_loop_inputs_raw", "layer_epilogue_raw", "ttt_linear_forward_fused_inputs_raw", "ttt_linear_adam_forward_raw", "ttt_mlpn_forward_raw", "FusedLinearAdam", "TTTLinearAdamConfig", "TTTLinearAdamState", "FusedMlpN", "TTTMLPNState", "rope_cos_sin", "ttt_lr_eta_logit_grad", "ttt_stack_forward_raw", "ttt_stack_workspace_bytes", "mlp_fwd_lost_workgroups",
    "synthetic", "lib", "TttDesc", "TttError", "TttStackLayer", "check", "LIB_PATH", "EXPORTS",
    "TTT_OK", "TTT_ERR_SHAPE", "TTT_ERR_UNSUPPORTED", "TTT_ERR_HIP", "TTT_ERR_NULL",
    "TTT_F32", "TTT_BF16", "TTT_HINT_AUTO", "TTT_HINT_LDS_TILES", "TTT_HINT_TEST_LOST_PARTNER", "TTT_HINT_TWO_CU", "TTT_HINT_OWN_LOADS", "TTT_HINT_ALL_LOADS", "TTT_HINT_TEST_OTHER_XCD", "TTT_HINT_F32_PRODUCTS", "TTT_HINT_ONE_WORKGROUP",
]
