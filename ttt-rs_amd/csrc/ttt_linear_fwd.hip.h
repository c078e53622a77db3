// Argument block shared by the TTT-Linear forward kernels (register-resident workgroup kernels in
// ttt_linear_fwd_mw.hip.h / ttt_linear_fwd_sk.hip.h, LDS-resident kernel in ttt_engine_fwd.hip.h).
// Field meaning follows ttt_linear_fwd in include/ttt_mi355x.h.
#pragma once
#include "ttt_frag.hip.h"

namespace ttt {

constexpr int kCkptFactors = 2;  // value of ckpt_packed for TTT_CKPT_FACTORS

struct LinearFwdArgs {
  const void* xq;
  const void* xk;
  const void* xv;
  const float* W0;
  const float* b0;
  const float* token_eta;
  const void* lr;
  const float* gamma;
  const float* beta;
  void* out;
  float* W_out;
  float* b_out;
  float* W_ckpt;
  float* b_ckpt;
  int B, H, seq, seq_stride, K, n_stages, ckpt_interval, n_ckpt, state_per_batch;
  int ckpt_packed;  // 1: W checkpoints as bf16 operand fragments (see store_ckpt_packed); kCkptFactors: update
                    // factors and the final state instead of states (see store_factor)
  float eps;
};

}  // namespace ttt
