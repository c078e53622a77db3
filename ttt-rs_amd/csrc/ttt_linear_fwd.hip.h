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
  const void* xin;  // null, or x [B,H,seq,d] io: the operands are x + xq, x + xk, x + xv (sums rounded to the I/O
                    // type), formed by the kernel; may be the same memory as `out` (a layer of a stack working in place)
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

// What the forward needs beside LinearFwdArgs when it forms its operands from the projections itself
// (ttt_linear_fwd_fi_kernel): the inputs and parameters of ttt_inner_inputs.  In that mode the fields xq, xk, xv, lr
// and token_eta of LinearFwdArgs are not read.
struct FusedInputsArgs {
  const void* xq;  // [B,seq,H,d] io, as the projections leave them
  const void* xk;
  const void* xv;
  const void* lr_logits;             // [B,seq,H] io
  const float* lr_bias;              // [H]
  const float* token_idx;            // [K]
  const float* learnable_token_idx;  // [K]
  const float* cos;                  // [npos, d/2] or null: no rotary embedding
  const float* sin;
  void* xq_out;  // [B,H,seq,d] io: the operands as the kernel used them (what ttt_linear_bwd needs); each may be null
  void* xk_out;
  void* xv_out;
  void* lr_out;          // [B,H,seq] io or null
  float* token_eta_out;  // [seq] or null
  float lr_scale;        // base_lr / d
  int pos_offset, pos_wrap;  // position of token t: (pos_offset + t) [% pos_wrap if > 0]
};

// TTT-Linear with an Adam inner optimiser (reference rust/core/src/linear_adam.rs): the moments of the state and the
// optimiser's constants.  Moments are per (batch, head) unit, f32, in the layout of the state.
struct AdamArgs {
  const float* Wm0;  // [B,H,d,d] first moment entering the call; the four inputs are null together: zero moments
  const float* bm0;  // [B,H,d]
  const float* Wv0;  // second moment
  const float* bv0;
  float* Wm_out;
  float* bm_out;
  float* Wv_out;
  float* bv_out;
  float beta1, beta2, eps, lr;
  int step0;  // Adam steps taken before this call (the reference's state.step)
};

}  // namespace ttt
