// C++ host-side mirror of the reference's TTT-MLP inner model above the C ABI of
// include/ttt_mi355x.h.  Names and argument meaning follow the reference:
//   TTTMLP / TTTMLPState           rust/core/src/mlp.rs:29-53
//   TTTMLP::init_state             rust/core/src/mlp.rs:119-125 ([H,..] parameters broadcast over batch)
//   TTTInnerModel::forward         rust/core/src/inner.rs:25-50 (full mini-batches, then the remainder)
//   TTTMLP::forward_mini_batch     rust/core/src/mlp.rs:127-208
// The reference has no fused MLP kernel; its backward is Burn autodiff over those ops, which
// FusedMlp::backward replaces (one call, no saved state besides the inputs).
// Ownership as in fused_tile_multi.hpp: caller-owned device buffers, nothing here allocates.
#pragma once

#include "fused_tile_multi.hpp"

namespace ttt {

/// mlp.rs:43-53: w1 [B,H,d,4d], b1 [B,H,4d], w2 [B,H,4d,d], b2 [B,H,d], f32.  Two sets of caller-owned buffers,
/// all eight always valid: a forward call reads the current set and writes `next_*`, then swap() makes those
/// current.  `initialised == false`: the current set holds no state yet and the first launch reads the layer's
/// [H,..] parameters instead (init_state without the copy), then sets the flag.
struct TTTMLPState {
  float* w1 = nullptr;
  float* b1 = nullptr;
  float* w2 = nullptr;
  float* b2 = nullptr;
  float* next_w1 = nullptr;
  float* next_b1 = nullptr;
  float* next_w2 = nullptr;
  float* next_b2 = nullptr;
  bool initialised = false;
  void swap() {
    float* t;
    t = w1; w1 = next_w1; next_w1 = t;
    t = b1; b1 = next_b1; next_b1 = t;
    t = w2; w2 = next_w2; next_w2 = t;
    t = b2; b2 = next_b2; next_b2 = t;
  }
};

/// Gradients w.r.t. the eleven inputs of the MLP inner loop.
struct TTTMLPGrads {
  void* grad_xq = nullptr;
  void* grad_xk = nullptr;
  void* grad_xv = nullptr;
  float* grad_w1 = nullptr;         // [B,H,d,4d] per batch element
  float* grad_b1 = nullptr;         // [B,H,4d]
  float* grad_w2 = nullptr;         // [B,H,4d,d]
  float* grad_b2 = nullptr;         // [B,H,d]
  void* grad_ttt_lr_eta = nullptr;  // [B,H,seq]
  float* grad_token_eta = nullptr;  // [seq], per position
  float* grad_ln_weight = nullptr;  // [H,d]
  float* grad_ln_bias = nullptr;    // [H,d]
};

/// Fused TTT-MLP inner model on MI355X (mlp_expansion_factor 4, mlp.rs:79).
class FusedMlp {
 public:
  /// Parameters as TTTMLP holds them (mlp.rs:29-41), device pointers, f32:
  /// w1_init [H,d,4d], b1_init [H,4d], w2_init [H,4d,d], b2_init [H,d], LayerNorm weight/bias [H,d].
  FusedMlp(const ModelConfig& config, const float* w1_init, const float* b1_init, const float* w2_init,
           const float* b2_init, const float* ln_weight, const float* ln_bias)
      : config_(config), w1_(w1_init), b1_(b1_init), w2_(w2_init), b2_(b2_init), ln_weight_(ln_weight),
        ln_bias_(ln_bias) {}

  static const char* name() { return "FusedTTTMLP"; }
  const ModelConfig& get_config() const { return config_; }

  ttt_desc desc(int batch, int seq, int mini_batch, ttt_dtype dtype, bool state_per_batch) const {
    ttt_desc d{};
    d.batch = batch;
    d.heads = config_.num_heads;
    d.seq = seq;
    d.head_dim = config_.head_dim;
    d.mini_batch = mini_batch;
    d.eps = config_.ttt.epsilon;
    d.checkpoint_interval = 1;
    d.io_dtype = dtype;
    d.state_per_batch = state_per_batch ? 1 : 0;
    d.seq_stride = 0;
    d.checkpoint_format = TTT_CKPT_F32;
    d.kernel_hint = config_.ttt.kernel_hint;
    return d;
  }

  /// inner.rs:25-50: all full mini-batches in one launch, then a trailing remainder as one short
  /// mini-batch, as in-place windows of the [B,H,seq,d] tensors.  A state that is not initialised yet
  /// makes the first launch read the [H,..] parameters directly (see TTTMLPState).
  void forward(TTTMLPState& state, const TTTInputsInner& in, void* out, void* stream) const {
    const int K = config_.ttt.mini_batch_size;
    const int full = (in.seq_len / K) * K;
    if (full > 0) launch(state, in, 0, full, K, out, stream);
    if (full < in.seq_len) launch(state, in, full, in.seq_len - full, in.seq_len - full, out, stream);
  }

  /// mlp.rs:127-208: the mini-batch [first, first+len), len <= mini_batch_size.
  void forward_mini_batch(TTTMLPState& state, const TTTInputsInner& in, int first, int len, void* out,
                          void* stream) const {
    if (len <= 0 || len > config_.ttt.mini_batch_size || first < 0 || first + len > in.seq_len)
      throw Error(TTT_ERR_SHAPE, "range must be non-empty, inside the sequence and at most mini_batch_size long");
    launch(state, in, first, len, len, out, stream);
  }

  /// Bytes of device workspace backward() needs for this batch and sequence length.
  std::int64_t backward_workspace_bytes(int batch, int seq, ttt_dtype dtype) const {
    ttt_desc d = desc(batch, seq, config_.ttt.mini_batch_size, dtype, false);
    return ttt_mlp_bwd_workspace_bytes(&d);
  }

  /// Gradients of the whole sequence (seq a multiple of mini_batch_size) from the initial state
  /// (state0 not initialised: the [H,..] parameters), grad_output [B,H,seq,d] and optional upstream gradients
  /// of the final state (all four or none).
  void backward(const TTTInputsInner& in, const TTTMLPState& state0, const void* grad_output,
                const float* grad_w1_out, const float* grad_b1_out, const float* grad_w2_out,
                const float* grad_b2_out, const TTTMLPGrads& g, void* workspace, void* stream) const {
    const bool per_batch = state0.initialised;
    ttt_desc d = desc(in.batch, in.seq_len, config_.ttt.mini_batch_size, in.dtype, per_batch);
    check(ttt_mlp_bwd(&d, in.qkv.xq, in.qkv.xk, in.qkv.xv, per_batch ? state0.w1 : w1_,
                      per_batch ? state0.b1 : b1_, per_batch ? state0.w2 : w2_, per_batch ? state0.b2 : b2_,
                      in.token_eta, in.ttt_lr_eta, ln_weight_, ln_bias_, grad_output, grad_w1_out, grad_b1_out,
                      grad_w2_out, grad_b2_out, g.grad_xq, g.grad_xk, g.grad_xv, g.grad_w1, g.grad_b1,
                      g.grad_w2, g.grad_b2, g.grad_ttt_lr_eta, g.grad_token_eta, g.grad_ln_weight,
                      g.grad_ln_bias, workspace, stream));
  }

  /// forward over a sequence of whole mini-batches that also saves, in `saved` (backward_workspace_bytes of device
  /// memory), what backward_saved needs: the training pair ttt_mlp_fwd_saving / ttt_mlp_bwd_saved, i.e. a backward
  /// without a forward sweep of its own.  Throws TTT_ERR_UNSUPPORTED where the forward runs on pairs of CUs
  /// (head_dim 128 with bf16 I/O): use forward + backward there.
  void forward_saving(TTTMLPState& state, const TTTInputsInner& in, void* out, void* saved, void* stream) const {
    if (in.seq_len % config_.ttt.mini_batch_size != 0)
      throw Error(TTT_ERR_SHAPE, "forward_saving: the sequence must be whole mini-batches");
    if (!state.next_w1 || !state.next_b1 || !state.next_w2 || !state.next_b2)
      throw Error(TTT_ERR_NULL, "TTTMLPState: both sets of state buffers must be valid");
    const bool per_batch = state.initialised;
    ttt_desc d = desc(in.batch, in.seq_len, config_.ttt.mini_batch_size, in.dtype, per_batch);
    check(ttt_mlp_fwd_saving(&d, in.qkv.xq, in.qkv.xk, in.qkv.xv, per_batch ? state.w1 : w1_,
                             per_batch ? state.b1 : b1_, per_batch ? state.w2 : w2_, per_batch ? state.b2 : b2_,
                             in.token_eta, in.ttt_lr_eta, ln_weight_, ln_bias_, out, state.next_w1, state.next_b1,
                             state.next_w2, state.next_b2, saved, stream));
    state.swap();
    state.initialised = true;
  }

  /// backward with the arguments of backward(), `saved` (written by forward_saving on the same inputs and state0) in
  /// place of the workspace; consumes `saved`.
  void backward_saved(const TTTInputsInner& in, const TTTMLPState& state0, const void* grad_output,
                      const float* grad_w1_out, const float* grad_b1_out, const float* grad_w2_out,
                      const float* grad_b2_out, const TTTMLPGrads& g, void* saved, void* stream) const {
    const bool per_batch = state0.initialised;
    ttt_desc d = desc(in.batch, in.seq_len, config_.ttt.mini_batch_size, in.dtype, per_batch);
    check(ttt_mlp_bwd_saved(&d, in.qkv.xq, in.qkv.xk, in.qkv.xv, per_batch ? state0.w1 : w1_,
                            per_batch ? state0.b1 : b1_, per_batch ? state0.w2 : w2_, per_batch ? state0.b2 : b2_,
                            in.token_eta, in.ttt_lr_eta, ln_weight_, ln_bias_, grad_output, grad_w1_out, grad_b1_out,
                            grad_w2_out, grad_b2_out, g.grad_xq, g.grad_xk, g.grad_xv, g.grad_w1, g.grad_b1,
                            g.grad_w2, g.grad_b2, g.grad_ttt_lr_eta, g.grad_token_eta, g.grad_ln_weight,
                            g.grad_ln_bias, saved, stream));
  }

 private:
  static const void* at(const void* p, std::size_t bytes) {
    return p ? static_cast<const char*>(p) + bytes : nullptr;
  }
  void launch(TTTMLPState& state, const TTTInputsInner& in, int first, int seq, int mini_batch, void* out,
              void* stream) const {
    if (!state.w1 || !state.b1 || !state.w2 || !state.b2 || !state.next_w1 || !state.next_b1 || !state.next_w2 ||
        !state.next_b2)
      throw Error(TTT_ERR_NULL, "TTTMLPState: both sets of state buffers must be valid");
    const bool per_batch = state.initialised;
    const std::size_t es = in.dtype == TTT_BF16 ? 2 : 4;
    const std::size_t row = (std::size_t)first * (std::size_t)config_.head_dim * es;
    ttt_desc d = desc(in.batch, seq, mini_batch, in.dtype, per_batch);
    d.seq_stride = in.seq_len;
    check(ttt_mlp_fwd(&d, at(in.qkv.xq, row), at(in.qkv.xk, row), at(in.qkv.xv, row),
                      per_batch ? state.w1 : w1_, per_batch ? state.b1 : b1_, per_batch ? state.w2 : w2_,
                      per_batch ? state.b2 : b2_, in.token_eta ? in.token_eta + first : nullptr,
                      at(in.ttt_lr_eta, (std::size_t)first * es), ln_weight_, ln_bias_,
                      const_cast<void*>(at(out, row)), state.next_w1, state.next_b1, state.next_w2,
                      state.next_b2, stream));
    state.swap();
    state.initialised = true;
  }

  ModelConfig config_;
  const float* w1_;
  const float* b1_;
  const float* w2_;
  const float* b2_;
  const float* ln_weight_;
  const float* ln_bias_;
};

/// The status word of the two-CU TTT-MLP forward (head_dim 128, bf16 I/O; see ttt_mlp_fwd in the C header): a
/// workgroup that waited for its partner in vain cannot fail the call that enqueued it, so a caller that runs such
/// layers -- directly or inside ttt_stack_fwd -- brackets its work with this guard: construct it before enqueueing,
/// call verify() once the stream's work has finished (both read the word with a blocking copy from the device).
class LostWorkgroupGuard {
 public:
  LostWorkgroupGuard() { check(ttt_mlp_fwd_lost_workgroups(&before_)); }
  /// Throws if the word moved since construction: the outputs of the affected units are NaN.
  void verify() const {
    std::int64_t now = 0;
    check(ttt_mlp_fwd_lost_workgroups(&now));
    if (now != before_)
      throw Error(TTT_ERR_HIP, std::to_string(now - before_) +
                                   " workgroups of the two-CU TTT-MLP kernel waited for their partner in vain");
  }

 private:
  std::int64_t before_ = 0;
};

/// ttt_stack_fwd (inner models applied layer by layer, optionally as a cross-layer wavefront over windows of
/// chunk_tokens tokens with the TTT-MLP launches on aux_stream) with the arguments of the C entry point.  Enqueues
/// only; a caller whose stack holds TTT-MLP layers at head_dim 128 keeps a LostWorkgroupGuard around the call and
/// verifies it after synchronising.
inline void stack_forward(const ttt_desc& desc, int n_layers, const ttt_stack_layer* layers, const float* token_eta,
                          void* out, void* workspace, int chunk_tokens, void* aux_stream, void* stream) {
  check(ttt_stack_fwd(&desc, n_layers, layers, token_eta, out, workspace, chunk_tokens, aux_stream, stream));
}

}  // namespace ttt
