// C++ host-side mirror of the reference's inner-model interface for the fused TTT-Linear layer,
// above the C ABI of include/ttt_mi355x.h (the reference's host code is Rust; this is the
// compiled-language counterpart a C++ caller links against).
//
// Names and argument meaning follow the reference:
//   trait TTTInnerModel            rust/core/src/inner.rs:13-58  (name / init_state / forward /
//                                  forward_mini_batch)
//   TTTInputsInner, Qkv            rust/core/src/inner.rs:60-119
//   TTTLinear / TTTLinearState     rust/core/src/linear.rs:17-33
//   Fused<B, TTTLinear, TileMultiKernel>  rust/fused/src/linear_fused_tile/wrapper.rs:81-211
//   backward bundle                rust/fused/src/linear_fused_tile/backward/launch.rs:332-438
//
// Ownership follows the C ABI: every tensor is a caller-owned device buffer described by a raw
// pointer; nothing here allocates, frees or synchronises.  Errors are the library's status codes,
// carried by ttt::Error (thrown on the C++ side of the boundary only).
#pragma once

#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>

#include "../../include/ttt_mi355x.h"

namespace ttt {

struct Error : std::runtime_error {
  int code;
  Error(int c, const std::string& what) : std::runtime_error(what), code(c) {}
};

inline void check(int rc) {
  if (rc != TTT_OK) throw Error(rc, ttt_last_error());
}

/// Subset of TTTConfig (rust/config/src/train.rs:11-141) the inner loop reads.
struct TTTConfig {
  int mini_batch_size = 16;
  float base_lr = 1.0f;
  float epsilon = 1e-6f;
  int checkpoint_interval = 1;
  /// ttt_desc.checkpoint_format: TTT_CKPT_F32 (what the reference saves), TTT_CKPT_PACKED (states as operand
  /// fragments in kernel order: interval 1 only, same gradients, less traffic) or TTT_CKPT_FACTORS (bf16 I/O,
  /// interval 1, head_dim <= 96: the update factors and the final state, least traffic).  No counterpart in
  /// the reference's config.
  int checkpoint_format = TTT_CKPT_F32;
  /// ttt_desc.kernel_hint (TTT_HINT_AUTO: the library chooses the kernels).
  int kernel_hint = TTT_HINT_AUTO;
};

struct ModelConfig {
  int num_heads = 0;
  int head_dim = 0;
  TTTConfig ttt;
};

/// [batch, heads, seq, head_dim] each, in the activation dtype (inner.rs:60-68).
struct Qkv {
  const void* xq = nullptr;
  const void* xk = nullptr;
  const void* xv = nullptr;
};

/// inner.rs:107-119.  token_eta: [seq] f32 (K-periodic; the kernel reads the first
/// mini_batch_size entries); ttt_lr_eta: [batch, heads, seq] in the activation dtype.
struct TTTInputsInner {
  Qkv qkv;
  const float* token_eta = nullptr;
  const void* ttt_lr_eta = nullptr;
  int batch = 0;
  int seq_len = 0;
  ttt_dtype dtype = TTT_F32;
  std::size_t start_idx = 0;
};

/// linear.rs:27-33: weight [B,H,d,d], bias [B,H,d], f32.  The library never writes a state in place, so a
/// state is TWO pairs of caller-owned buffers, all four always valid: a forward call reads weight/bias and
/// writes next_weight/next_bias, then swap() makes those current.  `initialised == false` means that
/// weight/bias do not hold a state yet: the first launch then reads the layer's parameters directly
/// ([H,..] broadcast over the batch: init_state of linear.rs:84-89 without the copy) and sets the flag.
struct TTTLinearState {
  float* weight = nullptr;
  float* bias = nullptr;
  float* next_weight = nullptr;
  float* next_bias = nullptr;
  bool initialised = false;
  void swap() {
    float* w = weight; weight = next_weight; next_weight = w;
    float* b = bias; bias = next_bias; next_bias = b;
  }
};

/// Optional checkpoint buffers written by forward for a later backward
/// ([B,H,C,d,d] and [B,H,C,d] f32, C = FusedTileMulti::num_checkpoints).
struct Checkpoints {
  float* weight = nullptr;
  float* bias = nullptr;
};

/// Gradients w.r.t. the nine kernel inputs (TttGradInputs, backward/launch.rs:427-437).
struct TTTLinearGrads {
  void* grad_xq = nullptr;
  void* grad_xk = nullptr;
  void* grad_xv = nullptr;
  float* grad_weight = nullptr;     // [B,H,d,d] per batch element
  float* grad_bias = nullptr;       // [B,H,d]
  void* grad_ttt_lr_eta = nullptr;  // [B,H,seq]
  float* grad_token_eta = nullptr;  // [seq], per position
  float* grad_ln_weight = nullptr;  // [H,d]
  float* grad_ln_bias = nullptr;    // [H,d]
};

/// `fused-tile-multi` TTT-Linear layer on MI355X.
class FusedTileMulti {
 public:
  /// Parameters as TTTLinear holds them (linear.rs:17-25), device pointers, f32:
  /// weight_init [H,d,d], bias_init [H,d], LayerNorm weight/bias [H,d].
  FusedTileMulti(const ModelConfig& config, const float* weight_init, const float* bias_init,
                 const float* ln_weight, const float* ln_bias)
      : config_(config), weight_init_(weight_init), bias_init_(bias_init), ln_weight_(ln_weight),
        ln_bias_(ln_bias) {}

  static const char* name() { return "FusedTileMultiTTTLinear"; }  // wrapper.rs:85-87
  const ModelConfig& get_config() const { return config_; }

  ttt_desc desc(int batch, int seq, int mini_batch, ttt_dtype dtype, bool state_per_batch) const {
    ttt_desc d{};
    d.batch = batch;
    d.heads = config_.num_heads;
    d.seq = seq;
    d.head_dim = config_.head_dim;
    d.mini_batch = mini_batch;
    d.eps = config_.ttt.epsilon;
    d.checkpoint_interval = config_.ttt.checkpoint_interval;
    d.io_dtype = dtype;
    d.state_per_batch = state_per_batch ? 1 : 0;
    d.seq_stride = 0;
    d.checkpoint_format = config_.ttt.checkpoint_format;
    d.kernel_hint = config_.ttt.kernel_hint;
    return d;
  }

  std::int64_t num_checkpoints(int batch, int seq) const {
    ttt_desc d = desc(batch, seq, config_.ttt.mini_batch_size, TTT_F32, true);
    return ttt_linear_num_checkpoints(&d);
  }

  /// wrapper.rs:102-164 / inner.rs:25-50: all full mini-batches in one launch, then a trailing
  /// remainder as one short mini-batch, both as in-place windows of the [B,H,seq,d] tensors
  /// (desc.seq_stride).  state.weight/bias are read, state.next_* written, then swapped, so on
  /// return `state` is the updated state.  A state that is not initialised yet makes the first launch
  /// read the parameters directly (see TTTLinearState).  Checkpoints, if given, cover the full mini-batches.
  void forward(TTTLinearState& state, const TTTInputsInner& in, void* out, const Checkpoints& ck,
               void* stream) const {
    const int K = config_.ttt.mini_batch_size;
    const int full = (in.seq_len / K) * K;
    if (full > 0) launch(state, in, 0, full, K, out, ck, stream);
    if (full < in.seq_len) launch(state, in, full, in.seq_len - full, in.seq_len - full, out, Checkpoints{}, stream);
  }

  /// wrapper.rs:166-211: the mini-batch [first, first+len) of the sequence, len <= mini_batch_size.
  void forward_mini_batch(TTTLinearState& state, const TTTInputsInner& in, int first, int len, void* out,
                          void* stream) const {
    if (len <= 0 || len > config_.ttt.mini_batch_size || first < 0 || first + len > in.seq_len)
      throw Error(TTT_ERR_SHAPE, "range must be non-empty, inside the sequence and at most mini_batch_size long");
    launch(state, in, first, len, len, out, Checkpoints{}, stream);
  }

  /// backward_multi (backward/launch.rs:332-438): consumes the saved inputs, the checkpoints
  /// written by forward and grad_output [B,H,seq,d]; upstream gradients of the final state are
  /// optional (null = zero, as the reference assumes, launch.rs:188-194).
  /// `workspace`: null, or backward_workspace_bytes() bytes of device memory (16-byte aligned): where that size is
  /// above zero the backward then runs every (batch, head) unit on two workgroups (ttt_linear_bwd_ws).
  void backward(const TTTInputsInner& in, const float* weight0, const float* bias0,
                bool state_per_batch, const Checkpoints& ck, const void* grad_output,
                const float* grad_weight_out, const float* grad_bias_out, const TTTLinearGrads& g,
                void* stream, void* workspace = nullptr) const {
    ttt_desc d = desc(in.batch, in.seq_len, config_.ttt.mini_batch_size, in.dtype, state_per_batch);
    check(ttt_linear_bwd_ws(&d, in.qkv.xq, in.qkv.xk, in.qkv.xv, weight0, bias0, in.token_eta,
                            in.ttt_lr_eta, ln_weight_, ln_bias_, ck.weight, ck.bias, grad_output,
                            grad_weight_out, grad_bias_out, g.grad_xq, g.grad_xk, g.grad_xv,
                            g.grad_weight, g.grad_bias, g.grad_ttt_lr_eta, g.grad_token_eta,
                            g.grad_ln_weight, g.grad_ln_bias, workspace, stream));
  }

  /// Bytes of device workspace backward() can use for this batch and sequence length (0: it needs none).
  std::int64_t backward_workspace_bytes(int batch, int seq, ttt_dtype dtype, bool state_per_batch) const {
    ttt_desc d = desc(batch, seq, config_.ttt.mini_batch_size, dtype, state_per_batch);
    const std::int64_t n = ttt_linear_bwd_workspace_bytes(&d);
    if (n < 0) check((int)n);
    return n;
  }

 private:
  static const void* at(const void* p, std::size_t bytes) {
    return p ? static_cast<const char*>(p) + bytes : nullptr;
  }
  // tokens [first, first+seq) of every (batch, head) unit, in place
  void launch(TTTLinearState& state, const TTTInputsInner& in, int first, int seq, int mini_batch,
              void* out, const Checkpoints& ck, void* stream) const {
    if (!state.weight || !state.bias || !state.next_weight || !state.next_bias)
      throw Error(TTT_ERR_NULL, "TTTLinearState: weight, bias, next_weight and next_bias must all be valid buffers");
    const bool per_batch = state.initialised;
    const std::size_t es = in.dtype == TTT_BF16 ? 2 : 4;
    const std::size_t row = (std::size_t)first * (std::size_t)config_.head_dim * es;
    ttt_desc d = desc(in.batch, seq, mini_batch, in.dtype, per_batch);
    d.seq_stride = in.seq_len;
    check(ttt_linear_fwd(&d, at(in.qkv.xq, row), at(in.qkv.xk, row), at(in.qkv.xv, row),
                         per_batch ? state.weight : weight_init_, per_batch ? state.bias : bias_init_,
                         in.token_eta ? in.token_eta + first : nullptr,
                         at(in.ttt_lr_eta, (std::size_t)first * es), ln_weight_, ln_bias_,
                         const_cast<void*>(at(out, row)), state.next_weight, state.next_bias, ck.weight,
                         ck.bias, stream));
    state.swap();
    state.initialised = true;
  }

  ModelConfig config_;
  const float* weight_init_;
  const float* bias_init_;
  const float* ln_weight_;
  const float* ln_bias_;
};

}  // namespace ttt
