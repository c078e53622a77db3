// C++ host-side mirrors of the reference's other inner models, above the C ABI of include/ttt_mi355x.h:
//   TTTLinearAdam / TTTLinearAdamState / TTTLinearAdamConfig   rust/core/src/linear_adam.rs:19-62, 134-236
//   TTTMLP2 / TTTMLP3 / TTTMLP4 and their states              rust/core/src/mlp2.rs:21-53, mlp3.rs:21-53, mlp4.rs:21-59
// with the TTTInnerModel interface (rust/core/src/inner.rs:13-58): name / get_config / forward / forward_mini_batch.
// Forward only, as the library's entry points for them.  Ownership and errors as in fused_tile_multi.hpp: caller-owned
// device buffers, nothing allocated here, ttt::Error carries the library's status.
#pragma once

#include "fused_tile_multi.hpp"

namespace ttt {

/// linear_adam.rs:46-62
struct TTTLinearAdamConfig {
  float beta1 = 0.9f;
  float beta2 = 0.999f;
  float epsilon = 1e-8f;
  float lr = 1e-3f;
};

/// linear_adam.rs:28-44: state, first and second moments [B,H,d,d] / [B,H,d] f32 and the step counter.  As in
/// TTTLinearState every tensor is a pair of buffers (the library never writes a state in place): a call reads the
/// current ones and writes the `next_` ones, then they swap.  `initialised == false`: the first call reads the
/// layer's parameters, zero moments and step 0 (TTTLinearAdam::init_state, linear_adam.rs:164-177, without a copy).
struct TTTLinearAdamState {
  float *weight = nullptr, *bias = nullptr, *weight_m = nullptr, *bias_m = nullptr, *weight_v = nullptr, *bias_v = nullptr;
  float *next_weight = nullptr, *next_bias = nullptr, *next_weight_m = nullptr, *next_bias_m = nullptr,
        *next_weight_v = nullptr, *next_bias_v = nullptr;
  int step = 0;
  bool initialised = false;
  void swap() {
    auto sw = [](float*& a, float*& b) { float* t = a; a = b; b = t; };
    sw(weight, next_weight); sw(bias, next_bias); sw(weight_m, next_weight_m); sw(bias_m, next_bias_m);
    sw(weight_v, next_weight_v); sw(bias_v, next_bias_v);
  }
  bool complete() const {
    return weight && bias && weight_m && bias_m && weight_v && bias_v && next_weight && next_bias && next_weight_m &&
           next_bias_m && next_weight_v && next_bias_v;
  }
};

/// TTT-Linear with an Adam inner optimiser on the fused kernel (ttt_linear_adam_fwd).
class FusedLinearAdam {
 public:
  FusedLinearAdam(const ModelConfig& config, const TTTLinearAdamConfig& adam, const float* weight_init,
                  const float* bias_init, const float* ln_weight, const float* ln_bias)
      : config_(config), adam_(adam), weight_init_(weight_init), bias_init_(bias_init), ln_weight_(ln_weight),
        ln_bias_(ln_bias) {}

  static const char* name() { return "TTTLinearAdam"; }  // linear_adam.rs:134-136
  const ModelConfig& get_config() const { return config_; }

  /// inner.rs:25-50: all full mini-batches in one launch, a trailing remainder as one short mini-batch.
  void forward(TTTLinearAdamState& state, const TTTInputsInner& in, void* out, void* stream) const {
    const int K = config_.ttt.mini_batch_size;
    const int full = (in.seq_len / K) * K;
    if (full > 0) launch(state, in, 0, full, K, out, stream);
    if (full < in.seq_len) launch(state, in, full, in.seq_len - full, in.seq_len - full, out, stream);
  }
  void forward_mini_batch(TTTLinearAdamState& state, const TTTInputsInner& in, int first, int len, void* out,
                          void* stream) const {
    if (len <= 0 || len > config_.ttt.mini_batch_size || first < 0 || first + len > in.seq_len)
      throw Error(TTT_ERR_SHAPE, "range must be non-empty, inside the sequence and at most mini_batch_size long");
    launch(state, in, first, len, len, out, stream);
  }

 private:
  static const void* at(const void* p, std::size_t bytes) { return p ? static_cast<const char*>(p) + bytes : nullptr; }
  void launch(TTTLinearAdamState& st, const TTTInputsInner& in, int first, int seq, int mini_batch, void* out,
              void* stream) const {
    if (!st.complete()) throw Error(TTT_ERR_NULL, "TTTLinearAdamState: all twelve buffers must be valid");
    const bool live = st.initialised;
    const std::size_t es = in.dtype == TTT_BF16 ? 2 : 4;
    const std::size_t row = (std::size_t)first * (std::size_t)config_.head_dim * es;
    ttt_desc d{};
    d.batch = in.batch; d.heads = config_.num_heads; d.seq = seq; d.head_dim = config_.head_dim;
    d.mini_batch = mini_batch; d.eps = config_.ttt.epsilon; d.checkpoint_interval = 1; d.io_dtype = in.dtype;
    d.state_per_batch = live ? 1 : 0; d.seq_stride = in.seq_len; d.checkpoint_format = TTT_CKPT_F32;
    d.kernel_hint = config_.ttt.kernel_hint;
    check(ttt_linear_adam_fwd(&d, at(in.qkv.xq, row), at(in.qkv.xk, row), at(in.qkv.xv, row),
                              live ? st.weight : weight_init_, live ? st.bias : bias_init_,
                              live ? st.weight_m : nullptr, live ? st.bias_m : nullptr, live ? st.weight_v : nullptr,
                              live ? st.bias_v : nullptr, live ? st.step : 0, adam_.beta1, adam_.beta2, adam_.epsilon,
                              adam_.lr, in.token_eta ? in.token_eta + first : nullptr,
                              at(in.ttt_lr_eta, (std::size_t)first * es), ln_weight_, ln_bias_,
                              const_cast<void*>(at(out, row)), st.next_weight, st.next_bias, st.next_weight_m,
                              st.next_bias_m, st.next_weight_v, st.next_bias_v, stream));
    st.swap();
    st.step = (live ? st.step : 0) + seq / mini_batch;
    st.initialised = true;
  }

  ModelConfig config_;
  TTTLinearAdamConfig adam_;
  const float *weight_init_, *bias_init_, *ln_weight_, *ln_bias_;
};

/// State of TTTMLP2 / 3 / 4 (mlp2.rs:38-53, mlp3.rs:42-53, mlp4.rs:46-59): n_hidden + 1 weight layers
/// [B,H,in_i,out_i] and biases [B,H,out_i], f32; pairs of buffers as above.
struct TTTMLPNState {
  static constexpr int kMaxLayers = 5;
  float* weight[kMaxLayers] = {};
  float* bias[kMaxLayers] = {};
  float* next_weight[kMaxLayers] = {};
  float* next_bias[kMaxLayers] = {};
  bool initialised = false;
  void swap() {
    for (int i = 0; i < kMaxLayers; ++i) {
      float* w = weight[i]; weight[i] = next_weight[i]; next_weight[i] = w;
      float* b = bias[i]; bias[i] = next_bias[i]; next_bias[i] = b;
    }
  }
};

/// TTT-MLP with 2, 3 or 4 hidden layers of width 4 d on the fused kernel (ttt_mlpn_fwd).
class FusedMlpN {
 public:
  /// weight_init[i] [H,in_i,out_i], bias_init[i] [H,out_i] for the n_hidden + 1 layers (device pointers, f32).
  FusedMlpN(const ModelConfig& config, int n_hidden, const float* const* weight_init, const float* const* bias_init,
            const float* ln_weight, const float* ln_bias)
      : config_(config), n_hidden_(n_hidden), ln_weight_(ln_weight), ln_bias_(ln_bias) {
    if (n_hidden < 2 || n_hidden > 4) throw Error(TTT_ERR_UNSUPPORTED, "FusedMlpN: 2, 3 or 4 hidden layers");
    for (int i = 0; i <= n_hidden; ++i) {
      weight_init_[i] = weight_init[i];
      bias_init_[i] = bias_init[i];
    }
  }

  /// mlp2.rs:70-72, mlp3.rs:70-72, mlp4.rs:76-78
  const char* name() const { return n_hidden_ == 2 ? "TTTMLP2" : n_hidden_ == 3 ? "TTTMLP3" : "TTTMLP4"; }
  const ModelConfig& get_config() const { return config_; }
  int n_hidden() const { return n_hidden_; }

  void forward(TTTMLPNState& state, const TTTInputsInner& in, void* out, void* stream) const {
    const int K = config_.ttt.mini_batch_size;
    const int full = (in.seq_len / K) * K;
    if (full > 0) launch(state, in, 0, full, K, out, stream);
    if (full < in.seq_len) launch(state, in, full, in.seq_len - full, in.seq_len - full, out, stream);
  }
  void forward_mini_batch(TTTMLPNState& state, const TTTInputsInner& in, int first, int len, void* out,
                          void* stream) const {
    if (len <= 0 || len > config_.ttt.mini_batch_size || first < 0 || first + len > in.seq_len)
      throw Error(TTT_ERR_SHAPE, "range must be non-empty, inside the sequence and at most mini_batch_size long");
    launch(state, in, first, len, len, out, stream);
  }

 private:
  static const void* at(const void* p, std::size_t bytes) { return p ? static_cast<const char*>(p) + bytes : nullptr; }
  void launch(TTTMLPNState& st, const TTTInputsInner& in, int first, int seq, int mini_batch, void* out,
              void* stream) const {
    for (int i = 0; i <= n_hidden_; ++i)
      if (!st.weight[i] || !st.bias[i] || !st.next_weight[i] || !st.next_bias[i])
        throw Error(TTT_ERR_NULL, "TTTMLPNState: every layer needs weight, bias, next_weight and next_bias");
    const bool live = st.initialised;
    const std::size_t es = in.dtype == TTT_BF16 ? 2 : 4;
    const std::size_t row = (std::size_t)first * (std::size_t)config_.head_dim * es;
    ttt_desc d{};
    d.batch = in.batch; d.heads = config_.num_heads; d.seq = seq; d.head_dim = config_.head_dim;
    d.mini_batch = mini_batch; d.eps = config_.ttt.epsilon; d.checkpoint_interval = 1; d.io_dtype = in.dtype;
    d.state_per_batch = live ? 1 : 0; d.seq_stride = in.seq_len; d.checkpoint_format = TTT_CKPT_F32;
    d.kernel_hint = config_.ttt.kernel_hint;
    check(ttt_mlpn_fwd(&d, n_hidden_, at(in.qkv.xq, row), at(in.qkv.xk, row), at(in.qkv.xv, row),
                       live ? st.weight : weight_init_, live ? st.bias : bias_init_,
                       in.token_eta ? in.token_eta + first : nullptr, at(in.ttt_lr_eta, (std::size_t)first * es),
                       ln_weight_, ln_bias_, const_cast<void*>(at(out, row)), st.next_weight, st.next_bias, stream));
    st.swap();
    st.initialised = true;
  }

  ModelConfig config_;
  int n_hidden_;
  const float* weight_init_[TTTMLPNState::kMaxLayers] = {};
  const float* bias_init_[TTTMLPNState::kMaxLayers] = {};
  const float *ln_weight_, *ln_bias_;
};

}  // namespace ttt
