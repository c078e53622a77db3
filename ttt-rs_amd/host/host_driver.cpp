// Thin C entry points over the C++ host classes (fused_tile_multi.hpp, fused_mlp.hpp, fused_others.hpp) so that a test
// process can drive them with device buffers it already owns: each function builds the class the way a
// C++ caller would and runs one forward (full mini-batches + remainder, as TTTInnerModel::forward,
// rust/core/src/inner.rs:25-50) and, where the sequence allows it, one backward.  Built as
// libttt_host_driver.so next to the library; nothing here allocates, copies or synchronises.
#include <cstring>

#include "fused_mlp.hpp"
#include "fused_others.hpp"
#include "fused_tile_multi.hpp"

namespace {
thread_local char g_msg[512] = "";
int report(const ttt::Error& e) {
  std::strncpy(g_msg, e.what(), sizeof(g_msg) - 1);
  return e.code;
}
}  // namespace

extern "C" {

const char* ttt_host_last_error(void) { return g_msg; }

// TTT-Linear: forward over `seq` tokens (any length), state buffers {w,b}[2] of [B,H,d,d] / [B,H,d];
// on return *cur says which of the two pairs holds the final state.  ck_w/ck_b may be null.
int ttt_host_linear_forward(int B, int H, int d, int K, int seq, int dtype, float eps, int ckpt_interval,
                            int ckpt_format, const float* W0, const float* b0, const float* gamma, const float* beta,
                            const void* xq, const void* xk, const void* xv, const float* token_eta, const void* lr,
                            void* out, float* w_a, float* b_a, float* w_b, float* b_b, float* ck_w, float* ck_b,
                            int* cur, void* stream) {
  try {
    ttt::ModelConfig cfg;
    cfg.num_heads = H;
    cfg.head_dim = d;
    cfg.ttt.mini_batch_size = K;
    cfg.ttt.epsilon = eps;
    cfg.ttt.checkpoint_interval = ckpt_interval;
    cfg.ttt.checkpoint_format = ckpt_format;
    ttt::FusedTileMulti model(cfg, W0, b0, gamma, beta);
    ttt::TTTInputsInner in;
    in.qkv = ttt::Qkv{xq, xk, xv};
    in.token_eta = token_eta;
    in.ttt_lr_eta = lr;
    in.batch = B;
    in.seq_len = seq;
    in.dtype = static_cast<ttt_dtype>(dtype);
    ttt::TTTLinearState st;
    st.weight = w_a; st.bias = b_a; st.next_weight = w_b; st.next_bias = b_b;
    model.forward(st, in, out, ttt::Checkpoints{ck_w, ck_b}, stream);
    *cur = st.weight == w_a ? 0 : 1;
    return TTT_OK;
  } catch (const ttt::Error& e) {
    return report(e);
  }
}

int ttt_host_linear_backward(int B, int H, int d, int K, int seq, int dtype, float eps, int ckpt_interval,
                             int ckpt_format, const float* W0, const float* b0, const float* gamma,
                             const float* beta, const void* xq, const void* xk, const void* xv,
                             const float* token_eta, const void* lr, const float* ck_w, const float* ck_b,
                             const void* d_out, void* d_xq, void* d_xk, void* d_xv, float* d_W, float* d_b,
                             void* d_lr, float* d_te, float* d_gamma, float* d_beta, void* stream,
                             void* workspace, long long workspace_bytes) {
  try {
    ttt::ModelConfig cfg;
    cfg.num_heads = H;
    cfg.head_dim = d;
    cfg.ttt.mini_batch_size = K;
    cfg.ttt.epsilon = eps;
    cfg.ttt.checkpoint_interval = ckpt_interval;
    cfg.ttt.checkpoint_format = ckpt_format;
    ttt::FusedTileMulti model(cfg, W0, b0, gamma, beta);
    // the caller's workspace is used when it is large enough for what the class asks for
    if (workspace != nullptr &&
        model.backward_workspace_bytes(B, seq, static_cast<ttt_dtype>(dtype), false) > workspace_bytes)
      throw ttt::Error(TTT_ERR_SHAPE, "workspace smaller than FusedTileMulti::backward_workspace_bytes");
    ttt::TTTInputsInner in;
    in.qkv = ttt::Qkv{xq, xk, xv};
    in.token_eta = token_eta;
    in.ttt_lr_eta = lr;
    in.batch = B;
    in.seq_len = seq;
    in.dtype = static_cast<ttt_dtype>(dtype);
    ttt::TTTLinearGrads g;
    g.grad_xq = d_xq; g.grad_xk = d_xk; g.grad_xv = d_xv; g.grad_weight = d_W; g.grad_bias = d_b;
    g.grad_ttt_lr_eta = d_lr; g.grad_token_eta = d_te; g.grad_ln_weight = d_gamma; g.grad_ln_bias = d_beta;
    model.backward(in, W0, b0, false, ttt::Checkpoints{const_cast<float*>(ck_w), const_cast<float*>(ck_b)}, d_out,
                   nullptr, nullptr, g, stream, workspace);
    return TTT_OK;
  } catch (const ttt::Error& e) {
    return report(e);
  }
}

// TTT-MLP: forward over `seq` tokens (any length) with two sets of state buffers; then, if ws is not null,
// the backward of the same sequence (seq must then be a multiple of K) from the parameters.
int ttt_host_mlp_forward_backward(int B, int H, int d, int K, int seq, int dtype, float eps, const float* W1,
                                  const float* b1, const float* W2, const float* b2, const float* gamma,
                                  const float* beta, const void* xq, const void* xk, const void* xv,
                                  const float* token_eta, const void* lr, void* out, float* const* state_a,
                                  float* const* state_b, int* cur, const void* d_out, void* d_xq, void* d_xk,
                                  void* d_xv, float* d_W1, float* d_b1, float* d_W2, float* d_b2, void* d_lr,
                                  float* d_te, float* d_gamma, float* d_beta, void* ws, void* stream) {
  try {
    ttt::ModelConfig cfg;
    cfg.num_heads = H;
    cfg.head_dim = d;
    cfg.ttt.mini_batch_size = K;
    cfg.ttt.epsilon = eps;
    ttt::FusedMlp model(cfg, W1, b1, W2, b2, gamma, beta);
    ttt::TTTInputsInner in;
    in.qkv = ttt::Qkv{xq, xk, xv};
    in.token_eta = token_eta;
    in.ttt_lr_eta = lr;
    in.batch = B;
    in.seq_len = seq;
    in.dtype = static_cast<ttt_dtype>(dtype);
    ttt::TTTMLPState st;
    st.w1 = state_a[0]; st.b1 = state_a[1]; st.w2 = state_a[2]; st.b2 = state_a[3];
    st.next_w1 = state_b[0]; st.next_b1 = state_b[1]; st.next_w2 = state_b[2]; st.next_b2 = state_b[3];
    model.forward(st, in, out, stream);
    *cur = st.w1 == state_a[0] ? 0 : 1;
    if (ws != nullptr) {
      ttt::TTTMLPGrads g;
      g.grad_xq = d_xq; g.grad_xk = d_xk; g.grad_xv = d_xv; g.grad_w1 = d_W1; g.grad_b1 = d_b1; g.grad_w2 = d_W2;
      g.grad_b2 = d_b2; g.grad_ttt_lr_eta = d_lr; g.grad_token_eta = d_te; g.grad_ln_weight = d_gamma;
      g.grad_ln_bias = d_beta;
      model.backward(in, ttt::TTTMLPState{}, d_out, nullptr, nullptr, nullptr, nullptr, g, ws, stream);
    }
    return TTT_OK;
  } catch (const ttt::Error& e) {
    return report(e);
  }
}

// TTT-Linear with the Adam inner optimiser: forward over `seq` tokens (any length).  bufs_a / bufs_b: the two sets of
// {weight, bias, weight_m, bias_m, weight_v, bias_v}; on return *cur says which set is current and *step holds the
// step counter.
int ttt_host_linear_adam_forward(int B, int H, int d, int K, int seq, int dtype, float eps, float beta1, float beta2,
                                 float adam_eps, float adam_lr, const float* W0, const float* b0, const float* gamma,
                                 const float* beta, const void* xq, const void* xk, const void* xv,
                                 const float* token_eta, const void* lr, void* out, float* const* bufs_a,
                                 float* const* bufs_b, int* cur, int* step, void* stream) {
  try {
    ttt::ModelConfig cfg;
    cfg.num_heads = H;
    cfg.head_dim = d;
    cfg.ttt.mini_batch_size = K;
    cfg.ttt.epsilon = eps;
    ttt::TTTLinearAdamConfig ac;
    ac.beta1 = beta1; ac.beta2 = beta2; ac.epsilon = adam_eps; ac.lr = adam_lr;
    ttt::FusedLinearAdam model(cfg, ac, W0, b0, gamma, beta);
    ttt::TTTInputsInner in;
    in.qkv = ttt::Qkv{xq, xk, xv};
    in.token_eta = token_eta;
    in.ttt_lr_eta = lr;
    in.batch = B;
    in.seq_len = seq;
    in.dtype = static_cast<ttt_dtype>(dtype);
    ttt::TTTLinearAdamState st;
    st.weight = bufs_a[0]; st.bias = bufs_a[1]; st.weight_m = bufs_a[2]; st.bias_m = bufs_a[3];
    st.weight_v = bufs_a[4]; st.bias_v = bufs_a[5];
    st.next_weight = bufs_b[0]; st.next_bias = bufs_b[1]; st.next_weight_m = bufs_b[2]; st.next_bias_m = bufs_b[3];
    st.next_weight_v = bufs_b[4]; st.next_bias_v = bufs_b[5];
    model.forward(st, in, out, stream);
    *cur = st.weight == bufs_a[0] ? 0 : 1;
    *step = st.step;
    return TTT_OK;
  } catch (const ttt::Error& e) {
    return report(e);
  }
}

// TTT-MLP with n_hidden hidden layers: forward over `seq` tokens (any length).  W0 / b0: the n_hidden + 1 parameter
// layers; w_a / b_a and w_b / b_b: the two sets of state buffers; *cur says which set is current on return.
int ttt_host_mlpn_forward(int B, int H, int d, int K, int seq, int dtype, float eps, int n_hidden,
                          const float* const* W0, const float* const* b0, const float* gamma, const float* beta,
                          const void* xq, const void* xk, const void* xv, const float* token_eta, const void* lr,
                          void* out, float* const* w_a, float* const* b_a, float* const* w_b, float* const* b_b, int* cur,
                          void* stream) {
  try {
    ttt::ModelConfig cfg;
    cfg.num_heads = H;
    cfg.head_dim = d;
    cfg.ttt.mini_batch_size = K;
    cfg.ttt.epsilon = eps;
    ttt::FusedMlpN model(cfg, n_hidden, W0, b0, gamma, beta);
    ttt::TTTInputsInner in;
    in.qkv = ttt::Qkv{xq, xk, xv};
    in.token_eta = token_eta;
    in.ttt_lr_eta = lr;
    in.batch = B;
    in.seq_len = seq;
    in.dtype = static_cast<ttt_dtype>(dtype);
    ttt::TTTMLPNState st;
    for (int i = 0; i <= n_hidden; ++i) {
      st.weight[i] = w_a[i]; st.bias[i] = b_a[i]; st.next_weight[i] = w_b[i]; st.next_bias[i] = b_b[i];
    }
    model.forward(st, in, out, stream);
    *cur = st.weight[0] == w_a[0] ? 0 : 1;
    return TTT_OK;
  } catch (const ttt::Error& e) {
    return report(e);
  }
}

// LostWorkgroupGuard (fused_mlp.hpp) for a test process: new -> its work -> synchronise -> verify -> free.
// These two calls read the device's status word with a blocking copy.
void* ttt_host_lost_guard_new(void) {
  try {
    return new ttt::LostWorkgroupGuard();
  } catch (const ttt::Error& e) {
    report(e);
    return nullptr;
  }
}

int ttt_host_lost_guard_verify_and_free(void* guard) {
  ttt::LostWorkgroupGuard* g = static_cast<ttt::LostWorkgroupGuard*>(guard);
  int rc = TTT_OK;
  try {
    g->verify();
  } catch (const ttt::Error& e) {
    rc = report(e);
  }
  delete g;
  return rc;
}

// ttt::stack_forward with the arguments of ttt_stack_fwd.
int ttt_host_stack_forward(const ttt_desc* desc, int n_layers, const ttt_stack_layer* layers, const float* token_eta,
                           void* out, void* workspace, int chunk_tokens, void* aux_stream, void* stream) {
  try {
    ttt::stack_forward(*desc, n_layers, layers, token_eta, out, workspace, chunk_tokens, aux_stream, stream);
    return TTT_OK;
  } catch (const ttt::Error& e) {
    return report(e);
  }
}

}  // extern "C"
