"""The C++ host class compiles against the C ABI header with a plain host compiler and reaches the
library's argument validation (no GPU needed: every call below is rejected before any launch)."""
import os
import subprocess
import sys
import textwrap

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def test_cpp_host_class_compiles_links_and_reports_errors(tmp_path):
    import importlib
    P = importlib.import_module("ttt-rs_amd")
    src = tmp_path / "t.cpp"
    src.write_text(textwrap.dedent(r'''
        #include <cstdio>
        #include <cstring>
        #include "ttt-rs_amd/host/fused_tile_multi.hpp"
        #include "ttt-rs_amd/host/fused_mlp.hpp"
        int main() {
          ttt::ModelConfig cfg; cfg.num_heads = 2; cfg.head_dim = 64;
          float dummy[4] = {0.f, 0.f, 0.f, 0.f};
          ttt::FusedTileMulti m(cfg, dummy, dummy, dummy, dummy);
          if (std::strcmp(m.name(), "FusedTileMultiTTTLinear")) return 1;
          if (m.num_checkpoints(2, 64) != 4) return 2;
          ttt::TTTInputsInner in; in.batch = 2; in.seq_len = 33;   // not a multiple of 16, > 16
          ttt::TTTLinearState st; alignas(16) char out[16];
          // a state without buffers is refused by the class itself
          in.seq_len = 32;
          try { m.forward(st, in, out, ttt::Checkpoints{}, nullptr); return 20; }
          catch (const ttt::Error& e) { if (e.code != TTT_ERR_NULL) return 21; }
          in.seq_len = 33;
          st.weight = st.bias = st.next_weight = st.next_bias = dummy;
          try { m.forward_mini_batch(st, in, 0, 33, out, nullptr); return 3; }
          catch (const ttt::Error& e) { if (e.code != TTT_ERR_SHAPE) return 4; }
          in.seq_len = 32;                                          // valid shape, null tensors
          try { m.forward(st, in, out, ttt::Checkpoints{}, nullptr); return 5; }
          catch (const ttt::Error& e) { if (e.code != TTT_ERR_NULL) return 6; std::printf("%s\n", e.what()); }
          // TTT-MLP host class: workspace query, shape and null-pointer rejection
          cfg.head_dim = 96;
          ttt::FusedMlp mlp(cfg, dummy, dummy, dummy, dummy, dummy, dummy);
          if (std::strcmp(mlp.name(), "FusedTTTMLP")) return 7;
          // per (batch, head): 2 d M + M + d + N 16 (M + d) + 9 * 16 M floats, M = 4 d; up to 128 units (two
          // workgroups per unit) a second state buffer, six more tiles, two exchange blocks, bf16 copies of both state
          // buffers and 32 counter words
          const long long xb = 48LL * 96 + 4 * 256 + 16 + 96;
          const long long per_unit = 2LL * 96 * 384 + 384 + 96 + 2LL * 16 * (384 + 96) + 9LL * 16 * 384
                                     + 2LL * 96 * 384 + 6LL * 16 * 384 + 2 * xb + 2LL * 96 * 384 + 32;
          if (mlp.backward_workspace_bytes(2, 32, TTT_BF16) != 4 * 2 * 2 * per_unit) return 8;
          ttt::TTTMLPState ms;
          ms.w1 = ms.b1 = ms.w2 = ms.b2 = ms.next_w1 = ms.next_b1 = ms.next_w2 = ms.next_b2 = dummy;
          try { mlp.forward_mini_batch(ms, in, 0, 17, out, nullptr); return 9; }
          catch (const ttt::Error& e) { if (e.code != TTT_ERR_SHAPE) return 10; }
          try { mlp.backward(in, ms, out, nullptr, nullptr, nullptr, nullptr, ttt::TTTMLPGrads{}, out, nullptr); return 11; }
          catch (const ttt::Error& e) { if (e.code != TTT_ERR_NULL) return 12; }
          // the saving pair: null tensors are refused, and so is the forward that runs on pairs of CUs
          in.dtype = TTT_BF16;
          try { mlp.forward_saving(ms, in, out, out, nullptr); return 13; }
          catch (const ttt::Error& e) { if (e.code != TTT_ERR_NULL) return 14; }
          try { mlp.backward_saved(in, ms, out, nullptr, nullptr, nullptr, nullptr, ttt::TTTMLPGrads{}, out, nullptr); return 15; }
          catch (const ttt::Error& e) { if (e.code != TTT_ERR_NULL) return 16; }
          cfg.head_dim = 128;
          ttt::FusedMlp wide(cfg, dummy, dummy, dummy, dummy, dummy, dummy);
          try { wide.forward_saving(ms, in, out, out, nullptr); return 17; }
          catch (const ttt::Error& e) { if (e.code != TTT_ERR_UNSUPPORTED) return 18; }
          return 0;
        }
    '''))
    exe = tmp_path / "t"
    libdir = os.path.dirname(P.LIB_PATH)
    subprocess.run(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-I", ROOT, str(src), "-o", str(exe),
                    "-L", libdir, "-lttt_mi355x", f"-Wl,-rpath,{libdir}"], check=True)
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0, (r.returncode, r.stdout, r.stderr)
    assert "NULL" in r.stdout


def test_cpp_host_state_buffers_across_a_forward_with_remainder(tmp_path):
    """The host classes against a stub of the C ABI that records what it is given: a forward with a remainder is
    two launches; both must read a valid state and write a valid, different buffer (the first from the layer's
    parameters when the state is not initialised), and the final state must end up where the class says."""
    src = tmp_path / "s.cpp"
    src.write_text(textwrap.dedent(r'''
        #include <cstdio>
        #include <vector>
        #include "ttt-rs_amd/host/fused_tile_multi.hpp"
        #include "ttt-rs_amd/host/fused_mlp.hpp"
        struct Call { const float* w_in; float* w_out; int seq, K, per_batch, stride; const void* xq; };
        static std::vector<Call> calls;
        extern "C" {
        const char* ttt_last_error(void) { return "stub"; }
        int64_t ttt_linear_num_checkpoints(const ttt_desc*) { return 0; }
        int64_t ttt_mlp_bwd_workspace_bytes(const ttt_desc*) { return 0; }
        int ttt_linear_fwd(const ttt_desc* d, const void* xq, const void*, const void*, const float* W0, const float* b0,
                           const float*, const void*, const float*, const float*, void* out, float* W_out, float* b_out,
                           float*, float*, void*) {
          if (!W0 || !b0 || !W_out || !b_out || !out) return TTT_ERR_NULL;
          calls.push_back({W0, W_out, d->seq, d->mini_batch, d->state_per_batch, d->seq_stride, xq});
          return TTT_OK;
        }
        int ttt_linear_bwd(const ttt_desc*, const void*, const void*, const void*, const float*, const float*, const float*,
                           const void*, const float*, const float*, const float*, const float*, const void*, const float*,
                           const float*, void*, void*, void*, float*, float*, void*, float*, float*, float*, void*) { return TTT_OK; }
        int ttt_mlp_fwd(const ttt_desc* d, const void* xq, const void*, const void*, const float* W1, const float* b1,
                        const float* W2, const float* b2, const float*, const void*, const float*, const float*, void* out,
                        float* W1o, float* b1o, float* W2o, float* b2o, void*) {
          if (!W1 || !b1 || !W2 || !b2 || !W1o || !b1o || !W2o || !b2o || !out) return TTT_ERR_NULL;
          calls.push_back({W1, W1o, d->seq, d->mini_batch, d->state_per_batch, d->seq_stride, xq});
          return TTT_OK;
        }
        int ttt_mlp_bwd(const ttt_desc*, const void*, const void*, const void*, const float*, const float*, const float*,
                        const float*, const float*, const void*, const float*, const float*, const void*, const float*,
                        const float*, const float*, const float*, void*, void*, void*, float*, float*, float*, float*, void*,
                        float*, float*, float*, void*, void*) { return TTT_OK; }
        }
        int main() {
          ttt::ModelConfig cfg; cfg.num_heads = 2; cfg.head_dim = 64;
          static float params[4], A[4], B[4], x[4 * 64 * 64];
          ttt::FusedTileMulti m(cfg, params, params, params, params);
          ttt::TTTInputsInner in; in.batch = 1; in.seq_len = 16 * 2 + 5; in.qkv = ttt::Qkv{x, x, x};
          in.token_eta = params; in.ttt_lr_eta = x;
          ttt::TTTLinearState st; st.weight = A; st.bias = A; st.next_weight = B; st.next_bias = B;
          m.forward(st, in, x, ttt::Checkpoints{}, nullptr);
          if (calls.size() != 2) return 1;
          // launch 1: parameters in ([H,..] broadcast), buffer B out, 32 tokens in mini-batches of 16
          if (calls[0].w_in != params || calls[0].w_out != B || calls[0].per_batch != 0 || calls[0].seq != 32 ||
              calls[0].K != 16 || calls[0].stride != 37) return 2;
          // launch 2: the remainder as one short mini-batch, reads B, writes A, window starts at token 32
          if (calls[1].w_in != B || calls[1].w_out != A || calls[1].per_batch != 1 || calls[1].seq != 5 ||
              calls[1].K != 5 || calls[1].stride != 37 || calls[1].xq != (const void*)(x + 32 * 64)) return 3;
          if (st.weight != A || st.next_weight != B || !st.initialised) return 4;
          // the next forward continues from the state (no re-read of the parameters)
          calls.clear();
          in.seq_len = 16;
          m.forward(st, in, x, ttt::Checkpoints{}, nullptr);
          if (calls.size() != 1 || calls[0].w_in != A || calls[0].w_out != B || calls[0].per_batch != 1) return 5;
          // TTT-MLP: same protocol
          calls.clear();
          ttt::FusedMlp mlp(cfg, params, params, params, params, params, params);
          ttt::TTTMLPState ms;
          ms.w1 = ms.b1 = ms.w2 = ms.b2 = A; ms.next_w1 = ms.next_b1 = ms.next_w2 = ms.next_b2 = B;
          in.seq_len = 16 + 3;
          mlp.forward(ms, in, x, nullptr);
          if (calls.size() != 2 || calls[0].w_in != params || calls[0].w_out != B || calls[1].w_in != B ||
              calls[1].w_out != A || calls[1].seq != 3 || ms.w1 != A || !ms.initialised) return 6;
          return 0;
        }
    '''))
    exe = tmp_path / "s"
    subprocess.run(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-I", ROOT, str(src), "-o", str(exe)], check=True)
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0, (r.returncode, r.stdout, r.stderr)


def test_cpp_other_inner_models_compile_and_report_errors(tmp_path):
    """host/fused_others.hpp (TTTLinearAdam, TTTMLP2/3/4): names as the reference's, incomplete states refused by the
    classes, unsupported shapes and null tensors by the library, all before any launch."""
    import importlib
    P = importlib.import_module("ttt-rs_amd")
    src = tmp_path / "o.cpp"
    src.write_text(textwrap.dedent(r'''
        #include <cstring>
        #include "ttt-rs_amd/host/fused_others.hpp"
        int main() {
          ttt::ModelConfig cfg; cfg.num_heads = 2; cfg.head_dim = 64;
          alignas(16) float dummy[4] = {0.f, 0.f, 0.f, 0.f};
          alignas(16) char out[16];
          ttt::TTTInputsInner in; in.batch = 2; in.seq_len = 32;
          ttt::FusedLinearAdam adam(cfg, ttt::TTTLinearAdamConfig{}, dummy, dummy, dummy, dummy);
          if (std::strcmp(adam.name(), "TTTLinearAdam")) return 1;
          ttt::TTTLinearAdamState as;
          try { adam.forward(as, in, out, nullptr); return 2; }
          catch (const ttt::Error& e) { if (e.code != TTT_ERR_NULL) return 3; }
          as.weight = as.bias = as.weight_m = as.bias_m = as.weight_v = as.bias_v = dummy;
          as.next_weight = as.next_bias = as.next_weight_m = as.next_bias_m = as.next_weight_v = as.next_bias_v = dummy;
          try { adam.forward_mini_batch(as, in, 0, 17, out, nullptr); return 4; }
          catch (const ttt::Error& e) { if (e.code != TTT_ERR_SHAPE) return 5; }
          try { adam.forward(as, in, out, nullptr); return 6; }          // null activations
          catch (const ttt::Error& e) { if (e.code != TTT_ERR_NULL) return 7; }
          if (as.initialised || as.step != 0) return 8;                    // a refused call leaves the state alone
          const float* layers[5] = {dummy, dummy, dummy, dummy, dummy};
          try { ttt::FusedMlpN bad(cfg, 5, layers, layers, dummy, dummy); return 9; }
          catch (const ttt::Error& e) { if (e.code != TTT_ERR_UNSUPPORTED) return 10; }
          ttt::FusedMlpN m3(cfg, 3, layers, layers, dummy, dummy);         // head_dim 64 has two hidden layers only
          if (std::strcmp(m3.name(), "TTTMLP3")) return 11;
          ttt::TTTMLPNState ms;
          try { m3.forward(ms, in, out, nullptr); return 12; }
          catch (const ttt::Error& e) { if (e.code != TTT_ERR_NULL) return 13; }
          for (int i = 0; i < 4; ++i) ms.weight[i] = ms.bias[i] = ms.next_weight[i] = ms.next_bias[i] = dummy;
          try { m3.forward(ms, in, out, nullptr); return 14; }
          catch (const ttt::Error& e) { if (e.code != TTT_ERR_UNSUPPORTED) return 15; }
          cfg.head_dim = 32;
          ttt::FusedMlpN m4(cfg, 4, layers, layers, dummy, dummy);
          if (std::strcmp(m4.name(), "TTTMLP4")) return 16;
          for (int i = 0; i < 5; ++i) ms.weight[i] = ms.bias[i] = ms.next_weight[i] = ms.next_bias[i] = dummy;
          try { m4.forward(ms, in, out, nullptr); return 17; }            // supported shape, null activations
          catch (const ttt::Error& e) { if (e.code != TTT_ERR_NULL) return 18; }
          return 0;
        }
    '''))
    exe = tmp_path / "o"
    libdir = os.path.dirname(P.LIB_PATH)
    subprocess.run(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-I", ROOT, str(src), "-o", str(exe),
                    "-L", libdir, "-lttt_mi355x", f"-Wl,-rpath,{libdir}"], check=True)
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0, (r.returncode, r.stdout, r.stderr)
