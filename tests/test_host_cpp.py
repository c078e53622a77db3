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
          ttt::TTTLinearState st; char out[4];
          try { m.forward_mini_batch(st, in, 0, 33, out, nullptr); return 3; }
          catch (const ttt::Error& e) { if (e.code != TTT_ERR_SHAPE) return 4; }
          in.seq_len = 32;                                          // valid shape, null tensors
          try { m.forward(st, in, out, ttt::Checkpoints{}, nullptr); return 5; }
          catch (const ttt::Error& e) { if (e.code != TTT_ERR_NULL) return 6; std::printf("%s\n", e.what()); }
          // TTT-MLP host class: workspace query, shape and null-pointer rejection
          cfg.head_dim = 96;
          ttt::FusedMlp mlp(cfg, dummy, dummy, dummy, dummy, dummy, dummy);
          if (std::strcmp(mlp.name(), "FusedTTTMLP")) return 7;
          // per (batch, head): 2 d M + M + d + N 16 (M + d) + 9 * 16 M floats, M = 4 d
          const long long per_unit = 2LL * 96 * 384 + 384 + 96 + 2LL * 16 * (384 + 96) + 9LL * 16 * 384;
          if (mlp.backward_workspace_bytes(2, 32, TTT_BF16) != 4 * 2 * 2 * per_unit) return 8;
          ttt::TTTMLPState ms;
          try { mlp.forward_mini_batch(ms, in, 0, 17, out, nullptr); return 9; }
          catch (const ttt::Error& e) { if (e.code != TTT_ERR_SHAPE) return 10; }
          try { mlp.backward(in, ms, out, nullptr, nullptr, nullptr, nullptr, ttt::TTTMLPGrads{}, out, nullptr); return 11; }
          catch (const ttt::Error& e) { if (e.code != TTT_ERR_NULL) return 12; }
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
