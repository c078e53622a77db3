// The two elementwise passes either side of the fused inner loop, each as one HBM-bound kernel.
//
// ttt_inner_inputs_kernel: everything TTT::get_inner_loop_inputs does after the projections
// (reference rust/layer/src/ttt.rs:147-194, 205-227, 247-268): head split [B,seq,H,d] ->
// [B,H,seq,d] of xq, xk, xv; rotary embedding of xq, xk (permute_qk -> rotate-half RoPE ->
// undo_permute_qk, ttt.rs:26-41 and rust/core/src/util.rs:349-392, which is a rotation of the
// ADJACENT pairs (x[2i], x[2i+1]) by pos * inv_freq[i]); ttt_lr_eta = base_lr * sigmoid(logit + bias) / d
// moved to [B,H,seq]; token_eta = max(token_idx + learnable_token_idx, 0) tiled over the sequence.
//
// ttt_layer_epilogue_kernel: TTT::forward after the inner model (ttt.rs:285-297): head merge
// [B,H,seq,d] -> [B,seq,H*d], post_norm LayerNorm over the hidden axis, times gelu_tanh(gate).
#pragma once
#include "ttt_engine.hip.h"

namespace ttt {

struct InnerInputsArgs {
  const void* xq;  // [B,seq,H,d] io
  const void* xk;
  const void* xv;
  const void* lr_logits;  // [B,seq,H] io
  const float* lr_bias;   // [H]
  const float* token_idx;            // [K]
  const float* learnable_token_idx;  // [K]
  const float* cos;  // [npos, d/2] or null: no rotary embedding
  const float* sin;
  void* xq_out;  // [B,H,seq,d] io
  void* xk_out;
  void* xv_out;
  void* lr_out;          // [B,H,seq] io
  float* token_eta_out;  // [seq]
  float lr_scale;        // base_lr / d
  int B, H, seq, D, K, pos_offset, pos_wrap;  // position of token t: (pos_offset + t) [% pos_wrap if > 0]
};

// One thread per 8 consecutive features of one (b, t, h): a 16-byte (bf16) or 32-byte (f32) chunk.
template <class T>
__global__ void __launch_bounds__(256) ttt_inner_inputs_kernel(InnerInputsArgs a) {
  using IO = Io<T>;
  using elem = typename IO::elem;
  const int cpr = a.D / 8;  // chunks per (b, t, h) row
  const size_t total = (size_t)a.B * a.seq * a.H * cpr;
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < (size_t)a.seq) {
    const int k = (int)(i % a.K);
    a.token_eta_out[i] = fmaxf(a.token_idx[k] + a.learnable_token_idx[k], 0.f);
  }
  if (i >= total) return;
  const int ch = (int)(i % cpr);
  const size_t r = i / cpr;  // (b, t, h) flattened in input order
  const int h = (int)(r % a.H);
  const size_t bt = r / a.H;
  const int t = (int)(bt % a.seq);
  const size_t b = bt / a.seq;
  const size_t src = r * a.D + 8 * ch;
  const size_t dst = ((b * a.H + h) * (size_t)a.seq + t) * a.D + 8 * ch;
  typename IO::frag lo, hi;
  // xv: head split only
  IO::load8(static_cast<const elem*>(a.xv) + src, true, lo, hi);
  IO::store8(static_cast<elem*>(a.xv_out) + dst, IO::to_f32(lo), IO::to_f32(hi));
  // xq, xk: head split + rotation of the four adjacent pairs of this chunk
  f32x4 cs = {1.f, 1.f, 1.f, 1.f}, sn = {0.f, 0.f, 0.f, 0.f};
  if (a.cos != nullptr) {
    int pos = a.pos_offset + t;
    if (a.pos_wrap > 0) pos %= a.pos_wrap;
    cs = *reinterpret_cast<const f32x4*>(a.cos + (size_t)pos * (a.D / 2) + 4 * ch);
    sn = *reinterpret_cast<const f32x4*>(a.sin + (size_t)pos * (a.D / 2) + 4 * ch);
  }
  auto rotate = [&](const void* in, void* out) {
    IO::load8(static_cast<const elem*>(in) + src, true, lo, hi);
    IO::store8(static_cast<elem*>(out) + dst, rope_rotate4(IO::to_f32(lo), f32x2{cs[0], cs[1]}, f32x2{sn[0], sn[1]}),
               rope_rotate4(IO::to_f32(hi), f32x2{cs[2], cs[3]}, f32x2{sn[2], sn[3]}));
  };
  rotate(a.xq, a.xq_out);
  rotate(a.xk, a.xk_out);
  if (ch == 0) {
    const float z = IO::load1(static_cast<const elem*>(a.lr_logits) + r) + a.lr_bias[h];
    IO::store1(static_cast<elem*>(a.lr_out) + (b * a.H + h) * (size_t)a.seq + t, lr_gate(z, a.lr_scale));
  }
}

struct LayerEpilogueArgs {
  const void* inner_out;  // [B,H,seq,d] io
  const float* gamma;     // [H*d]
  const float* beta;
  const void* gate;  // [B,seq,H*d] io or null
  void* out;         // [B,seq,H*d] io
  int B, H, seq, D;
  float eps;
};

// One wave per token (b, t): the H*d hidden values are gathered from the H head rows in chunks of
// 8, NC chunks per lane (hidden <= 512 * NC), normalised in registers and written as one row.
template <class T, int NC>
__global__ void __launch_bounds__(256) ttt_layer_epilogue_kernel(LayerEpilogueArgs a) {
  using IO = Io<T>;
  using elem = typename IO::elem;
  const int lane = threadIdx.x & 63;
  const size_t tok = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (tok >= (size_t)a.B * a.seq) return;
  const int t = (int)(tok % a.seq);
  const size_t b = tok / a.seq;
  const int hidden = a.H * a.D, nch = hidden / 8;
  f32x4 v[NC][2];
  typename IO::frag xlo[NC], xhi[NC], glo[NC], ghi[NC];
  float s = 0.f;
  // every load of the token is issued before the first use: the row statistics would otherwise
  // serialise the gate load behind two wave reductions
#pragma unroll
  for (int j = 0; j < NC; ++j) {
    const int ci = lane + 64 * j;
    const bool ok = ci < nch;
    const int f = 8 * (ok ? ci : 0), h = f / a.D, o = f - h * a.D;
    IO::load8(static_cast<const elem*>(a.inner_out) + ((b * a.H + h) * (size_t)a.seq + t) * a.D + o, ok, xlo[j], xhi[j]);
    IO::load8(static_cast<const elem*>(a.gate != nullptr ? a.gate : a.inner_out) + (a.gate != nullptr ? tok * hidden + f : 0),
              ok && a.gate != nullptr, glo[j], ghi[j]);
  }
#pragma unroll
  for (int j = 0; j < NC; ++j) {
    v[j][0] = IO::to_f32(xlo[j]);
    v[j][1] = IO::to_f32(xhi[j]);
#pragma unroll
    for (int r = 0; r < 4; ++r) s += v[j][0][r] + v[j][1][r];
  }
  auto wave_sum = [](float x) {
    return xg_sum(row16_sum_dpp(x));
  };
  const float mu = wave_sum(s) / hidden;
  float q = 0.f;
#pragma unroll
  for (int j = 0; j < NC; ++j)
    if (lane + 64 * j < nch)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        v[j][0][r] -= mu;
        v[j][1][r] -= mu;
        q += v[j][0][r] * v[j][0][r] + v[j][1][r] * v[j][1][r];
      }
  const float rstd = __builtin_amdgcn_rsqf(wave_sum(q) / hidden + a.eps);
#pragma unroll
  for (int j = 0; j < NC; ++j) {
    const int ci = lane + 64 * j;
    if (ci < nch) {
      const int f = 8 * ci;
      const f32x4 ga0 = *reinterpret_cast<const f32x4*>(a.gamma + f), ga1 = *reinterpret_cast<const f32x4*>(a.gamma + f + 4);
      const f32x4 be0 = *reinterpret_cast<const f32x4*>(a.beta + f), be1 = *reinterpret_cast<const f32x4*>(a.beta + f + 4);
      f32x4 y0 = ga0 * (v[j][0] * rstd) + be0, y1 = ga1 * (v[j][1] * rstd) + be1;
      if (a.gate != nullptr) {
        const f32x4 g0 = IO::to_f32(glo[j]), g1 = IO::to_f32(ghi[j]);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          y0[r] *= gelu_fast(g0[r]);
          y1[r] *= gelu_fast(g1[r]);
        }
      }
      IO::store8(static_cast<elem*>(a.out) + tok * hidden + f, y0, y1);
    }
  }
}

// Inputs of one layer of a stack: xq = x + pq, xk = x + pk, xv = x + pv (f32 sums rounded to the I/O type), x read
// once for all three.  One thread per 16 bytes.
struct LayerInputsArgs {
  const void *x, *pq, *pk, *pv;  // all pointing at the first token of the window in unit 0
  void *xq, *xk, *xv;
  size_t n16;      // number of 16-byte chunks to process: units * win16
  size_t win16;    // 16-byte chunks of one unit's window
  size_t pitch16;  // 16-byte chunks between consecutive (batch, head) units
};
template <class T>
__global__ void __launch_bounds__(256) ttt_layer_inputs_kernel(Problems<LayerInputsArgs> problems) {
  const LayerInputsArgs& a = problems.p[blockIdx.y];
  using IO = Io<T>;
  constexpr int E = 16 / IO::kBytes;  // elements per chunk
  const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= a.n16) return;
  const size_t i = (t / a.win16) * a.pitch16 + t % a.win16;
  const u32x4 rx = static_cast<const u32x4*>(a.x)[i];
  const u32x4 rq = static_cast<const u32x4*>(a.pq)[i], rk = static_cast<const u32x4*>(a.pk)[i],
              rv = static_cast<const u32x4*>(a.pv)[i];
  auto add = [&](u32x4 p) {
    u32x4 o;
    if (E == 4) {
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = __float_as_uint(__uint_as_float(rx[e]) + __uint_as_float(p[e]));
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float lo = __uint_as_float(rx[e] << 16) + __uint_as_float(p[e] << 16);
        const float hi = __uint_as_float(rx[e] & 0xffff0000u) + __uint_as_float(p[e] & 0xffff0000u);
        const bf16x2 r = __builtin_convertvector(f32x2{lo, hi}, bf16x2);
        o[e] = __builtin_bit_cast(uint32_t, r);
      }
    }
    return o;
  };
  static_cast<u32x4*>(a.xq)[i] = add(rq);
  static_cast<u32x4*>(a.xk)[i] = add(rk);
  static_cast<u32x4*>(a.xv)[i] = add(rv);
}

}  // namespace ttt
