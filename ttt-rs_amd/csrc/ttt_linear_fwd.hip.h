// TTT-Linear multi-stage forward for gfx950: one wavefront per (batch, head).
//
// Follows the arithmetic of TTTLinear::forward_mini_batch (reference
// rust/core/src/linear.rs:91-149) looped over mini-batches (rust/core/src/inner.rs:25-50),
// with the kernel-level behaviour of fused_ttt_forward_kernel_multi
// (rust/fused/src/linear_fused_tile/forward/kernel.rs:91-176): checkpoints hold the state
// entering a stage, token_eta is indexed by the position inside the mini-batch.
//
// Design (nothing here is taken from the reference's kernels):
//  * The f32 state W [d,d] never leaves registers: it is kept as NT x NT MFMA accumulator tiles
//    (NT = d/16), updated in place by the W -= XK^T (eta_last * G) contraction, and fed back
//    as the A operand of the next stage's XK.W / XQ.W contractions (see ttt_frag.hip.h for why
//    this needs no data movement).  There is no LDS use and no barrier.
//  * Everything elementwise is done "token-major": lane (c, g) owns token c and the features
//    {f(J, 4g+r)}; LayerNorm row statistics are 4*NT in-lane adds plus one reduction over the
//    four lane groups.  Activations come from HBM in exactly this layout (16-byte loads), are
//    prefetched PF stages ahead in registers, and the output leaves in it (16-byte stores).
//  * Two operands need tokens along k (the update's XK^T and G): they are transposed with one
//    MFMA against an identity fragment each.
#pragma once
#include "ttt_frag.hip.h"

namespace ttt {

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
  int B, H, seq, K, n_stages, ckpt_interval, n_ckpt, state_per_batch;
  float eps;
};

template <class T, int NT>
struct StageIn {
  typename Io<T>::frag q[NT], k[NT], v[NT];
  float lr;
};

// FULL: mini_batch == 16, so every lane has a token; a prefetch past the last stage re-reads the
// last stage instead of branching.
template <class T, int D, bool FULL>
__device__ __forceinline__ void load_stage(StageIn<T, D / 16>& s, const LinearFwdArgs& a, size_t bh,
                                           int stage, int c, int g) {
  using IO = Io<T>;
  using elem = typename IO::elem;
  constexpr int NT = D / 16;
  if (FULL) stage = min(stage, a.n_stages - 1);
  const bool ok = FULL || ((c < a.K) && (stage < a.n_stages));
  const size_t tok = bh * a.seq + (size_t)stage * a.K + c;
  const elem* pq = static_cast<const elem*>(a.xq) + tok * D + 8 * g;
  const elem* pk = static_cast<const elem*>(a.xk) + tok * D + 8 * g;
  const elem* pv = static_cast<const elem*>(a.xv) + tok * D + 8 * g;
#pragma unroll
  for (int q = 0; q < NT / 2; ++q) {
    IO::load8(pq + 32 * q, ok, s.q[2 * q], s.q[2 * q + 1]);
    IO::load8(pk + 32 * q, ok, s.k[2 * q], s.k[2 * q + 1]);
    IO::load8(pv + 32 * q, ok, s.v[2 * q], s.v[2 * q + 1]);
  }
  s.lr = ok ? IO::load1(static_cast<const elem*>(a.lr) + tok) : 0.f;
}

// In-lane sum of NT float4 followed by the cross-group reduction: a row sum over all d features.
template <int NT>
__device__ __forceinline__ float row_sum(const f32x4 (&v)[NT]) {
  float s = 0.f;
#pragma unroll
  for (int J = 0; J < NT; ++J) s += (v[J][0] + v[J][1]) + (v[J][2] + v[J][3]);
  return xg_sum(s);
}

template <class T, int D, int PF, bool FULL>
__global__ void __launch_bounds__(64) ttt_linear_fwd_kernel(LinearFwdArgs a) {
  using IO = Io<T>;
  using frag = typename IO::frag;
  using elem = typename IO::elem;
  constexpr int NT = D / 16;
  constexpr float inv_d = 1.0f / D;

  const int lane = threadIdx.x;
  const int c = lane & 15, g = lane >> 4;
  const size_t bh = blockIdx.x;  // = b*H + h
  const int h = (int)(bh % a.H);
  const int K = a.K;

  // ---- per-lane constants
  const float te_c = (c < K) ? a.token_eta[c] : 0.f;
  const float te_last = a.token_eta[K - 1];
  const frag ident = identity_frag<T>(c, g);
  const frag ones = splat_frag<T>(1.f);
  f32x4 gam[NT], bet[NT], bT[NT];
  const size_t sb = a.state_per_batch ? bh : (size_t)h;
#pragma unroll
  for (int J = 0; J < NT; ++J)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int f = feat(J, 4 * g + r);
      gam[J][r] = a.gamma[h * D + f];
      bet[J][r] = a.beta[h * D + f];
      bT[J][r] = a.b0[sb * D + f];
    }
  // ---- state: Wc[I][J][r] = W[feat(I,4g+r)][feat(J,c)]
  f32x4 Wc[NT][NT];
  {
    const float* W0 = a.W0 + sb * D * D;
#pragma unroll
    for (int I = 0; I < NT; ++I)
#pragma unroll
      for (int J = 0; J < NT; ++J)
#pragma unroll
        for (int r = 0; r < 4; ++r) Wc[I][J][r] = W0[feat(I, 4 * g + r) * D + feat(J, c)];
  }

  StageIn<T, NT> buf[PF];
#pragma unroll
  for (int u = 0; u < PF; ++u) load_stage<T, D, FULL>(buf[u], a, bh, u, c, g);

  for (int st0 = 0; st0 < a.n_stages; st0 += PF) {
#pragma unroll
    for (int u = 0; u < PF; ++u) {
      const int st = st0 + u;
      if (st >= a.n_stages) break;
      const StageIn<T, NT> cur = buf[u];
      load_stage<T, D, FULL>(buf[u], a, bh, st + PF, c, g);  // prefetch; consumed PF stages later

      // ---- checkpoint: state entering stage st
      if (a.W_ckpt != nullptr && (st % a.ckpt_interval) == 0) {
        const size_t ci = bh * a.n_ckpt + st / a.ckpt_interval;
        float* Wd = a.W_ckpt + ci * D * D;
#pragma unroll
        for (int I = 0; I < NT; ++I)
#pragma unroll
          for (int J = 0; J < NT; ++J)
#pragma unroll
            for (int r = 0; r < 4; ++r) Wd[feat(I, 4 * g + r) * D + feat(J, c)] = Wc[I][J][r];
        if (c == 0) {
          float* bd = a.b_ckpt + ci * D;
#pragma unroll
          for (int J = 0; J < NT; ++J)
#pragma unroll
            for (int r = 0; r < 4; ++r) bd[feat(J, 4 * g + r)] = bT[J][r];
        }
      }

      // ---- state as MFMA operand
      frag Wf[NT][NT];
#pragma unroll
      for (int I = 0; I < NT; ++I)
#pragma unroll
        for (int J = 0; J < NT; ++J) Wf[I][J] = IO::to_frag(Wc[I][J]);

      // Z1^T = b + W^T XK^T ; Zb^T = b + W^T XQ^T   (rows: features, columns: tokens)
      f32x4 z1[NT], zb[NT];
#pragma unroll
      for (int J = 0; J < NT; ++J) {
        z1[J] = bT[J];
        zb[J] = bT[J];
#pragma unroll
        for (int q = 0; q < NT / 2; ++q) {
          IO::mma2(z1[J], Wf[2 * q][J], Wf[2 * q + 1][J], cur.k[2 * q], cur.k[2 * q + 1]);
          IO::mma2(zb[J], Wf[2 * q][J], Wf[2 * q + 1][J], cur.q[2 * q], cur.q[2 * q + 1]);
        }
      }
      // At[r] = <xq_c, xk_s>, s = 4g+r  (attention scores, transposed: rows s, columns t=c)
      f32x4 At = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int q = 0; q < NT / 2; ++q)
        IO::mma2(At, cur.k[2 * q], cur.k[2 * q + 1], cur.q[2 * q], cur.q[2 * q + 1]);

      // ---- LayerNorm + L2 gradient on Z1 (util.rs:155-182), token-major
      f32x4 xh[NT], G[NT];
      {
        const float mu = row_sum<NT>(z1) * inv_d;
#pragma unroll
        for (int J = 0; J < NT; ++J) xh[J] = z1[J] - mu;
        f32x4 sq[NT];
#pragma unroll
        for (int J = 0; J < NT; ++J) sq[J] = xh[J] * xh[J];
        const float var = row_sum<NT>(sq) * inv_d;
        const float rstd = __builtin_amdgcn_rsqf(var + a.eps);
        f32x4 gx[NT], gxx[NT];
#pragma unroll
        for (int J = 0; J < NT; ++J) {
          xh[J] = xh[J] * rstd;
          const f32x4 tgt = IO::to_f32(cur.v[J]) - IO::to_f32(cur.k[J]);
          gx[J] = (gam[J] * xh[J] + bet[J] - tgt) * gam[J];
          gxx[J] = gx[J] * xh[J];
        }
        const float m1 = row_sum<NT>(gx) * inv_d;
        const float m2 = row_sum<NT>(gxx) * inv_d;
        // G scaled by this token's learning rate: eta_ij = te_i * lr_j, and lr_j belongs to
        // the token that produced row j of G (linear.rs:111-117)
        const float p = rstd * cur.lr;
#pragma unroll
        for (int J = 0; J < NT; ++J) G[J] = (gx[J] - m1 - xh[J] * m2) * p;
      }
      // ---- G with tokens along k: Gd[J][r] = lr_s G[s = 4g+r][feat(J,c)]
      frag Gd[NT];
#pragma unroll
      for (int J = 0; J < NT; ++J) {
        f32x4 t = {0.f, 0.f, 0.f, 0.f};
        IO::mma(t, IO::to_frag(G[J]), ident);
        Gd[J] = IO::to_frag(t);
      }
      // ---- causal correction: Zb^T -= Gd^T M^T,  M[t][s] = te_t (1 + A[t][s]) for s <= t
      {
        f32x4 m;
#pragma unroll
        for (int r = 0; r < 4; ++r) m[r] = (4 * g + r <= c) ? -te_c * (1.f + At[r]) : 0.f;
        const frag Mf = IO::to_frag(m);
#pragma unroll
        for (int J = 0; J < NT; ++J) IO::mma(zb[J], Gd[J], Mf);
      }
      // ---- out = XQ + LN(Zb)  (linear.rs:146-148)
      {
        const float mu = row_sum<NT>(zb) * inv_d;
        f32x4 sq[NT];
#pragma unroll
        for (int J = 0; J < NT; ++J) {
          zb[J] = zb[J] - mu;
          sq[J] = zb[J] * zb[J];
        }
        const float var = row_sum<NT>(sq) * inv_d;
        const float rstd = __builtin_amdgcn_rsqf(var + a.eps);
        if (FULL || c < K) {
          elem* po = static_cast<elem*>(a.out) + (bh * a.seq + (size_t)st * K + c) * D + 8 * g;
#pragma unroll
          for (int q = 0; q < NT / 2; ++q) {
            f32x4 o0 = IO::to_f32(cur.q[2 * q]) + (gam[2 * q] * (zb[2 * q] * rstd) + bet[2 * q]);
            f32x4 o1 = IO::to_f32(cur.q[2 * q + 1]) + (gam[2 * q + 1] * (zb[2 * q + 1] * rstd) + bet[2 * q + 1]);
            IO::store8(po + 32 * q, o0, o1);
          }
        }
      }
      // ---- state update: W -= te_last XK^T Gd ; b -= te_last colsum(Gd)   (linear.rs:134-144)
#pragma unroll
      for (int I = 0; I < NT; ++I) {
        f32x4 t = {0.f, 0.f, 0.f, 0.f};
        IO::mma(t, cur.k[I], ident);          // t[r] = XK[s = 4g+r][feat(I,c)]
        const frag kd = IO::to_frag(t * (-te_last));
#pragma unroll
        for (int J = 0; J < NT; ++J) IO::mma(Wc[I][J], kd, Gd[J]);
      }
#pragma unroll
      for (int J = 0; J < NT; ++J) {
        f32x4 s = {0.f, 0.f, 0.f, 0.f};
        IO::mma(s, Gd[J], ones);              // s[r] = sum_s Gd[s][feat(J,4g+r)], any column
        bT[J] = bT[J] - s * te_last;
      }
    }
  }

  // ---- final state
  {
    float* Wd = a.W_out + bh * D * D;
#pragma unroll
    for (int I = 0; I < NT; ++I)
#pragma unroll
      for (int J = 0; J < NT; ++J)
#pragma unroll
        for (int r = 0; r < 4; ++r) Wd[feat(I, 4 * g + r) * D + feat(J, c)] = Wc[I][J][r];
    if (c == 0) {
      float* bd = a.b_out + bh * D;
#pragma unroll
      for (int J = 0; J < NT; ++J)
#pragma unroll
        for (int r = 0; r < 4; ++r) bd[feat(J, 4 * g + r)] = bT[J][r];
    }
  }
}

}  // namespace ttt
