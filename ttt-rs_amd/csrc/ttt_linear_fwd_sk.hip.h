// TTT-Linear multi-stage forward for gfx950: the workgroup kernel of ttt_linear_fwd_mw.hip.h with
// the output path skewed by one mini-batch.
//
// Per mini-batch t a wave has two dependency chains:
//   recurrence  W_t -> Z1 -> LayerNorm statistics -> G -> W_{t+1}     (must finish before t+1 starts)
//   output      Zbar_t -> LayerNorm statistics -> out_t               (nothing waits for it)
// Each needs its own cross-wave exchange of row sums.  Here the output chain of mini-batch t-1 runs
// inside iteration t: its two sums travel in the same LDS exchange as the six sums of the
// recurrence (lane group g publishes sums g and g+4: eight in all), so there is ONE barrier per
// mini-batch, and between two barriers the instruction stream always holds two independent chains
// for the in-order issue to interleave.  The exchange buffer is double-buffered by parity because
// one barrier per iteration does not separate a fast wave's next write from a slow wave's read.
#pragma once
#include <type_traits>

#include "ttt_linear_fwd_mw.hip.h"

namespace ttt {

template <class T, int D, int NW, int PF, bool FULL, bool FAC = false>
__global__ void __launch_bounds__(64 * NW) ttt_linear_fwd_sk_kernel(Problems<LinearFwdArgs> problems) {
  const LinearFwdArgs& a = problems.p[blockIdx.y];
  using IO = Io<T>;
  using frag = typename IO::frag;
  using elem = typename IO::elem;
  constexpr int NT = D / 16, TPW = NT / NW;
  constexpr bool BF = sizeof(elem) == 2;
  constexpr float inv_d = 1.0f / D;
  static_assert(NW > 1, "the skewed kernel is for two or more waves per unit");
  __shared__ float ex[2][8 * 16 * NW];
  // f32 products with one feature tile per wave are bound by the f32 matrix instructions: the waves then share what
  // each would otherwise compute for itself.  Every wave transposes its own XK tile and forms the attention block over
  // its own 16 features; both cross LDS with the row sums (same barrier, same double buffering) and are read back
  // behind it: 8 matrix instructions per wave and mini-batch instead of 32.
  constexpr bool SHARE = !BF && TPW == 1;
  __shared__ f32x4 kdx[SHARE ? 2 : 1][SHARE ? NT : 1][64];
  __shared__ f32x4 atx[SHARE ? 2 : 1][SHARE ? NW : 1][64];

  const int lane = threadIdx.x & 63, w = (threadIdx.x >> 6) % NW;
  const int c = lane & 15, g = lane >> 4;
  const size_t bh = blockIdx.x;
  const int h = (int)(bh % a.H);
  const int K = a.K, n_stages_ = a.n_stages;
  const UnitBase<T, D> ub(a, bh);

  // same scale folding as the unskewed kernel: G'' = -sc lr G, M'' = (token_eta[t]/sc)(1 + A)
  const float te_last = a.token_eta[K - 1];
  const bool upd = te_last != 0.f;
  const float sc = upd ? te_last : 1.f;
  const float rho_c = (c < K) ? a.token_eta[c] / sc : 0.f;
  const frag ident = identity_frag<T>(c, g);
  const frag nident = identity_frag<T>(c, g, -1.f);
  const frag ones = splat_frag<T>(1.f);
  const size_t sb = a.state_per_batch ? bh : (size_t)h;
  f32x4 gam[TPW], bet[TPW], bT[TPW], a2[TPW];
  float sum_a = 0.f;
#pragma unroll
  for (int jj = 0; jj < TPW; ++jj)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int f = own_offset<TPW>(w, jj, g) + r;
      gam[jj][r] = a.gamma[h * D + f];
      bet[jj][r] = a.beta[h * D + f];
      bT[jj][r] = a.b0[sb * D + f];
      a2[jj][r] = gam[jj][r] * gam[jj][r];
    }
  for (int f = 0; f < D; ++f) sum_a += a.gamma[h * D + f] * a.gamma[h * D + f];
  f32x4 Wc[NT][TPW];
  {
    const float* W0 = a.W0 + sb * D * D;
#pragma unroll
    for (int I = 0; I < NT; ++I)
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj)
#pragma unroll
        for (int r = 0; r < 4; ++r) Wc[I][jj][r] = W0[feat(I, 4 * g + r) * D + feat(w * TPW + jj, c)];
  }
  // the kernel carries the centred state (see centre_state): row means in LDS, the exchange buffer as scratch
  __shared__ __attribute__((aligned(16))) float m0s[D + 4];
  static_assert(NW * D <= 2 * 8 * 16 * NW, "the exchange buffer doubles as scratch of centre_state");
  centre_state<D, NW, TPW>(Wc, bT, a.b0 + sb * D, m0s, &ex[0][0], w, c, g);

  // pending output of the previous mini-batch (its LayerNorm sums travel in the next exchange) and of the
  // one before (sums known: it is finished while the next exchange is in flight)
  f32x4 zbp[TPW], zbo[TPW];
  frag qop[TPW], qoo[TPW];
  float so0 = 0.f, so1 = 0.f;
#pragma unroll
  for (int jj = 0; jj < TPW; ++jj) {
    zbp[jj] = zbo[jj] = f32x4{0.f, 0.f, 0.f, 0.f};
    qop[jj] = qoo[jj] = IO::zero();
  }

  // publish this lane group's two sums ...
  auto exchange8_publish = [&](const float (&S)[8], int parity) {
    // lane group g ends up with sums g and g+4 reduced over the wave, and publishes them
    const float v0 = xg_sum4_scatter(S[0], S[1], S[2], S[3]);
    const float v1 = xg_sum4_scatter(S[4], S[5], S[6], S[7]);
    float* e = ex[parity];
    e[(g * 16 + c) * NW + w] = v0;
    e[((g + 4) * 16 + c) * NW + w] = v1;
  };
  // ... wait for the other waves, add up
  auto exchange8_collect = [&](float (&S)[8], int parity) {
    const float* e = ex[parity];
    lds_barrier();
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float s = 0.f;
#pragma unroll
      for (int ww = 0; ww < NW; ++ww) s += e[(i * 16 + c) * NW + ww];
      S[i] = s;
    }
  };
  auto exchange8 = [&](float (&S)[8], int parity) {
    exchange8_publish(S, parity);
    exchange8_collect(S, parity);
  };
  // In-lane sums of a pending Zbar.  One routine with explicit fused multiply-adds for every place that forms
  // them: a sequence processed in several calls must give the same bits as one call.
  auto pend_sums = [&](const f32x4 (&z)[TPW], float& s0, float& s1) {
    s0 = s1 = 0.f;
#pragma unroll
    for (int jj = 0; jj < TPW; ++jj)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        s0 += z[jj][r];
        s1 = __builtin_fmaf(z[jj][r], z[jj][r], s1);
      }
  };
  // out = xq + gamma (zbar - mu) rstd + beta for the pending mini-batch
  auto emit_output = [&](float s0, float s1, int stage, const f32x4 (&zbp)[TPW], const frag (&qop)[TPW]) {
    const float mu = s0 * inv_d;
    const float rstd = __builtin_amdgcn_rsqf(fmaxf(s1 * inv_d - mu * mu, 0.f) + a.eps);
    if (FULL || c < K) {
      elem* po = reinterpret_cast<elem*>(ub.out + UnitBase<T, D>::row_off(stage, K, c));
      f32x4 o[TPW];
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) {
        f32x4 qb;
        if (BF) {
          qb = bet[jj];
          IO::mma(qb, ident, qop[jj]);
        } else {
          qb = IO::to_f32(qop[jj]) + bet[jj];
        }
        o[jj] = qb + gam[jj] * ((zbp[jj] - mu) * rstd);
      }
      if (TPW == 1) {
        store4<T>(po + own_offset<TPW>(w, 0, g), o[0]);
      } else {
#pragma unroll
        for (int qq = 0; qq < TPW / 2; ++qq)
          IO::store8(po + own_offset<TPW>(w, 2 * qq, g), o[2 * qq], o[2 * qq + 1]);
      }
    }
  };

  // token_eta[K-1] == 0 means "no state update": instead of a branch inside the loop the two operands
  // that carry tokens into the update (XK^T, the ones column of the bias update) are made zero
  const frag ident_upd = upd ? ident : IO::zero();
  const frag ones_upd = upd ? ones : IO::zero();

  constexpr int R = PF + 1;
  StageInMw<T, NT, TPW> buf[R];
#pragma unroll
  for (int u = 0; u < PF; ++u) load_stage_mw<T, D, NW, FULL>(buf[u], ub, K, n_stages_, u, c, g, w);

  // One pass over R mini-batches (the ring of prefetch registers is indexed at compile time).  CHECKED:
  // the first and the last pass, which test for "no pending output yet" and "past the end"; the passes in
  // between run without any branch, so that everything between two barriers -- the tail of one mini-batch
  // (pending output, G, state update) and the head of the next (products, moments) -- is one basic block and
  // the compiler can interleave the two dependency chains.
  float ps0 = 0.f, ps1 = 0.f;
  CkptCursor<D> ck(a, bh);
  const float b_mean = __builtin_amdgcn_readfirstlane(m0s[D]);  // mean of the initial bias (split off by centre_state)
  static_assert(!FAC || BF, "update factors are saved with bf16 I/O only");
  unsigned char* fac = FAC ? factor_base<D>(a.W_ckpt, a.n_ckpt, bh) : nullptr;
  auto pass = [&](auto checked_tag, int st0) {
    constexpr bool CHECKED = decltype(checked_tag)::value;
#pragma unroll
    for (int u = 0; u < R; ++u) {
      const int st = st0 + u;
      load_stage_mw<T, D, NW, FULL>(buf[(u + PF) % R], ub, K, n_stages_, st + PF, c, g, w);
      if (CHECKED && st >= a.n_stages) continue;
      const StageInMw<T, NT, TPW>& cur = buf[u];

      // ---- XK with tokens along k for the state update: depends on nothing computed here, so it
      // is issued first and fills the gaps of the dependent chain below
      frag kd[NT];
      if constexpr (SHARE) {
        f32x4 t = {0.f, 0.f, 0.f, 0.f};
        IO::mma(t, cur.ko[0], ident_upd);  // the own tile; the others come back from LDS behind the barrier
        kdx[st & 1][w][lane] = t;
      } else {
#pragma unroll
        for (int I = 0; I < NT; ++I) {
          f32x4 t = {0.f, 0.f, 0.f, 0.f};
          IO::mma(t, cur.k[I], ident_upd);  // t[r] = XK[s = 4g+r][feat(I,c)]
          kd[I] = IO::to_frag(t);
        }
      }
      // ---- Z1^T, Zbar^T (this wave's feature rows) and the attention block
      f32x4 z1[TPW], zb[TPW], At = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) {
        z1[jj] = bT[jj];
        zb[jj] = bT[jj];
      }
#pragma unroll
      for (int q = 0; q < NT / 2; ++q) {
#pragma unroll
        for (int jj = 0; jj < TPW; ++jj) {
          const frag w0 = IO::to_frag(Wc[2 * q][jj]), w1 = IO::to_frag(Wc[2 * q + 1][jj]);
          IO::mma2(z1[jj], w0, w1, cur.k[2 * q], cur.k[2 * q + 1]);
          IO::mma2(zb[jj], w0, w1, cur.q[2 * q], cur.q[2 * q + 1]);
        }
        if constexpr (!SHARE) IO::mma2(At, cur.k[2 * q], cur.k[2 * q + 1], cur.q[2 * q], cur.q[2 * q + 1]);
      }
      if constexpr (SHARE) {
        IO::mma(At, cur.ko[0], cur.qo[0]);  // over the own 16 features
        atx[st & 1][w][lane] = At;
      }
      // ---- row sums: six raw moments of Z1 (this mini-batch), two of the pending Zbar
      f32x4 bq[TPW];
      float S[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, ps0, ps1};  // the pending Zbar's in-lane sums are ready
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) {
        f32x4 uu;  // beta - (xv - xk)
        if (BF) {
          uu = bet[jj];
          IO::mma2(uu, nident, ident, cur.vo[jj], cur.ko[jj]);
        } else {
          uu = bet[jj] - (IO::to_f32(cur.vo[jj]) - IO::to_f32(cur.ko[jj]));
        }
        bq[jj] = gam[jj] * uu;
        const f32x4 az = a2[jj] * z1[jj];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          S[0] += z1[jj][r];
          S[1] += z1[jj][r] * z1[jj][r];
          S[2] += az[r];
          S[3] += az[r] * z1[jj][r];
          S[4] += bq[jj][r];
          S[5] += bq[jj][r] * z1[jj][r];
        }
      }
      // ---- checkpoint of the state entering this mini-batch (W and b change only behind the barrier);
      // placed at the barrier so that its branch does not cut the stretch in two
      if (ck.due()) {
        if (ck.packed) {
          store_ckpt_packed<T, NT, TPW>(ck.W, Wc, w, lane);
          store_bias_true<D, TPW>(ck.b, bT, b_mean, w, c, g);
        } else {
          store_state_f32<D, TPW>(ck.W, ck.b, Wc, bT, m0s, w, c, g);
        }
        ck.advance();
      }
      ck.next_stage();
      exchange8_publish(S, st & 1);
      // ---- the output pending since two mini-batches (sums known since the last exchange): nothing waits
      // for it, and here it runs while this exchange is in flight (LDS write, barrier, LDS read)
      if (!CHECKED || st > 1) emit_output(so0, so1, st - 2, zbo, qoo);
      exchange8_collect(S, st & 1);
      so0 = S[6];
      so1 = S[7];
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) {
        zbo[jj] = zbp[jj];
        qoo[jj] = qop[jj];
      }
      if constexpr (SHARE) {
#pragma unroll
        for (int I = 0; I < NT; ++I) kd[I] = IO::to_frag(kdx[st & 1][I][lane]);
        At = atx[st & 1][0][lane];
#pragma unroll
        for (int ww = 1; ww < NW; ++ww) At += atx[st & 1][ww][lane];
      }

      // ---- recurrence: G'' , causal correction, state update
      f32x4 G[TPW];
      {
        const float mu = S[0] * inv_d;
        const float var = S[1] * inv_d - mu * mu;
        const float rstd = __builtin_amdgcn_rsqf(fmaxf(var, 0.f) + a.eps);
        const float s1 = rstd * (S[2] - mu * sum_a) + S[4];
        const float s2 = rstd * rstd * (S[3] - 2.f * mu * S[2] + mu * mu * sum_a) + rstd * (S[5] - mu * S[4]);
        const float p = -sc * cur.lr * rstd;
        const float c1 = p * rstd, c2 = -c1 * s2 * inv_d, c3 = -p * s1 * inv_d;
#pragma unroll
        for (int jj = 0; jj < TPW; ++jj) G[jj] = (z1[jj] - mu) * (a2[jj] * c1 + c2) + (bq[jj] * p + c3);
      }
      frag Gd[TPW];
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) {
        f32x4 t = {0.f, 0.f, 0.f, 0.f};
        IO::mma(t, IO::to_frag(G[jj]), ident);
        Gd[jj] = IO::to_frag(t);
      }
      if constexpr (FAC) {
        store_factor<TPW>(fac, Gd, w, lane);
        fac += 32 * D;
      }
      {
        f32x4 m;
#pragma unroll
        for (int r = 0; r < 4; ++r) m[r] = (4 * g + r <= c) ? rho_c * (1.f + At[r]) : 0.f;
        const frag Mf = IO::to_frag(m);
#pragma unroll
        for (int jj = 0; jj < TPW; ++jj) IO::mma(zb[jj], Gd[jj], Mf);
      }
#pragma unroll
      for (int I = 0; I < NT; ++I)
#pragma unroll
        for (int jj = 0; jj < TPW; ++jj) IO::mma(Wc[I][jj], kd[I], Gd[jj]);
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) IO::mma(bT[jj], Gd[jj], ones_upd);
      // this mini-batch's Zbar and xq become the pending output; its in-lane sums are formed here, in the
      // shadow of the state update, not between the next Z1 and its exchange
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) {
        zbp[jj] = zb[jj];
        qop[jj] = cur.qo[jj];
      }
      pend_sums(zbp, ps0, ps1);
    }
  };
  if constexpr (NT <= 4) {
    int st0 = 0;
    pass(std::true_type{}, st0);
    for (st0 = R; st0 + R <= a.n_stages; st0 += R) pass(std::false_type{}, st0);
    if (st0 < a.n_stages) pass(std::true_type{}, st0);
  } else {
    // Wide heads (d = 96, 128) keep the loop with its branches: in one long basic block the scheduler overlaps
    // so much that the state tiles no longer fit the register file (d = 128: 30 spilled registers).
    for (int st0 = 0; st0 < a.n_stages; st0 += R) {
#pragma unroll
      for (int u = 0; u < R; ++u) {
        const int st = st0 + u;
        load_stage_mw<T, D, NW, FULL>(buf[(u + PF) % R], ub, K, n_stages_, st + PF, c, g, w);
        if (st >= a.n_stages) continue;
        const StageInMw<T, NT, TPW>& cur = buf[u];

        if (ck.due()) {
          if (ck.packed) {
            store_ckpt_packed<T, NT, TPW>(ck.W, Wc, w, lane);
            store_bias_true<D, TPW>(ck.b, bT, b_mean, w, c, g);
          } else {
            store_state_f32<D, TPW>(ck.W, ck.b, Wc, bT, m0s, w, c, g);
          }
          ck.advance();
        }
        ck.next_stage();

        // ---- XK with tokens along k for the state update: depends on nothing computed here, so it
        // is issued first and fills the gaps of the dependent chain below
        frag kd[NT];
#pragma unroll
        for (int I = 0; I < NT; ++I) {
          f32x4 t = {0.f, 0.f, 0.f, 0.f};
          IO::mma(t, cur.k[I], ident);  // t[r] = XK[s = 4g+r][feat(I,c)]
          kd[I] = IO::to_frag(t);
        }
        // ---- Z1^T, Zbar^T (this wave's feature rows) and the attention block
        f32x4 z1[TPW], zb[TPW], At = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int jj = 0; jj < TPW; ++jj) {
          z1[jj] = bT[jj];
          zb[jj] = bT[jj];
        }
#pragma unroll
        for (int q = 0; q < NT / 2; ++q) {
#pragma unroll
          for (int jj = 0; jj < TPW; ++jj) {
            const frag w0 = IO::to_frag(Wc[2 * q][jj]), w1 = IO::to_frag(Wc[2 * q + 1][jj]);
            IO::mma2(z1[jj], w0, w1, cur.k[2 * q], cur.k[2 * q + 1]);
            IO::mma2(zb[jj], w0, w1, cur.q[2 * q], cur.q[2 * q + 1]);
          }
          IO::mma2(At, cur.k[2 * q], cur.k[2 * q + 1], cur.q[2 * q], cur.q[2 * q + 1]);
        }
        // ---- row sums: six raw moments of Z1 (this mini-batch), two of the pending Zbar
        f32x4 bq[TPW];
        float S[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int jj = 0; jj < TPW; ++jj) {
          f32x4 uu;  // beta - (xv - xk)
          if (BF) {
            uu = bet[jj];
            IO::mma2(uu, nident, ident, cur.vo[jj], cur.ko[jj]);
          } else {
            uu = bet[jj] - (IO::to_f32(cur.vo[jj]) - IO::to_f32(cur.ko[jj]));
          }
          bq[jj] = gam[jj] * uu;
          const f32x4 az = a2[jj] * z1[jj];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            S[0] += z1[jj][r];
            S[1] += z1[jj][r] * z1[jj][r];
            S[2] += az[r];
            S[3] += az[r] * z1[jj][r];
            S[4] += bq[jj][r];
            S[5] += bq[jj][r] * z1[jj][r];
          }
        }
        pend_sums(zbp, S[6], S[7]);
        exchange8_publish(S, st & 1);
        if (st > 1) emit_output(so0, so1, st - 2, zbo, qoo);  // inside the exchange window, as above
        exchange8_collect(S, st & 1);
        so0 = S[6];
        so1 = S[7];
#pragma unroll
        for (int jj = 0; jj < TPW; ++jj) {
          zbo[jj] = zbp[jj];
          qoo[jj] = qop[jj];
        }

        // ---- recurrence: G'' , causal correction, state update
        f32x4 G[TPW];
        {
          const float mu = S[0] * inv_d;
          const float var = S[1] * inv_d - mu * mu;
          const float rstd = __builtin_amdgcn_rsqf(fmaxf(var, 0.f) + a.eps);
          const float s1 = rstd * (S[2] - mu * sum_a) + S[4];
          const float s2 = rstd * rstd * (S[3] - 2.f * mu * S[2] + mu * mu * sum_a) + rstd * (S[5] - mu * S[4]);
          const float p = -sc * cur.lr * rstd;
          const float c1 = p * rstd, c2 = -c1 * s2 * inv_d, c3 = -p * s1 * inv_d;
#pragma unroll
          for (int jj = 0; jj < TPW; ++jj) G[jj] = (z1[jj] - mu) * (a2[jj] * c1 + c2) + (bq[jj] * p + c3);
        }
        frag Gd[TPW];
#pragma unroll
        for (int jj = 0; jj < TPW; ++jj) {
          f32x4 t = {0.f, 0.f, 0.f, 0.f};
          IO::mma(t, IO::to_frag(G[jj]), ident);
          Gd[jj] = IO::to_frag(t);
        }
        if constexpr (FAC) {
          store_factor<TPW>(fac, Gd, w, lane);
          fac += 32 * D;
        }
        {
          f32x4 m;
#pragma unroll
          for (int r = 0; r < 4; ++r) m[r] = (4 * g + r <= c) ? rho_c * (1.f + At[r]) : 0.f;
          const frag Mf = IO::to_frag(m);
#pragma unroll
          for (int jj = 0; jj < TPW; ++jj) IO::mma(zb[jj], Gd[jj], Mf);
        }
        if (upd) {
#pragma unroll
          for (int I = 0; I < NT; ++I)
#pragma unroll
            for (int jj = 0; jj < TPW; ++jj) IO::mma(Wc[I][jj], kd[I], Gd[jj]);
#pragma unroll
          for (int jj = 0; jj < TPW; ++jj) IO::mma(bT[jj], Gd[jj], ones);
        }
        // this mini-batch's Zbar and xq become the pending output
#pragma unroll
        for (int jj = 0; jj < TPW; ++jj) {
          zbp[jj] = zb[jj];
          qop[jj] = cur.qo[jj];
        }
      }
    }

  }

  // ---- flush the last mini-batch's output
  {
    float S[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    pend_sums(zbp, S[6], S[7]);
    exchange8(S, a.n_stages & 1);
    if (a.n_stages >= 2) emit_output(so0, so1, a.n_stages - 2, zbo, qoo);
    emit_output(S[6], S[7], a.n_stages - 1, zbp, qop);
  }
  store_state_final<D, TPW>(a.W_out + bh * D * D, a.b_out + bh * D, a.W0 + sb * D * D, a.b0 + sb * D, Wc, bT, m0s, w, c, g);
  if constexpr (FAC)
    store_state_tiles<D, TPW>(a.W_ckpt + bh * (size_t)a.n_ckpt * (D * D), a.b_ckpt + bh * (size_t)a.n_ckpt * D, Wc, bT, w, lane);
}

}  // namespace ttt
