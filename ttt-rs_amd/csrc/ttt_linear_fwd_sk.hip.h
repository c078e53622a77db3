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

// RAW = 0: the operands are given (xq, xk, xv [B,H,seq,d], lr, token_eta of LinearFwdArgs).
// RAW > 0: the kernel forms them from the projections (FusedInputsArgs: head split by addressing, rotary embedding
// of xq and xk, lr gate, token_eta), i.e. it does the work of ttt_inner_inputs_kernel inside its tile loads:
//   * a wave loads only the features it owns of the raw xq, xk, xv rows (strided [B,seq,H,d] rows), three
//     mini-batches ahead, rotates its xq and xk features in the shadow of the state update two mini-batches ahead
//     of their use, and puts them into LDS; behind the next barrier (the one the recurrence has anyway) every wave
//     reads the full rotated rows back.  The rotation is therefore done once per unit, not once per wave, and no
//     barrier is added;
//   * RAW = 1: the position of a token repeats with the mini-batch (pos_wrap divides K: the reference's default),
//     cosines and sines stay in registers; RAW = 2: positions run over the sequence (pos_wrap = 0), cosines and sines
//     are loaded with the rows;
//   * the operands as used (rotated xq, xk; xv; lr) are written out in [B,H,seq,d] order when the caller asks for them
//     (ttt_linear_bwd needs them): the wave that owns a feature stores it.
// RAW = 3: the operands are given, and fetched the same way: every wave loads only the features it owns and the
// full xq, xk rows reach the waves through LDS (half the vector loads of RAW = 0, where every wave loads every row).
// RAW = 4: as RAW = 3 with the operands formed as x + xq, x + xk, x + xv (LinearFwdArgs::xin: a layer of a stack whose
// input is the output of the layer below plus its own projections); x may be the memory `out` is written to: a wave
// reads a row's own features three mini-batches before it writes that row's own features, and no other wave
// touches them.
// RAW = 5: the operands are given, and a CONTROL WAVE beside the NW compute waves brings them in: it copies the rows of
// xq, xk, xv and lr of a mini-batch global -> LDS without passing registers (one 1 KiB row per feature tile and
// tensor, 16 bytes per lane: exactly the fragment that lane holds of the tile), four mini-batches ahead into a ring of
// four slots, and takes part in every barrier.  The compute waves issue no global load at all: behind the barrier of a
// mini-batch they read the next one's fragments from LDS.  (A load costs the wave that issues it up to a hundred
// cycles of stalled issue, nine of them per wave and mini-batch with f32 I/O.)  For f32 I/O with one feature tile per
// wave, where a unit has a CU to itself (the control wave shares a SIMD with a compute wave: the kernel must stay
// within 256 registers) and whole mini-batches of 16 tokens.
// ADAM: the state update W -= XK^T (eta_last G) is replaced by one Adam step on that gradient per mini-batch
// (reference rust/core/src/linear_adam.rs:76-128): the gradient tile is formed by the same matrix instructions into a
// zero accumulator, the moments live in registers beside the state (three times the state's registers), bias
// corrections come from running powers of beta1, beta2.  Everything else -- products, LayerNorm, output -- is the
// plain kernel's; the output of a mini-batch does not see its own update in either.
template <class T, int D, int NW, int PF, bool FULL, bool FAC, int RAW, bool ADAM = false>
__device__ __forceinline__ void linear_fwd_sk_body(const LinearFwdArgs& a, const FusedInputsArgs* fip,
                                                   const AdamArgs* adam = nullptr) {
  static_assert(!ADAM || (D <= 64 && !FAC && RAW == 0), "Adam inner optimiser: head_dim <= 64, no checkpoints");
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

  constexpr bool DMA = RAW == 5;
  const int lane = threadIdx.x & 63, w = (threadIdx.x >> 6) % NW;
  // RAW = 5: the wave behind the compute waves is the control wave; up to the point where it branches off it does what
  // wave 0 does (w == 0: valid loads, LDS writes of the same values) and it stores nothing
  const bool ctlw = DMA && __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)) == NW;
  const int c = lane & 15, g = lane >> 4;
  const size_t bh = blockIdx.x;
  const int h = (int)(bh % a.H);
  const int K = a.K, n_stages_ = a.n_stages;
  const UnitBase<T, D> ub(a, bh);

  // same scale folding as the unskewed kernel: G'' = -sc lr G, M'' = (token_eta[t]/sc)(1 + A)
  constexpr bool FORM = RAW == 1 || RAW == 2;  // the operands are formed here from the projections
  auto tok_eta = [&](int i) {
    if constexpr (FORM) return fmaxf(fip->token_idx[i] + fip->learnable_token_idx[i], 0.f);
    else return a.token_eta[i];
  };
  const float te_last = tok_eta(K - 1);
  const bool upd = te_last != 0.f;
  const float sc = upd ? te_last : 1.f;
  const float rho_c = (c < K) ? tok_eta(c) / sc : 0.f;
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

  // ADAM: first and second moments of this wave's W tiles and bias rows, and the running powers beta^step
  f32x4 Wm[ADAM ? NT : 1][TPW], Wv[ADAM ? NT : 1][TPW], bm[TPW], bv[TPW];
  float pw1 = 1.f, pw2 = 1.f;
  if constexpr (ADAM) {
    const bool have = adam->Wm0 != nullptr;
#pragma unroll
    for (int I = 0; I < NT; ++I)
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const size_t at = bh * D * D + feat(I, 4 * g + r) * D + feat(w * TPW + jj, c);
          Wm[I][jj][r] = have ? adam->Wm0[at] : 0.f;
          Wv[I][jj][r] = have ? adam->Wv0[at] : 0.f;
        }
#pragma unroll
    for (int jj = 0; jj < TPW; ++jj)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const size_t at = bh * D + own_offset<TPW>(w, jj, g) + r;
        bm[jj][r] = have ? adam->bm0[at] : 0.f;
        bv[jj][r] = have ? adam->bv0[at] : 0.f;
      }
    for (int i = 0; i < adam->step0; ++i) {
      pw1 *= adam->beta1;
      pw2 *= adam->beta2;
    }
  }
  // one Adam step on a tile: gneg = -gradient (what the plain kernel would add to the state)
  float ad_a1 = 0.f, ad_ic2 = 0.f;  // lr / (1 - beta1^t), 1 / (1 - beta2^t) of the current step
  auto adam_tile = [&](f32x4& x, f32x4& m, f32x4& v, f32x4 gneg) {
    if constexpr (ADAM) {
      const float b1 = adam->beta1, b2 = adam->beta2;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float gr = -gneg[r];
        m[r] = __builtin_fmaf(b1, m[r], (1.f - b1) * gr);
        v[r] = __builtin_fmaf(b2, v[r], (1.f - b2) * (gr * gr));
        const float den = __builtin_amdgcn_sqrtf(v[r] * ad_ic2) + adam->eps;  // 1 ulp; v is far above the denormals
        x[r] = __builtin_fmaf(-(ad_a1 * m[r]), __builtin_amdgcn_rcpf(den), x[r]);
      }
    }
  };
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

  // b += colsum G''.  The bias is the accumulator input of the next mini-batch's Z1 and Zbar products, which are
  // k = 32 matrix instructions with bf16 I/O, and the scheduler is free to place them right behind this k = 16 update:
  // a matrix instruction that takes its accumulator from one of ANOTHER shape less than five wait states earlier
  // reads a stale value (the hardware interlocks only equal shapes; measured, see ttt_selftest.hip.h).  The wait
  // states are therefore put behind the update by hand, tied to the bias registers so that no reader of the bias can
  // be scheduled in front of them: nothing measurable at any size.  (Issuing the update as a k = 32 instruction with
  // a zero half, the other way to make the shapes equal, cost 10 % of the kernel's time at every size.)  In most
  // instantiations the scheduler leaves the W update's matrix instructions between the pair anyway; the one that had
  // them adjacent gave outputs 1 % off from the sixth mini-batch on.  The build's assembly scan (isa_check.py) refuses
  // any code in which such a pair is closer than five wait states.
  auto bias_update = [&](f32x4 (&b)[TPW], const frag (&gd)[TPW], frag ones_or_zero) {
#pragma unroll
    for (int jj = 0; jj < TPW; ++jj) IO::mma(b[jj], gd[jj], ones_or_zero);
    if constexpr (BF) {
      if constexpr (TPW == 1) asm volatile("s_nop 4" : "+v"(b[0]));
      else if constexpr (TPW == 2) asm volatile("s_nop 4" : "+v"(b[0]), "+v"(b[1]));
      else
#pragma unroll
        for (int jj = 0; jj < TPW; ++jj) asm volatile("s_nop 4" : "+v"(b[jj]));
    }
  };
  // token_eta[K-1] == 0 means "no state update": instead of a branch inside the loop the two operands
  // that carry tokens into the update (XK^T, the ones column of the bias update) are made zero
  const frag ident_upd = upd ? ident : IO::zero();
  const frag ones_upd = upd ? ones : IO::zero();

  constexpr int R = PF + 1;
  StageInMw<T, NT, TPW> buf[R];
  // ---- RAW: the raw rows of the own features, three mini-batches ahead (ring index = mini-batch % R, as for buf)
  struct RawIn {
    frag q[TPW], k[TPW], v[TPW];
    frag x[TPW];                // RAW = 4 only
    float z;                    // lr logit of the lane's token
    f32x2 cs[TPW], sn[TPW];     // RAW = 2 only
  };
  RawIn raw[RAW != 0 ? R : 1];
  f32x2 cs_fix[TPW], sn_fix[TPW];  // RAW = 1: cosines and sines of the lane's token position and own feature pairs
  u32x4* xrot = nullptr;           // rotated rows in LDS: [2 buffers][xq, xk][feature pair][lane]
  float lr_bias_h = 0.f;
  if constexpr (RAW != 0 && !DMA) {
    static_assert(BF && PF == 2, "rows shared through LDS: bf16 I/O");
    static_assert(!FORM || NT <= 4, "operands formed from the projections: head_dim <= 64");
    __shared__ u32x4 xrot_s[2][2][NT / 2][64];
    xrot = &xrot_s[0][0][0][0];
#pragma unroll
    for (int jj = 0; jj < TPW; ++jj) {
      cs_fix[jj] = f32x2{1.f, 1.f};
      sn_fix[jj] = f32x2{0.f, 0.f};
    }
  }
  if constexpr (FORM) {
    lr_bias_h = fip->lr_bias[h];
    if (RAW == 1 && fip->cos != nullptr) {
      const int pos = (fip->pos_offset + c) % fip->pos_wrap;
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) {
        const size_t o = (size_t)pos * (D / 2) + own_offset<TPW>(w, jj, g) / 2;
        cs_fix[jj] = *reinterpret_cast<const f32x2*>(fip->cos + o);
        sn_fix[jj] = *reinterpret_cast<const f32x2*>(fip->sin + o);
      }
    }
    if (fip->token_eta_out != nullptr && bh == 0)
      for (int i = threadIdx.x; i < a.seq; i += 64 * NW) fip->token_eta_out[i] = tok_eta(i % K);
  }
  const bool has_x = a.xin != nullptr;  // RAW = 4: a problem without x takes the operands as they are (x = 0)
  // raw rows of unit (b, h): token t of the unit is row (b * seq + t) * H + h of the [B,seq,H,d] tensors
  const size_t bidx = bh / a.H;
  const unsigned raw_row = (unsigned)a.H * (unsigned)(D * sizeof(elem));  // bytes from one token to the next
  auto load_raw = [&](RawIn& r, int stage) {
    if constexpr (RAW != 0 && !DMA) {
      if (FULL) stage = min(stage, n_stages_ - 1);
      const bool ok = FULL || ((c < K) && (stage < n_stages_));
      const unsigned t = (unsigned)stage * (unsigned)K + (unsigned)c;
      const unsigned char *bq, *bk, *bv;
      unsigned off;
      if constexpr (FORM) {
        const size_t row0 = (bidx * (size_t)a.seq * a.H + h) * (D * sizeof(elem));
        bq = static_cast<const unsigned char*>(fip->xq) + row0;
        bk = static_cast<const unsigned char*>(fip->xk) + row0;
        bv = static_cast<const unsigned char*>(fip->xv) + row0;
        off = t * raw_row;
      } else {
        bq = ub.xq;
        bk = ub.xk;
        bv = ub.xv;
        off = UnitBase<T, D>::row_off(stage, K, c);
      }
      if (TPW == 1) {
        const unsigned o1 = off + own_offset<TPW>(w, 0, g) * (unsigned)sizeof(elem);
        r.q[0] = ok ? load4<T>(reinterpret_cast<const elem*>(bq + o1)) : IO::zero();
        r.k[0] = ok ? load4<T>(reinterpret_cast<const elem*>(bk + o1)) : IO::zero();
        r.v[0] = ok ? load4<T>(reinterpret_cast<const elem*>(bv + o1)) : IO::zero();
        if constexpr (RAW == 4) r.x[0] = (ok && has_x) ? load4<T>(reinterpret_cast<const elem*>(ub.xin + o1)) : IO::zero();
      } else {
#pragma unroll
        for (int qq = 0; qq < TPW / 2; ++qq) {
          const unsigned o2 = off + own_offset<TPW>(w, 2 * qq, g) * (unsigned)sizeof(elem);
          IO::load8(reinterpret_cast<const elem*>(bq + o2), ok, r.q[2 * qq], r.q[2 * qq + 1]);
          IO::load8(reinterpret_cast<const elem*>(bk + o2), ok, r.k[2 * qq], r.k[2 * qq + 1]);
          IO::load8(reinterpret_cast<const elem*>(bv + o2), ok, r.v[2 * qq], r.v[2 * qq + 1]);
          if constexpr (RAW == 4) IO::load8(reinterpret_cast<const elem*>(ub.xin + o2), ok && has_x, r.x[2 * qq], r.x[2 * qq + 1]);
        }
      }
      if constexpr (FORM) {
        const elem* zl = static_cast<const elem*>(fip->lr_logits) + (bidx * (size_t)a.seq * a.H + h);
        r.z = ok ? IO::load1(zl + (size_t)t * a.H) : 0.f;
      } else {
        r.z = ok ? IO::load1(reinterpret_cast<const elem*>(ub.lr + t * (unsigned)sizeof(elem))) : 0.f;  // lr itself
      }
      if constexpr (RAW == 2) {
#pragma unroll
        for (int jj = 0; jj < TPW; ++jj) {
          const size_t o = (size_t)(fip->pos_offset + (int)t) * (D / 2) + own_offset<TPW>(w, jj, g) / 2;
          r.cs[jj] = fip->cos != nullptr ? *reinterpret_cast<const f32x2*>(fip->cos + o) : f32x2{1.f, 1.f};
          r.sn[jj] = fip->sin != nullptr ? *reinterpret_cast<const f32x2*>(fip->sin + o) : f32x2{0.f, 0.f};
        }
      }
    }
  };
  // own features of a mini-batch: rotate, keep (own-feature operands of dst), share through LDS buffer `pb`, store
  auto rotate_share = [&](const RawIn& r, StageInMw<T, NT, TPW>& dst, int stage, int pb) {
    if constexpr (RAW != 0 && !DMA) {
      const bool tok = FULL || c < K;
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) {
        if constexpr (FORM) {
          const f32x2 cs = RAW == 2 ? r.cs[jj] : cs_fix[jj], sn = RAW == 2 ? r.sn[jj] : sn_fix[jj];
          dst.qo[jj] = IO::to_frag(rope_rotate4(IO::to_f32(r.q[jj]), cs, sn));
          dst.ko[jj] = IO::to_frag(rope_rotate4(IO::to_f32(r.k[jj]), cs, sn));
          dst.vo[jj] = r.v[jj];
        } else if constexpr (RAW == 4) {
          const f32x4 x = IO::to_f32(r.x[jj]);
          dst.qo[jj] = IO::to_frag(x + IO::to_f32(r.q[jj]));
          dst.ko[jj] = IO::to_frag(x + IO::to_f32(r.k[jj]));
          dst.vo[jj] = IO::to_frag(x + IO::to_f32(r.v[jj]));
        } else {
          dst.qo[jj] = r.q[jj];
          dst.ko[jj] = r.k[jj];
          dst.vo[jj] = r.v[jj];
        }
      }
      // the gate in the precision the operand has when it is a tensor of its own
      // (a token past the end of a short mini-batch has no learning rate: it must not reach the state update)
      if constexpr (FORM) dst.lr = tok ? IO::rounded(lr_gate(r.z + lr_bias_h, fip->lr_scale)) : 0.f;
      else dst.lr = r.z;
      u32x4* xb = xrot + (size_t)pb * 2 * (NT / 2) * 64;
      if (TPW == 1) {
        const int J = w;
        unsigned char* pq_ = reinterpret_cast<unsigned char*>(xb + (0 * (NT / 2) + (J >> 1)) * 64 + lane) + 8 * (J & 1);
        unsigned char* pk_ = reinterpret_cast<unsigned char*>(xb + (1 * (NT / 2) + (J >> 1)) * 64 + lane) + 8 * (J & 1);
        *reinterpret_cast<u32x2*>(pq_) = __builtin_bit_cast(u32x2, dst.qo[0]);
        *reinterpret_cast<u32x2*>(pk_) = __builtin_bit_cast(u32x2, dst.ko[0]);
      } else {
#pragma unroll
        for (int qq = 0; qq < TPW / 2; ++qq) {
          const int q = w * (TPW / 2) + qq;
          const u32x2 a0 = __builtin_bit_cast(u32x2, dst.qo[2 * qq]), a1 = __builtin_bit_cast(u32x2, dst.qo[2 * qq + 1]);
          const u32x2 b0 = __builtin_bit_cast(u32x2, dst.ko[2 * qq]), b1 = __builtin_bit_cast(u32x2, dst.ko[2 * qq + 1]);
          xb[(0 * (NT / 2) + q) * 64 + lane] = u32x4{a0[0], a0[1], a1[0], a1[1]};
          xb[(1 * (NT / 2) + q) * 64 + lane] = u32x4{b0[0], b0[1], b1[0], b1[1]};
        }
      }
      if (FORM && stage < n_stages_ && tok) {
        const unsigned off = UnitBase<T, D>::row_off(stage, K, c);
        const size_t u0 = bh * (size_t)a.seq * (D * sizeof(elem));
        auto put = [&](void* base, const frag (&x)[TPW]) {
          if (base == nullptr) return;
          unsigned char* pb_ = static_cast<unsigned char*>(base) + u0 + off;
          if (TPW == 1) {
            *reinterpret_cast<u32x2*>(pb_ + own_offset<TPW>(w, 0, g) * sizeof(elem)) = __builtin_bit_cast(u32x2, x[0]);
          } else {
#pragma unroll
            for (int qq = 0; qq < TPW / 2; ++qq) {
              const u32x2 a0 = __builtin_bit_cast(u32x2, x[2 * qq]), a1 = __builtin_bit_cast(u32x2, x[2 * qq + 1]);
              *reinterpret_cast<u32x4*>(pb_ + own_offset<TPW>(w, 2 * qq, g) * sizeof(elem)) = u32x4{a0[0], a0[1], a1[0], a1[1]};
            }
          }
        };
        put(fip->xq_out, dst.qo);
        put(fip->xk_out, dst.ko);
        put(fip->xv_out, dst.vo);
        if (fip->lr_out != nullptr && w == 0 && g == 0)
          IO::store1(static_cast<elem*>(fip->lr_out) + bh * (size_t)a.seq + (size_t)stage * K + c, dst.lr);
      }
    }
  };
  // the full rotated rows of a mini-batch, from LDS buffer `pb` (behind a barrier that follows rotate_share)
  auto gather_rows = [&](StageInMw<T, NT, TPW>& dst, int pb) {
    if constexpr (RAW != 0 && !DMA) {
      const u32x4* xb = xrot + (size_t)pb * 2 * (NT / 2) * 64;
#pragma unroll
      for (int q = 0; q < NT / 2; ++q) {
        const u32x4 vq = xb[(0 * (NT / 2) + q) * 64 + lane], vk = xb[(1 * (NT / 2) + q) * 64 + lane];
        dst.q[2 * q] = __builtin_bit_cast(frag, u32x2{vq[0], vq[1]});
        dst.q[2 * q + 1] = __builtin_bit_cast(frag, u32x2{vq[2], vq[3]});
        dst.k[2 * q] = __builtin_bit_cast(frag, u32x2{vk[0], vk[1]});
        dst.k[2 * q + 1] = __builtin_bit_cast(frag, u32x2{vk[2], vk[3]});
      }
    }
  };
  // ---- RAW = 5: the ring the control wave fills, and the control wave itself
  constexpr int RS = 4;                                  // slots = mini-batches in flight
  constexpr int kCopies = 3 * NT + 1;                    // copies per mini-batch: the tile rows of xq, xk, xv, and lr
  __shared__ f32x4 ring_s[DMA ? RS : 1][3][DMA ? NT : 1][64];  // [slot][xq, xk, xv][feature tile][lane]
  __shared__ float ringlr_s[DMA ? RS : 1][64];           // lr of the lane's token c
  auto gather_dma = [&](StageInMw<T, NT, TPW>& dst, int stage) {
    if constexpr (DMA) {
      static_assert(!BF && TPW == 1 && FULL && !FAC, "control-wave loads: f32 I/O, one feature tile per wave, whole mini-batches");
      const int sl = stage & (RS - 1);
#pragma unroll
      for (int J = 0; J < NT; ++J) {
        dst.q[J] = ring_s[sl][0][J][lane];
        dst.k[J] = ring_s[sl][1][J][lane];
      }
      dst.qo[0] = ring_s[sl][0][w][lane];
      dst.ko[0] = ring_s[sl][1][w][lane];
      dst.vo[0] = ring_s[sl][2][w][lane];
      dst.lr = ringlr_s[sl][c];
    }
  };
  if constexpr (DMA) {
    if (ctlw) {
      const unsigned ring0 = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)&ring_s[0][0][0][0];
      const unsigned lr0 = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)&ringlr_s[0][0];
      // the copies of one mini-batch (past the end: the last one again, into a slot nobody reads)
      auto copy_in = [&](int stage) {
        const unsigned dst = ring0 + (unsigned)(stage & (RS - 1)) * (3 * NT * 1024);
        const int st_ld = min(stage, n_stages_ - 1);
        const unsigned off = UnitBase<T, D>::row_off(st_ld, K, c);
#pragma unroll
        for (int J = 0; J < NT; ++J) {
          const unsigned fo = (unsigned)(32 * (J >> 1) + 8 * g + 4 * (J & 1)) * 4u;  // the lane's four features of tile J
          lds_dma16(ub.xq, off + fo, dst + (0 * NT + J) * 1024);
          lds_dma16(ub.xk, off + fo, dst + (1 * NT + J) * 1024);
          lds_dma16(ub.xv, off + fo, dst + (2 * NT + J) * 1024);
        }
        // every lane issues (the count of copies in flight must not depend on the lane): lanes 16.. repeat token c's
        lds_dma4(ub.lr, ((unsigned)st_ld * (unsigned)K + (unsigned)c) * 4u, lr0 + (unsigned)(stage & (RS - 1)) * 256u);
      };
#pragma unroll
      for (int u = 0; u < RS; ++u) copy_in(u);
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"((RS - 1) * kCopies) : "memory");  // mini-batch 0 has landed
      asm volatile("s_barrier" ::: "memory");
      for (int st = 0; st < n_stages_; ++st) {
        // mini-batch st + 1 has landed (st + 2 .. st + RS - 1 may be in flight); behind the barrier the compute waves
        // read it, and the slot of mini-batch st, read behind the barrier before, is free
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((RS - 2) * kCopies) : "memory");
        asm volatile("s_barrier" ::: "memory");
        copy_in(st + RS);
      }
      asm volatile("s_barrier" ::: "memory");  // the exchange that flushes the last output
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      return;
    }
  }
  if constexpr (DMA) {
    lds_barrier();
    gather_dma(buf[0], 0);
  } else if constexpr (RAW != 0) {
    // mini-batch 0 complete, mini-batch 1 rotated and on its way through LDS (read behind the first barrier of the
    // loop), the raw rows of mini-batch 2 in flight
#pragma unroll
    for (int u = 0; u < R; ++u) load_raw(raw[u], u);
    rotate_share(raw[0], buf[0], 0, 0);
    lds_barrier();
    gather_rows(buf[0], 0);
    rotate_share(raw[1], buf[1], 1, 1);
  } else {
#pragma unroll
    for (int u = 0; u < PF; ++u) load_stage_mw<T, D, NW, FULL>(buf[u], ub, K, n_stages_, u, c, g, w);
  }

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
      if constexpr (RAW != 0)
        load_raw(raw[u], st + R);  // its previous content, mini-batch st, was rotated two mini-batches ago
      else
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
      // RAW: the rows of the next mini-batch, rotated by their owners before this barrier
      if constexpr (DMA) gather_dma(buf[(u + 1) % R], st + 1);
      else if constexpr (RAW != 0) gather_rows(buf[(u + 1) % R], (st + 1) & 1);
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
      if constexpr (ADAM) {
        pw1 *= adam->beta1;
        pw2 *= adam->beta2;
        ad_a1 = adam->lr / (1.f - pw1);
        ad_ic2 = 1.f / (1.f - pw2);
#pragma unroll
        for (int I = 0; I < NT; ++I)
#pragma unroll
          for (int jj = 0; jj < TPW; ++jj) {
            f32x4 gneg = {0.f, 0.f, 0.f, 0.f};
            IO::mma(gneg, kd[I], Gd[jj]);
            adam_tile(Wc[I][jj], Wm[I][jj], Wv[I][jj], gneg);
          }
#pragma unroll
        for (int jj = 0; jj < TPW; ++jj) {
          f32x4 gneg = {0.f, 0.f, 0.f, 0.f};
          IO::mma(gneg, Gd[jj], ones_upd);
          adam_tile(bT[jj], bm[jj], bv[jj], gneg);
        }
      } else {
#pragma unroll
        for (int I = 0; I < NT; ++I)
#pragma unroll
          for (int jj = 0; jj < TPW; ++jj) IO::mma(Wc[I][jj], kd[I], Gd[jj]);
        bias_update(bT, Gd, ones_upd);
      }
      // this mini-batch's Zbar and xq become the pending output; its in-lane sums are formed here, in the
      // shadow of the state update, not between the next Z1 and its exchange
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) {
        zbp[jj] = zb[jj];
        qop[jj] = cur.qo[jj];
      }
      pend_sums(zbp, ps0, ps1);
      // RAW: the own features of the mini-batch after the next, loaded during the previous pass of the loop; read
      // back by every wave behind the next barrier.  LDS buffer st & 1 was last read behind the barrier of the
      // previous mini-batch, which every wave has left.
      if constexpr (RAW != 0) rotate_share(raw[(u + 2) % R], buf[(u + 2) % R], st + 2, st & 1);
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
        if constexpr (RAW != 0)
          load_raw(raw[u], st + R);
        else
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
        if constexpr (RAW != 0) gather_rows(buf[(u + 1) % R], (st + 1) & 1);
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
          bias_update(bT, Gd, ones);
        }
        // this mini-batch's Zbar and xq become the pending output
#pragma unroll
        for (int jj = 0; jj < TPW; ++jj) {
          zbp[jj] = zb[jj];
          qop[jj] = cur.qo[jj];
        }
        if constexpr (RAW != 0) rotate_share(raw[(u + 2) % R], buf[(u + 2) % R], st + 2, st & 1);
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
  if constexpr (ADAM) {
#pragma unroll
    for (int I = 0; I < NT; ++I)
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const size_t at = bh * D * D + feat(I, 4 * g + r) * D + feat(w * TPW + jj, c);
          adam->Wm_out[at] = Wm[I][jj][r];
          adam->Wv_out[at] = Wv[I][jj][r];
        }
    if (c == 0) {
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) {
        const size_t at = bh * D + own_offset<TPW>(w, jj, g);
        *reinterpret_cast<f32x4*>(adam->bm_out + at) = bm[jj];
        *reinterpret_cast<f32x4*>(adam->bv_out + at) = bv[jj];
      }
    }
  }
  if constexpr (FAC)
    store_state_tiles<D, TPW>(a.W_ckpt + bh * (size_t)a.n_ckpt * (D * D), a.b_ckpt + bh * (size_t)a.n_ckpt * D, Wc, bT, w, lane);
}

// OWN = 1: every wave loads only the features it owns, full rows through LDS (RAW = 3); OWN = 2: the same with the
// operands formed as x + xq, x + xk, x + xv (RAW = 4)
template <class T, int D, int NW, int PF, bool FULL, bool FAC = false, int OWN = 0>
__global__ void __launch_bounds__(64 * NW) ttt_linear_fwd_sk_kernel(Problems<LinearFwdArgs> problems) {
  linear_fwd_sk_body<T, D, NW, PF, FULL, FAC, OWN == 0 ? 0 : OWN + 2>(problems.p[blockIdx.y], nullptr);
}

// The forward with a control wave that brings the operands in: see RAW = 5 above.
template <class T, int D, int NW, int PF>
__global__ void __launch_bounds__(64 * (NW + 1)) ttt_linear_fwd_dma_kernel(Problems<LinearFwdArgs> problems) {
  linear_fwd_sk_body<T, D, NW, PF, true, false, 5>(problems.p[blockIdx.y], nullptr);
}

// TTT-Linear with the Adam inner optimiser: see ADAM above.
template <class T, int D, int NW, int PF, bool FULL>
__global__ void __launch_bounds__(64 * NW) ttt_linear_adam_fwd_kernel(LinearFwdArgs a, AdamArgs ad) {
  linear_fwd_sk_body<T, D, NW, PF, FULL, false, 0, true>(a, nullptr, &ad);
}

// The same forward on the projections as they leave the GEMMs: see RAW above.
template <class T, int D, int NW, int PF, bool FULL, bool FAC, int RAW>
__global__ void __launch_bounds__(64 * NW) ttt_linear_fwd_fi_kernel(LinearFwdArgs a, FusedInputsArgs fi) {
  static_assert(RAW == 1 || RAW == 2, "RAW selects how positions are looked up");
  linear_fwd_sk_body<T, D, NW, PF, FULL, FAC, RAW>(a, &fi);
}

}  // namespace ttt
