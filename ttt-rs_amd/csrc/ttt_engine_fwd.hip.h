// LDS-engine forward kernels: TTT-Linear for every supported head_dim (32..128) and TTT-MLP.
//
// TTT-Linear arithmetic: reference rust/core/src/linear.rs:91-149 (one mini-batch) looped as
// rust/core/src/inner.rs:25-50, checkpoints as
// rust/fused/src/linear_fused_tile/forward/kernel.rs:143-150.
// TTT-MLP arithmetic: reference rust/core/src/mlp.rs:127-208 (the reference has no fused MLP
// kernel; this is its Burn-op inner model restated as one persistent kernel).
//
// One workgroup per (batch, head) walks the mini-batches in order.  TTT-Linear keeps W, b in
// LDS for the whole sequence.  The TTT-MLP state (W1 [d,4d], W2 [4d,d], f32) is larger than a
// CU's LDS for d >= 96, so it lives in the caller's W1_out/W2_out buffers (L2-resident working
// set), is read in place as an MFMA operand and updated in place; b1, b2 stay in LDS.
#pragma once
#include "ttt_engine.hip.h"
#include "ttt_linear_fwd.hip.h"

namespace ttt {

// ------------------------------------------------------------------------------------------
// Shared elementwise pieces.  Thread (t = tid / GW, cg = tid % GW) owns token t and features
// cg + GW*j; GW lanes of one token are an aligned lane group.
// ------------------------------------------------------------------------------------------

// z (+ bias) -> x_hat, rstd over D features for this thread's token
template <int D, int GW>
__device__ __forceinline__ void ln_stats(const float* zrow, const float* bias, int cg, float eps,
                                         float (&xh)[D / GW], float& rstd) {
  constexpr int NJ = D / GW;
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    xh[j] = zrow[cg + GW * j] + bias[cg + GW * j];
    s += xh[j];
  }
  const float mu = rowgroup_sum<GW>(s) * (1.0f / D);
  float v = 0.f;
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    xh[j] -= mu;
    v += xh[j] * xh[j];
  }
  rstd = __builtin_amdgcn_rsqf(rowgroup_sum<GW>(v) * (1.0f / D) + eps);
#pragma unroll
  for (int j = 0; j < NJ; ++j) xh[j] *= rstd;
}

// G = d/dz 0.5 || LN(z) - target ||^2   (reference rust/core/src/util.rs:155-182)
template <int D, int GW>
__device__ __forceinline__ void ln_l2_grad(const float* zrow, const float* bias, const float* tgrow,
                                           const float* gam, const float* bet, int cg, float eps,
                                           float (&G)[D / GW]) {
  constexpr int NJ = D / GW;
  float xh[NJ], rstd, gx[NJ], s1 = 0.f, s2 = 0.f;
  ln_stats<D, GW>(zrow, bias, cg, eps, xh, rstd);
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const float ga = gam[cg + GW * j];
    gx[j] = (ga * xh[j] + bet[cg + GW * j] - tgrow[cg + GW * j]) * ga;
    s1 += gx[j];
    s2 += gx[j] * xh[j];
  }
  s1 = rowgroup_sum<GW>(s1) * (1.0f / D);
  s2 = rowgroup_sum<GW>(s2) * (1.0f / D);
#pragma unroll
  for (int j = 0; j < NJ; ++j) G[j] = (gx[j] - s1 - xh[j] * s2) * rstd;
}

// ------------------------------------------------------------------------------------------
// TTT-Linear forward, W resident in LDS.  MT tiles of 16 token rows (mini_batch <= 16 MT), 256 MT threads, GW = 16.
// MT = 2 is the kernel of the reference's (mini_batch 32, head_dim 32) tile
// (rust/fused/src/linear_fused_tile/mod.rs:38).
// ------------------------------------------------------------------------------------------
template <int D, int MT = 1>
struct LinFwdLds {
  static constexpr int KT = 16 * MT, LD = D + 4, LK = KT + 1, TILE = KT * LD, KK = KT * LK;
  static constexpr int W = 0, XQ = W + D * LD, XK = XQ + TILE, TG = XK + TILE, G = TG + TILE,
                       ZB = G + TILE, A = ZB + TILE, M = A + KK, b = M + KK, gam = b + D,
                       bet = gam + D, lr = bet + D, te = lr + KT, END = te + KT;
  static constexpr size_t BYTES = sizeof(float) * END;
};

// BF: operands of the products rounded to bf16 (see ttt_linear_bwd_kernel)
template <class T, int D, int MT = 1, bool BF = false>
__global__ void __launch_bounds__(256 * MT) ttt_linear_fwd_lds_kernel(Problems<LinearFwdArgs> problems) {
  const LinearFwdArgs& a = problems.p[blockIdx.y];
  using E = Eng<BF>;
  using IO = Io<T>;
  using elem = typename IO::elem;
  using L = LinFwdLds<D, MT>;
  constexpr int LD = L::LD, LK = L::LK, KT = L::KT, NJ = D / 16, NT = D / 16, NTH = 256 * MT, NW = 4 * MT;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int t = tid >> 4, cg = tid & 15;
  const size_t bh = blockIdx.x;
  const int h = (int)(bh % a.H), K = a.K;
  float *sW = lds + L::W, *sb = lds + L::b, *sgam = lds + L::gam, *sbet = lds + L::bet,
        *slr = lds + L::lr, *ste = lds + L::te;
  const size_t sbase = a.state_per_batch ? bh : (size_t)h;

  for (int i = tid; i < D * D; i += NTH) sW[(i / D) * LD + (i % D)] = a.W0[sbase * D * D + i];
  for (int i = tid; i < D; i += NTH) {
    sb[i] = a.b0[sbase * D + i];
    sgam[i] = a.gamma[h * D + i];
    sbet[i] = a.beta[h * D + i];
  }
  if (tid < KT) ste[tid] = (tid < K) ? a.token_eta[tid] : 0.f;
  __syncthreads();
  const float te_last = ste[K - 1];

  // the next mini-batch's xq/xk/xv/lr are fetched into registers while this one computes
  float pq[NJ], pk[NJ], pv[NJ], plr = 0.f;
  auto fetch = [&](int stage) {
    const size_t r = (bh * (size_t)a.seq_stride + (size_t)stage * K + t) * D;
    const bool ok = t < K;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int o = cg + 16 * j;
      pq[j] = ok ? IO::load1(static_cast<const elem*>(a.xq) + r + o) : 0.f;
      pk[j] = ok ? IO::load1(static_cast<const elem*>(a.xk) + r + o) : 0.f;
      pv[j] = ok ? IO::load1(static_cast<const elem*>(a.xv) + r + o) : 0.f;
    }
    if (tid < KT)
      plr = (tid < K) ? IO::load1(static_cast<const elem*>(a.lr) + bh * (size_t)a.seq_stride + (size_t)stage * K + tid) : 0.f;
  };
  fetch(0);

  for (int st = 0; st < a.n_stages; ++st) {
    const size_t row = bh * (size_t)a.seq_stride + (size_t)st * K + t;
    if (a.W_ckpt != nullptr && (st % a.ckpt_interval) == 0) {
      const size_t ci = bh * a.n_ckpt + st / a.ckpt_interval;
      for (int i = tid; i < D * D; i += NTH) a.W_ckpt[ci * D * D + i] = sW[(i / D) * LD + (i % D)];
      for (int i = tid; i < D; i += NTH) a.b_ckpt[ci * D + i] = sb[i];
    }
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int o = cg + 16 * j;
      lds[L::XQ + t * LD + o] = pq[j];
      lds[L::XK + t * LD + o] = pk[j];
      lds[L::TG + t * LD + o] = pv[j] - pk[j];
    }
    if (tid < KT) slr[tid] = plr;
    __syncthreads();
    if (st + 1 < a.n_stages) fetch(st + 1);
    E::template lds<0, NW>(lds + L::G, LD, lds + L::XK, LD, 1, sW, LD, 1, MT, NT, D, wave, lane);
    E::template lds<0, NW>(lds + L::ZB, LD, lds + L::XQ, LD, 1, sW, LD, 1, MT, NT, D, wave, lane, (MT * NT) % NW);
    E::template lds<0, NW>(lds + L::A, LK, lds + L::XQ, LD, 1, lds + L::XK, 1, LD, MT, MT, D, wave, lane, (2 * MT * NT) % NW);
    __syncthreads();
    {
      float Gv[NJ];
      ln_l2_grad<D, 16>(lds + L::G + t * LD, sb, lds + L::TG + t * LD, sgam, sbet, cg, a.eps, Gv);
#pragma unroll
      for (int j = 0; j < NJ; ++j) lds[L::G + t * LD + cg + 16 * j] = Gv[j];
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const int s = cg + 16 * i;
        const float at = lds[L::A + t * LK + s];
        lds[L::M + t * LK + s] = (s <= t) ? ste[t] * slr[s] * (1.f + at) : 0.f;
      }
    }
    __syncthreads();
    E::template lds<2, NW, 1, 4>(lds + L::ZB, LD, lds + L::M, LK, 1, lds + L::G, LD, 1, MT, NT, KT, wave, lane);
    __syncthreads();
    {
      float xh[NJ], rstd;
      ln_stats<D, 16>(lds + L::ZB + t * LD, sb, cg, a.eps, xh, rstd);
      const float last = te_last * slr[t];
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int o = cg + 16 * j;
        if (t < K)
          IO::store1(static_cast<elem*>(a.out) + row * D + o,
                     lds[L::XQ + t * LD + o] + (sgam[o] * xh[j] + sbet[o]));
        lds[L::G + t * LD + o] *= last;
      }
    }
    __syncthreads();
    E::template lds<2, NW, (NT % 4 == 0 ? 4 : 2), 4>(sW, LD, lds + L::XK, 1, LD, lds + L::G, LD, 1, NT, NT, KT, wave, lane);
    if (tid < D) {
      float s = 0.f;
      for (int r = 0; r < KT; ++r) s += lds[L::G + r * LD + tid];
      sb[tid] -= s;
    }
    __syncthreads();
  }
  for (int i = tid; i < D * D; i += NTH) a.W_out[bh * D * D + i] = sW[(i / D) * LD + (i % D)];
  for (int i = tid; i < D; i += NTH) a.b_out[bh * D + i] = sb[i];
}

// ------------------------------------------------------------------------------------------
// TTT-MLP forward.  512 threads (8 waves), GW = 32.  M = 4 D hidden units.
// ------------------------------------------------------------------------------------------
struct MlpFwdArgs {
  const void* xq;
  const void* xk;
  const void* xv;
  const float* W1_0;
  const float* b1_0;
  const float* W2_0;
  const float* b2_0;
  const float* token_eta;
  const void* lr;
  const float* gamma;
  const float* beta;
  void* out;
  float* W1;  // [B,H,D,M] live state, ends as W1_out
  float* b1;
  float* W2;  // [B,H,M,D]
  float* b2;
  // optional (LDS-tile kernel only): per mini-batch, the rank-16 factors of the state update,
  // eta_last * G1 [B*H][N][16][M] and eta_last * G2 [B*H][N][16][D], for ttt_mlp_bwd; out may then be null
  float* G1_save;
  float* G2_save;
  int B, H, seq, seq_stride, K, n_stages, state_per_batch;
  float eps;
  int unit_base;  // two-CU kernel only: first (batch, head) unit of this launch (the units are launched in batches)
  int spin_limit;  // two-CU kernel only: polls before a wait for the partner gives up (0: give up at once; testing)
  int exchange_cleared;  // two-CU kernel only, read by the host: the exchange area (W2) has been zeroed by the caller
  int assume_other_xcd;  // two-CU kernel only: treat the partner as sitting on another XCD whatever it reports (testing)
};

template <int D>
struct MlpLds {
  static constexpr int M = 4 * D, LD = D + 4, LM = M + 4, LK = 17, KK = 16 * LK;
  static constexpr int TD = 16 * LD, TM = 16 * LM;
  // m-wide buffers: BA (Z1 -> gelu'(Z1) -> G1), BB (X2), BC (Zbar1 -> Xbar2)
  static constexpr int BA = 0, BB = BA + TM, BC = BB + TM;
  // d-wide tiles: TG (target), Z2 (Z2 -> G2), ZB2 ; PART: eight [16 x 16] split-k partials of A2
  static constexpr int XQ = BC + TM, XK = XQ + TD, TG = XK + TD, Z2 = TG + TD, ZB2 = Z2 + TD;
  static constexpr int PART = ZB2 + TD;
  static constexpr int A1 = PART + 8 * 256, M1 = A1 + KK, M2 = M1 + KK, ETA = M2 + KK;
  static constexpr int b1 = ETA + KK, b2 = b1 + M, gam = b2 + D, bet = gam + D, lr = bet + D,
                       te = lr + 16, END = te + 16;
  static constexpr size_t BYTES = sizeof(float) * END;
  static_assert(BYTES <= 160 * 1024, "exceeds the 160 KiB of LDS of a gfx950 CU");
};

template <class T, int D>
// one workgroup per CU (LDS), two waves per SIMD: stated so that the scheduler does not serialise loads to save registers
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) ttt_mlp_fwd_kernel(Problems<MlpFwdArgs> problems) {
  const MlpFwdArgs& a = problems.p[blockIdx.y];
  using IO = Io<T>;
  using elem = typename IO::elem;
  using L = MlpLds<D>;
  constexpr int M = L::M, LD = L::LD, LM = L::LM, LK = L::LK;
  constexpr int NW = 8, GW = 32, NJD = D / GW, NJM = M / GW, NTD = D / 16, NTM = M / 16;
  constexpr int NBM = NTM / NW;  // hidden-side tile columns per job: one job per wave
  constexpr int NBD = NTD % 3 == 0 ? 3 : 2;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  // re-derived from an opaque copy at the top of every mini-batch, so that the address arithmetic of the
  // tile products is recomputed there instead of being hoisted out of the scan into (spilled) registers
  int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int t = tid >> 5, cg = tid & 31;
  const size_t bh = blockIdx.x;
  const int h = (int)(bh % a.H), K = a.K;
  float *sb1 = lds + L::b1, *sb2 = lds + L::b2, *sgam = lds + L::gam, *sbet = lds + L::bet,
        *slr = lds + L::lr, *ste = lds + L::te;
  float* W1 = a.W1 + bh * (size_t)D * M;
  float* W2 = a.W2 + bh * (size_t)M * D;
  const size_t sbase = a.state_per_batch ? bh : (size_t)h;

  // ---- initial state -> live buffers
  for (int i = tid; i < D * M; i += 512) {
    W1[i] = a.W1_0[sbase * D * M + i];
    W2[i] = a.W2_0[sbase * D * M + i];
  }
  for (int i = tid; i < M; i += 512) sb1[i] = a.b1_0[sbase * M + i];
  for (int i = tid; i < D; i += 512) {
    sb2[i] = a.b2_0[sbase * D + i];
    sgam[i] = a.gamma[h * D + i];
    sbet[i] = a.beta[h * D + i];
  }
  if (tid < 16) ste[tid] = (tid < K) ? a.token_eta[tid] : 0.f;
  __syncthreads();
  const float te_last = ste[K - 1];

  // the next mini-batch's xq/xk/xv/lr are fetched into registers while this one computes
  float pq[NJD], pk[NJD], pv[NJD], plr = 0.f;
  auto fetch = [&](int stage) {
    const size_t r = (bh * (size_t)a.seq_stride + (size_t)stage * K + t) * D;
    const bool ok = t < K;
#pragma unroll
    for (int j = 0; j < NJD; ++j) {
      const int o = cg + GW * j;
      pq[j] = ok ? IO::load1(static_cast<const elem*>(a.xq) + r + o) : 0.f;
      pk[j] = ok ? IO::load1(static_cast<const elem*>(a.xk) + r + o) : 0.f;
      pv[j] = ok ? IO::load1(static_cast<const elem*>(a.xv) + r + o) : 0.f;
    }
    if (tid < 16)
      plr = (tid < K) ? IO::load1(static_cast<const elem*>(a.lr) + bh * (size_t)a.seq_stride + (size_t)stage * K + tid) : 0.f;
  };
  fetch(0);

  // without an output buffer (the sweep that the backward runs for the update factors and the final state) the
  // output branch of every mini-batch is skipped: two of the five passes over the state and eight barriers
  const bool want_out = a.out != nullptr;
  for (int st = 0; st < a.n_stages; ++st) {
    asm volatile("" : "+v"(tid));
    lane = tid & 63, wave = tid >> 6, t = tid >> 5, cg = tid & 31;
    const size_t row = bh * (size_t)a.seq_stride + (size_t)st * K + t;
    // ---- XQ, XK, target = XV - XK from the prefetch registers
#pragma unroll
    for (int j = 0; j < NJD; ++j) {
      const int o = cg + GW * j;
      lds[L::XQ + t * LD + o] = pq[j];
      lds[L::XK + t * LD + o] = pk[j];
      lds[L::TG + t * LD + o] = pv[j] - pk[j];
    }
    if (tid < 16) slr[tid] = plr;
    __syncthreads();
    if (st + 1 < a.n_stages) fetch(st + 1);
    // ---- Z1 = XK W1 ; Zbar1 = XQ W1 ; A1 = XQ XK^T            (mlp.rs:139,160,167)
    mm_lds<0, NW, NBM>(lds + L::BA, LM, lds + L::XK, LD, 1, W1, M, 1, 1, NTM, D, wave, lane);
    if (want_out) {
      mm_lds<0, NW, NBM>(lds + L::BC, LM, lds + L::XQ, LD, 1, W1, M, 1, 1, NTM, D, wave, lane);
      mm_lds<0, NW>(lds + L::A1, LK, lds + L::XQ, LD, 1, lds + L::XK, 1, LD, 1, 1, D, wave, lane);
    }
    __syncthreads();
    // ---- X2 = gelu(Z1 + b1), keep gelu'(Z1 + b1) ; eta, M1 = eta (1 + A1)   (mlp.rs:141,154-162)
#pragma unroll
    for (int j = 0; j < NJM; ++j) {
      const int o = cg + GW * j;
      float y, dy;
      gelu_tanh_pair(lds[L::BA + t * LM + o] + sb1[o], y, dy);
      lds[L::BB + t * LM + o] = y;
      lds[L::BA + t * LM + o] = dy;
    }
    if (want_out && tid < 256) {
      const int tt = tid >> 4, s = tid & 15;
      const float et = (s <= tt) ? ste[tt] * slr[s] : 0.f;
      lds[L::ETA + tt * LK + s] = et;
      lds[L::M1 + tt * LK + s] = et * (1.f + lds[L::A1 + tt * LK + s]);
    }
    __syncthreads();
    // ---- Z2 = X2 W2                                           (mlp.rs:143)
    mm_lds<0, NW>(lds + L::Z2, LD, lds + L::BB, LM, 1, W2, D, 1, 1, NTD, M, wave, lane);
    __syncthreads();
    // ---- G2 = LN-L2 gradient of Z2 + b2 against the target    (mlp.rs:145-149)
    {
      float Gv[NJD];
      ln_l2_grad<D, GW>(lds + L::Z2 + t * LD, sb2, lds + L::TG + t * LD, sgam, sbet, cg, a.eps, Gv);
#pragma unroll
      for (int j = 0; j < NJD; ++j) lds[L::Z2 + t * LD + cg + GW * j] = Gv[j];
    }
    __syncthreads();
    // ---- G1 = (G2 W2^T) * gelu'(Z1)                           (mlp.rs:151-152)
    mm_lds<3, NW, NBM, 2, true>(lds + L::BA, LM, lds + L::Z2, LD, 1, W2, 1, D, 1, NTM, D, wave, lane);
    __syncthreads();
    if (want_out) {  // the output branch: skipped when only the update factors and the final state are wanted
      // ---- Zbar1 -= M1 G1                                       (mlp.rs:164-169)
      mm_lds<2, NW, NBM, 4>(lds + L::BC, LM, lds + L::M1, LK, 1, lds + L::BA, LM, 1, 1, NTM, 16, wave, lane);
      __syncthreads();
      // ---- Xbar2 = gelu(Zbar1 + b1)                             (mlp.rs:171)
#pragma unroll
      for (int j = 0; j < NJM; ++j) {
        const int o = cg + GW * j;
        float y, dy;
        gelu_tanh_pair(lds[L::BC + t * LM + o] + sb1[o], y, dy);
        lds[L::BC + t * LM + o] = y;
      }
      __syncthreads();
      // ---- A2 = Xbar2 X2^T (split over k, one slice per wave) ; Zbar2 = Xbar2 W2   (mlp.rs:173,178)
      {
        const int c = lane & 15, g = lane >> 4;
        constexpr int KS = M / NW;  // k-slice per wave (multiple of 4)
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        const float* Ap = lds + L::BC + c * LM + wave * KS + g;
        const float* Bp = lds + L::BB + c * LM + wave * KS + g;
#pragma unroll 4
        for (int k = 0; k < KS; k += 4) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(Ap[k], Bp[k], acc, 0, 0, 0);
#pragma unroll
        for (int r = 0; r < 4; ++r) lds[L::PART + wave * 256 + (4 * g + r) * 16 + c] = acc[r];
      }
      mm_lds<0, NW>(lds + L::ZB2, LD, lds + L::BC, LM, 1, W2, D, 1, 1, NTD, M, wave, lane);
      __syncthreads();
      if (tid < 256) {
        const int tt = tid >> 4, s = tid & 15;
        float a2 = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) a2 += lds[L::PART + w * 256 + tt * 16 + s];
        lds[L::M2 + tt * LK + s] = lds[L::ETA + tt * LK + s] * (1.f + a2);
      }
      __syncthreads();
      // ---- Zbar2 -= M2 G2                                       (mlp.rs:175-180)
      mm_lds<2, NW, 1, 4>(lds + L::ZB2, LD, lds + L::M2, LK, 1, lds + L::Z2, LD, 1, 1, NTD, 16, wave, lane);
      __syncthreads();
    }
    // ---- out = XQ + LN(Zbar2 + b2) ; scale G1, G2 by eta_last  (mlp.rs:182-207)
    {
      const float last = te_last * slr[t];
      if (want_out) {
        float xh[NJD], rstd;
        ln_stats<D, GW>(lds + L::ZB2 + t * LD, sb2, cg, a.eps, xh, rstd);
#pragma unroll
        for (int j = 0; j < NJD; ++j) {
          const int o = cg + GW * j;
          if (t < K)
            IO::store1(static_cast<elem*>(a.out) + row * D + o,
                       lds[L::XQ + t * LD + o] + (sgam[o] * xh[j] + sbet[o]));
        }
      }
#pragma unroll
      for (int j = 0; j < NJD; ++j) lds[L::Z2 + t * LD + cg + GW * j] *= last;
#pragma unroll
      for (int j = 0; j < NJM; ++j) lds[L::BA + t * LM + cg + GW * j] *= last;
      if (a.G1_save != nullptr) {
        const size_t srow = (bh * (size_t)a.n_stages + st) * 16 + t;
#pragma unroll
        for (int j = 0; j < NJD; ++j) a.G2_save[srow * D + cg + GW * j] = lds[L::Z2 + t * LD + cg + GW * j];
#pragma unroll
        for (int j = 0; j < NJM; ++j) a.G1_save[srow * M + cg + GW * j] = lds[L::BA + t * LM + cg + GW * j];
      }
    }
    __syncthreads();
    // ---- W1 -= XK^T G1l ; W2 -= X2^T G2l ; b1 -= colsum(G1l) ; b2 -= colsum(G2l)
    mm_rank<2, NW, NBM, 4>(W1, M, lds + L::XK, 1, LD, lds + L::BA, LM, 1, NTD, NTM, wave, lane);
    mm_rank<2, NW, NBD, 4>(W2, D, lds + L::BB, 1, LM, lds + L::Z2, LD, 1, NTM, NTD, wave, lane);
    if (tid < M) {
      float s = 0.f;
      for (int r = 0; r < 16; ++r) s += lds[L::BA + r * LM + tid];
      sb1[tid] -= s;
    }
    if (tid < D) {
      float s = 0.f;
      for (int r = 0; r < 16; ++r) s += lds[L::Z2 + r * LD + tid];
      sb2[tid] -= s;
    }
    __syncthreads();
  }
  for (int i = tid; i < M; i += 512) a.b1[bh * M + i] = sb1[i];
  for (int i = tid; i < D; i += 512) a.b2[bh * D + i] = sb2[i];
}

}  // namespace ttt
