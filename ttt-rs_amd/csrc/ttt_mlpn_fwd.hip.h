// TTT-MLP with NL hidden layers (NL = 2, 3, 4), multi-stage forward: the reference's TTTMLP2 / TTTMLP3 / TTTMLP4 inner
// models (rust/core/src/mlp2.rs:152-243, mlp3.rs:162-279, mlp4.rs:186-324) looped as rust/core/src/inner.rs:25-50.
// The reference has no fused kernel for them; this is their Burn-op mini-batch restated as one persistent kernel on
// the LDS tile engine, the NL-layer generalisation of ttt_mlp_fwd_kernel (ttt_engine_fwd.hip.h):
//
//   weight layer i = 0 .. NL:  W[i] [in_i x out_i], in_0 = d, out_NL = d, every other side M = 4 d
//   forward chain   X[0] = XK;  Z[i] = X[i] W[i] + b[i];  X[i+1] = gelu(Z[i])  (i < NL)
//   gradients       G[NL] = LN-L2 gradient of Z[NL] against XV - XK;  G[i] = (G[i+1] W[i+1]^T) * gelu'(Z[i])
//   output chain    Xb[0] = XQ;  Zb[i] = Xb[i] W[i] - (eta (1 + tril(Xb[i] X[i]^T))) G[i] + b[i];  Xb[i+1] = gelu(Zb[i])
//   out = XQ + LN(Zb[NL]);   W[i] -= (eta_last X[i])^T G[i];   b[i] -= colsum(eta_last G[i])
//
// One workgroup of 8 waves per (batch, head).  The state (up to 4 d x 4 d floats per hidden-to-hidden layer) lives in
// the caller's output buffers, is read in place as a matrix operand and updated in place (an L2-resident working
// set); the [16 x 4d] and [16 x d] tiles of a mini-batch, the biases and the 16 x 16 matrices are in LDS.  All
// products are f32 matrix instructions for both I/O types.  LDS holds 2 NL + 2 hidden-wide tiles, which bounds the
// shapes: head_dim 32 with up to four hidden layers, head_dim 64 with two.
#pragma once
#include "ttt_engine_fwd.hip.h"

namespace ttt {

constexpr int kMlpNMaxLayers = 5;  // weight layers of the deepest variant (four hidden layers)

struct MlpNFwdArgs {
  const void* xq;
  const void* xk;
  const void* xv;
  const float* W0[kMlpNMaxLayers];  // initial state of weight layer i: [H,in,out] or [B,H,in,out]
  const float* b0[kMlpNMaxLayers];  // [H,out] or [B,H,out]
  float* W[kMlpNMaxLayers];         // [B,H,in,out]: live state during the call, final state after it
  float* b[kMlpNMaxLayers];         // [B,H,out]
  const float* token_eta;
  const void* lr;
  const float* gamma;
  const float* beta;
  void* out;
  int B, H, seq, seq_stride, K, n_stages, state_per_batch;  // seq_stride: tokens between consecutive (b, h) units
  float eps;
};

template <int D, int NL>
struct MlpNLds {
  static constexpr int M = 4 * D, LD = D + 4, LM = M + 4, LK = 17, KK = 16 * LK;
  static constexpr int TD = 16 * LD, TM = 16 * LM;
  // hidden-wide tiles: BA[i] (Z[i] -> gelu'(Z[i]) -> G[i]) and BB[i] (X[i+1]) per hidden layer, two for the output
  // chain (Zb[i] -> Xb[i+1], used alternately)
  static constexpr int BA = 0, BB = BA + NL * TM, BC = BB + NL * TM;
  static constexpr int XQ = BC + 2 * TM, XK = XQ + TD, TG = XK + TD, ZL = TG + TD, ZBL = ZL + TD;
  static constexpr int PART = ZBL + TD;  // eight [16 x 16] split-k partials of an attention block
  static constexpr int AT = PART + 8 * 256, MX = AT + KK, ETA = MX + KK;
  static constexpr int bh = ETA + KK;       // NL hidden biases
  static constexpr int bl = bh + NL * M;    // bias of the last layer
  static constexpr int gam = bl + D, bet = gam + D, lr = bet + D, te = lr + 16, END = te + 16;
  static constexpr size_t BYTES = sizeof(float) * END;
  static_assert(BYTES <= 160 * 1024, "exceeds the 160 KiB of LDS of a gfx950 CU");
};

template <class T, int D, int NL>
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) ttt_mlpn_fwd_kernel(MlpNFwdArgs a) {
  using IO = Io<T>;
  using elem = typename IO::elem;
  using L = MlpNLds<D, NL>;
  constexpr int M = L::M, LD = L::LD, LM = L::LM, LK = L::LK, TM = L::TM;
  constexpr int NW = 8, GW = 32, NJD = D / GW, NJM = M / GW, NTD = D / 16, NTM = M / 16;
  constexpr int NBM = NTM / NW;  // hidden-side tile columns per job: one job per wave
  constexpr int NBD = NTD % 3 == 0 ? 3 : (NTD % 2 == 0 ? 2 : 1);
  static_assert(NTM % NW == 0, "hidden tiles must divide among the waves");
  extern __shared__ __attribute__((aligned(16))) float lds[];
  int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int t = tid >> 5, cg = tid & 31;
  const size_t bh = blockIdx.x;
  const int h = (int)(bh % a.H), K = a.K;
  float *sbl = lds + L::bl, *sgam = lds + L::gam, *sbet = lds + L::bet, *slr = lds + L::lr, *ste = lds + L::te;
  const size_t sbase = a.state_per_batch ? bh : (size_t)h;
  auto in_dim = [](int i) { return i == 0 ? D : M; };
  auto out_dim = [](int i) { return i == NL ? D : M; };

  // ---- initial state -> live buffers
  float* W[NL + 1];
#pragma unroll
  for (int i = 0; i <= NL; ++i) {
    const size_t n = (size_t)in_dim(i) * out_dim(i);
    W[i] = a.W[i] + bh * n;
    for (size_t e = tid; e < n; e += 512) W[i][e] = a.W0[i][sbase * n + e];
  }
#pragma unroll
  for (int i = 0; i < NL; ++i)
    for (int e = tid; e < M; e += 512) lds[L::bh + i * M + e] = a.b0[i][sbase * M + e];
  for (int e = tid; e < D; e += 512) {
    sbl[e] = a.b0[NL][sbase * D + e];
    sgam[e] = a.gamma[h * D + e];
    sbet[e] = a.beta[h * D + e];
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

  for (int st = 0; st < a.n_stages; ++st) {
    // re-derived from an opaque copy every mini-batch, so that the address arithmetic of the tile products is
    // recomputed here instead of being hoisted out of the scan into (spilled) registers
    asm volatile("" : "+v"(tid));
    lane = tid & 63, wave = tid >> 6, t = tid >> 5, cg = tid & 31;
    const size_t row = bh * (size_t)a.seq_stride + (size_t)st * K + t;
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

    // ---- forward chain: Z[i] = X[i] W[i]; X[i+1] = gelu(Z[i] + b[i]), gelu' kept in place of Z[i]
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      float* BAi = lds + L::BA + i * TM;
      float* BBi = lds + L::BB + i * TM;
      if (i == 0)
        mm_lds<0, NW, NBM>(BAi, LM, lds + L::XK, LD, 1, W[0], M, 1, 1, NTM, D, wave, lane);
      else
        mm_lds<0, NW, NBM>(BAi, LM, lds + L::BB + (i - 1) * TM, LM, 1, W[i], M, 1, 1, NTM, M, wave, lane);
      __syncthreads();
      const float* sb = lds + L::bh + i * M;
#pragma unroll
      for (int j = 0; j < NJM; ++j) {
        const int o = cg + GW * j;
        float y, dy;
        gelu_tanh_pair(BAi[t * LM + o] + sb[o], y, dy);
        BBi[t * LM + o] = y;
        BAi[t * LM + o] = dy;
      }
      __syncthreads();
    }
    // ---- Z[NL] = X[NL] W[NL]; G[NL] = LN-L2 gradient of Z[NL] + b[NL] against the target
    mm_lds<0, NW>(lds + L::ZL, LD, lds + L::BB + (NL - 1) * TM, LM, 1, W[NL], D, 1, 1, NTD, M, wave, lane);
    if (tid < 256) {
      const int tt = tid >> 4, s = tid & 15;
      lds[L::ETA + tt * LK + s] = (s <= tt) ? ste[tt] * slr[s] : 0.f;
    }
    __syncthreads();
    {
      float Gv[NJD];
      ln_l2_grad<D, GW>(lds + L::ZL + t * LD, sbl, lds + L::TG + t * LD, sgam, sbet, cg, a.eps, Gv);
#pragma unroll
      for (int j = 0; j < NJD; ++j) lds[L::ZL + t * LD + cg + GW * j] = Gv[j];
    }
    __syncthreads();
    // ---- G[i] = (G[i+1] W[i+1]^T) * gelu'(Z[i]), from the last hidden layer down
#pragma unroll
    for (int i = NL - 1; i >= 0; --i) {
      float* BAi = lds + L::BA + i * TM;
      if (i == NL - 1)
        mm_lds<3, NW, NBM, 2, true>(BAi, LM, lds + L::ZL, LD, 1, W[NL], 1, D, 1, NTM, D, wave, lane);
      else
        mm_lds<3, NW, NBM, 2, true>(BAi, LM, lds + L::BA + (i + 1) * TM, LM, 1, W[i + 1], 1, M, 1, NTM, M, wave, lane);
      __syncthreads();
    }
    // ---- output chain
#pragma unroll
    for (int i = 0; i <= NL; ++i) {
      float* zb = i == NL ? lds + L::ZBL : lds + L::BC + (i & 1) * TM;
      const float* xb = i == 0 ? lds + L::XQ : lds + L::BC + ((i - 1) & 1) * TM;
      const float* gi = i == NL ? lds + L::ZL : lds + L::BA + i * TM;
      if (i == 0) {
        // attention block and product over k = d
        mm_lds<0, NW>(lds + L::AT, LK, lds + L::XQ, LD, 1, lds + L::XK, 1, LD, 1, 1, D, wave, lane);
        mm_lds<0, NW, NBM>(zb, LM, xb, LD, 1, W[0], M, 1, 1, NTM, D, wave, lane);
      } else {
        // attention block Xb[i] X[i]^T over k = M, split over the waves
        {
          const int c = lane & 15, g = lane >> 4;
          constexpr int KS = M / NW;
          f32x4 acc = {0.f, 0.f, 0.f, 0.f};
          const float* Ap = xb + c * LM + wave * KS + g;
          const float* Bp = lds + L::BB + (i - 1) * TM + c * LM + wave * KS + g;
#pragma unroll 4
          for (int k = 0; k < KS; k += 4) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(Ap[k], Bp[k], acc, 0, 0, 0);
#pragma unroll
          for (int r = 0; r < 4; ++r) lds[L::PART + wave * 256 + (4 * g + r) * 16 + c] = acc[r];
        }
        if (i < NL)
          mm_lds<0, NW, NBM>(zb, LM, xb, LM, 1, W[i], M, 1, 1, NTM, M, wave, lane);
        else
          mm_lds<0, NW>(zb, LD, xb, LM, 1, W[NL], D, 1, 1, NTD, M, wave, lane);
      }
      __syncthreads();
      if (tid < 256) {
        const int tt = tid >> 4, s = tid & 15;
        float at;
        if (i == 0) {
          at = lds[L::AT + tt * LK + s];
        } else {
          at = 0.f;
#pragma unroll
          for (int w = 0; w < NW; ++w) at += lds[L::PART + w * 256 + tt * 16 + s];
        }
        lds[L::MX + tt * LK + s] = lds[L::ETA + tt * LK + s] * (1.f + at);
      }
      __syncthreads();
      if (i < NL)
        mm_lds<2, NW, NBM, 4>(zb, LM, lds + L::MX, LK, 1, gi, LM, 1, 1, NTM, 16, wave, lane);
      else
        mm_lds<2, NW, 1, 4>(zb, LD, lds + L::MX, LK, 1, gi, LD, 1, 1, NTD, 16, wave, lane);
      __syncthreads();
      if (i < NL) {
        const float* sb = lds + L::bh + i * M;
#pragma unroll
        for (int j = 0; j < NJM; ++j) {
          const int o = cg + GW * j;
          float y, dy;
          gelu_tanh_pair(zb[t * LM + o] + sb[o], y, dy);
          zb[t * LM + o] = y;
        }
        __syncthreads();
      }
    }
    // ---- out = XQ + LN(Zb[NL] + b[NL]); the gradients scaled by eta_last for the update
    {
      const float last = te_last * slr[t];
      float xh[NJD], rstd;
      ln_stats<D, GW>(lds + L::ZBL + t * LD, sbl, cg, a.eps, xh, rstd);
#pragma unroll
      for (int j = 0; j < NJD; ++j) {
        const int o = cg + GW * j;
        if (t < K)
          IO::store1(static_cast<elem*>(a.out) + row * D + o, lds[L::XQ + t * LD + o] + (sgam[o] * xh[j] + sbet[o]));
        lds[L::ZL + t * LD + o] *= last;
      }
#pragma unroll
      for (int i = 0; i < NL; ++i)
#pragma unroll
        for (int j = 0; j < NJM; ++j) lds[L::BA + i * TM + t * LM + cg + GW * j] *= last;
    }
    __syncthreads();
    // ---- W[i] -= X[i]^T G[i]l ; b[i] -= colsum(G[i]l)
    mm_rank<2, NW, NBM, 4>(W[0], M, lds + L::XK, 1, LD, lds + L::BA, LM, 1, NTD, NTM, wave, lane);
#pragma unroll
    for (int i = 1; i < NL; ++i)
      mm_rank<2, NW, NBM, 4>(W[i], M, lds + L::BB + (i - 1) * TM, 1, LM, lds + L::BA + i * TM, LM, 1, NTM, NTM, wave, lane);
    mm_rank<2, NW, NBD, 4>(W[NL], D, lds + L::BB + (NL - 1) * TM, 1, LM, lds + L::ZL, LD, 1, NTM, NTD, wave, lane);
#pragma unroll
    for (int i = 0; i < NL; ++i)
      for (int e = tid; e < M; e += 512) {
        float s = 0.f;
        for (int r = 0; r < 16; ++r) s += lds[L::BA + i * TM + r * LM + e];
        lds[L::bh + i * M + e] -= s;
      }
    if (tid < D) {
      float s = 0.f;
      for (int r = 0; r < 16; ++r) s += lds[L::ZL + r * LD + tid];
      sbl[tid] -= s;
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < NL; ++i)
    for (int e = tid; e < M; e += 512) a.b[i][bh * M + e] = lds[L::bh + i * M + e];
  for (int e = tid; e < D; e += 512) a.b[NL][bh * D + e] = sbl[e];
}

}  // namespace ttt
