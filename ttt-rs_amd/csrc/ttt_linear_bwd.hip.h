// TTT-Linear fused backward for gfx950: one workgroup (4 wavefronts) per (batch, head).
//
// Arithmetic: reverse scan over mini-batches (reference
// rust/fused/src/linear_fused_tile/backward/kernel.rs:253-429) of the one-stage backward
// (backward/stage.rs:42-1006; second-order LayerNorm term layer_norm.rs:428-709), with the
// state entering each stage rebuilt from the forward's checkpoints by re-running the state
// update (backward/kernel.rs:134-246).  Semantics kept from the reference: upstream gradients
// of the final state default to zero, d_token_eta is per position and summed over batch and
// heads with atomics, d_gamma/d_beta carry both the output-LayerNorm and the through-G terms.
//
// Design: every operand of a stage ([16 x d] tiles, the [d x d] state W and its gradient dW,
// the [16 x 16] causal matrices) lives in LDS as f32 with a padded row stride, and all
// contractions are true-f32 MFMA (v_mfma_f32_16x16x4_f32) whose A/B elements are read from
// LDS with arbitrary (row, column) strides, so transposed operands cost nothing extra.  dW and
// db stay in LDS for the whole scan (the reference round-trips them through global memory
// every stage).  Elementwise work uses thread (t = tid/16, cg = tid%16) for token t and
// features cg, cg+16, ...; row statistics are 16-lane shuffles.  Arithmetic is f32 for both
// I/O dtypes; bf16 tensors are converted at the tile loads and stores.  The barriers inside the scan order
// LDS traffic only (lds_barrier): a full __syncthreads() would also wait for every global store and for
// the contended d_token_eta atomics of the mini-batch.
#pragma once
#include "ttt_engine.hip.h"

namespace ttt {

struct LinearBwdArgs {
  const void* xq;
  const void* xk;
  const void* xv;
  const float* token_eta;
  const void* lr;
  const float* gamma;
  const float* beta;
  const float* W_ckpt;
  const float* b_ckpt;
  const void* d_out;
  const float* d_W_out;
  const float* d_b_out;
  void* d_xq;
  void* d_xk;
  void* d_xv;
  float* d_W0;
  float* d_b0;
  void* d_lr;
  float* d_token_eta;
  float* d_gamma;
  float* d_beta;
  int B, H, seq, seq_stride, K, n_stages, ckpt_interval, n_ckpt;
  int ckpt_packed;  // W checkpoints as bf16 operand fragments (register-resident kernels, bf16 I/O)
  float eps;
};

// MT tiles of 16 token rows: mini_batch <= KT = 16 MT.  MT = 2 serves the reference's (mini_batch 32, head_dim 32)
// tile (rust/fused/src/linear_fused_tile/mod.rs:38).
// WG: the state W of a mini-batch is read in place from its checkpoint in global memory (one checkpoint per
// mini-batch); DG: the state gradient dW lives in the d_W0 output buffer for the whole scan.  With both, head_dim 128
// fits: LDS then holds only the tiles of a stage.
template <int D, int MT = 1, bool WG = false, bool DG = false>
struct BwdLds {
  static constexpr int KT = 16 * MT;
  static constexpr int LD = D + 4;     // padded row stride (floats) of every [*, D] array
  static constexpr int LK = KT + 1;    // row stride of the [KT x KT] matrices
  static constexpr int TILE = KT * LD;
  static constexpr int WSZ = D * LD;
  static constexpr int KK = KT * LK;
  // offsets in floats
  static constexpr int W = 0, dW = W + (WG ? 0 : WSZ);
  static constexpr int XQ = dW + (DG ? 0 : WSZ), XK = XQ + TILE, TG = XK + TILE, DO = TG + TILE, XH = DO + TILE,
                       G = XH + TILE, XH2 = G + TILE, DZB = XH2 + TILE, S = DZB + TILE,
                       TMP = S + TILE, DK = TMP + TILE, DZ1 = DK + TILE, DQ = DZ1 + TILE,
                       DGM = DQ + TILE;
  static constexpr int A = DGM + TILE, ETA = A + KK, M = ETA + KK, P = M + KK, DA = P + KK,
                       DETA = DA + KK;
  static constexpr int b = DETA + KK, db = b + D, gam = db + D, bet = gam + D, lr = bet + D,
                       te = lr + KT, rstd1 = te + KT, dlast = rstd1 + KT, END = dlast + KT;
  static_assert(sizeof(float) * END <= 160 * 1024, "exceeds the 160 KiB of LDS of a gfx950 CU");
  static constexpr size_t BYTES = sizeof(float) * END;
};

// BF: the operands of every product are rounded to bf16 (bf16 I/O when this kernel is the library's own choice, not
// a request for f32 products): an eighth of the matrix-pipe time; tiles, state and accumulation stay f32.
template <class T, int D, int MT = 1, bool WG = false, bool DG = false, bool BF = false>
__global__ void __launch_bounds__(256 * MT) ttt_linear_bwd_kernel(LinearBwdArgs a) {
  using IO = Io<T>;
  using elem = typename IO::elem;
  using L = BwdLds<D, MT, WG, DG>;
  using E = Eng<BF>;
  constexpr int LD = L::LD, LK = L::LK, KT = L::KT, NJ = D / 16, NTH = 256 * MT, NW = 4 * MT;
  constexpr int NB2 = NJ >= 2 ? 2 : 1;  // tile columns per job of a [16 x D] product
  constexpr float inv_d = 1.0f / D;
  extern __shared__ __attribute__((aligned(16))) float lds[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int t = tid >> 4, cg = tid & 15;  // elementwise mapping: token t, features cg + 16 j
  const size_t bh = blockIdx.x;
  const int h = (int)(bh % a.H);
  const int K = a.K;

  float* sW = lds + L::W;
  // W(k, n) = Wp[k * wld + n]: the LDS copy, or (WG) the checkpoint of the mini-batch itself, set per stage
  const float* Wp = sW;
  constexpr int wld = WG ? D : LD;
  // dW likewise: LDS, or (DG) the caller's d_W0 buffer of this unit
  float* sdW = DG ? a.d_W0 + bh * (size_t)D * D : lds + L::dW;
  constexpr int dld = DG ? D : LD;
  // stores to dW in global memory must have landed before another wave reads them: a full barrier then
  auto bar = [&]() {
    if constexpr (WG || DG)
      __syncthreads();
    else
      lds_barrier();
  };
  float* sb = lds + L::b;
  float* sdb = lds + L::db;
  float* sgam = lds + L::gam;
  float* sbet = lds + L::bet;
  float* slr = lds + L::lr;
  float* ste = lds + L::te;

  // ---- one-time setup
  for (int i = tid; i < D; i += NTH) {
    sgam[i] = a.gamma[h * D + i];
    sbet[i] = a.beta[h * D + i];
    sdb[i] = a.d_b_out ? a.d_b_out[bh * D + i] : 0.f;
  }
  for (int i = tid; i < D * D; i += NTH) {
    const int r = i / D, cc = i - r * D;
    sdW[r * dld + cc] = a.d_W_out ? a.d_W_out[bh * D * D + i] : 0.f;
  }
  if (tid < KT) ste[tid] = (tid < K) ? a.token_eta[tid] : 0.f;
  float dgam_acc[NJ], dbet_acc[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) dgam_acc[j] = dbet_acc[j] = 0.f;
  __syncthreads();
  const float te_last = ste[K - 1];

  // load one [K x D] activation tile into LDS as f32 (rows >= K are zero)
  auto load_tile = [&](float* dst, const void* src, int stage) {
    const elem* p = static_cast<const elem*>(src) + (bh * (size_t)a.seq_stride + (size_t)stage * K + t) * D;
#pragma unroll
    for (int j = 0; j < NJ; ++j) dst[t * LD + cg + 16 * j] = (t < K) ? IO::load1(p + cg + 16 * j) : 0.f;
  };
  auto load_lr = [&](int stage) {
    if (tid < KT)
      slr[tid] = (tid < K) ? IO::load1(static_cast<const elem*>(a.lr) + bh * (size_t)a.seq_stride + (size_t)stage * K + tid) : 0.f;
  };

  // LayerNorm + L2-gradient pieces for this thread's token (row of `z` + bias): returns x_hat,
  // rstd and G for its NJ features.
  auto ln1 = [&](const float* z, const float* tg, float (&xh)[NJ], float (&Gv)[NJ], float& rstd) {
    float zv[NJ], s = 0.f;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      zv[j] = z[t * LD + cg + 16 * j] + sb[cg + 16 * j];
      s += zv[j];
    }
    const float mu = row16_sum(s) * inv_d;
    float v = 0.f;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      zv[j] -= mu;
      v += zv[j] * zv[j];
    }
    rstd = __builtin_amdgcn_rsqf(row16_sum(v) * inv_d + a.eps);
    float gx[NJ], s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const float ga = sgam[cg + 16 * j];
      xh[j] = zv[j] * rstd;
      gx[j] = (ga * xh[j] + sbet[cg + 16 * j] - tg[t * LD + cg + 16 * j]) * ga;
      s1 += gx[j];
      s2 += gx[j] * xh[j];
    }
    s1 = row16_sum(s1) * inv_d;
    s2 = row16_sum(s2) * inv_d;
#pragma unroll
    for (int j = 0; j < NJ; ++j) Gv[j] = (gx[j] - s1 - xh[j] * s2) * rstd;
  };

  // ---- register prefetch of everything a stage reads from HBM: the checkpoint (W, b) and the four
  // activation tiles of the NEXT stage to be processed are fetched while the current one computes,
  // and only copied into LDS at the top of that stage.  Thread tid owns EP contiguous elements of
  // each [16 x D] tile and WP float4 pieces of the checkpoint.
  constexpr int EP = D / 16;          // KT*D elements / NTH threads
  constexpr int WP = WG ? 1 : (D * D + 4 * NTH - 1) / (4 * NTH);  // float4 pieces of the checkpoint per thread
  constexpr bool WALL = D * D % (4 * NTH) == 0;          // every thread has all WP pieces
  const int pt = (tid * EP) / D, pc = (tid * EP) % D;  // token row / first feature of this thread's piece
  struct Prefetch {
    f32x4 w[WP];
    float b, lr;
    float q[EP], k[EP], v[EP], o[EP];
  } pre;
  auto fetch_tile = [&](float (&dst)[EP], const void* src, int stage) {
    const elem* p = static_cast<const elem*>(src) + (bh * (size_t)a.seq_stride + (size_t)stage * K + pt) * D + pc;
#pragma unroll
    for (int e = 0; e < EP; ++e) dst[e] = (pt < K) ? IO::load1(p + e) : 0.f;
  };
  auto fetch_stage = [&](int stage) {
    const int ckp = stage / a.ckpt_interval;
    const f32x4* Wg = reinterpret_cast<const f32x4*>(a.W_ckpt + (bh * a.n_ckpt + ckp) * D * D);
    if constexpr (!WG) {
#pragma unroll
      for (int i = 0; i < WP; ++i) pre.w[i] = Wg[(WALL || 4 * (tid + NTH * i) < D * D) ? tid + NTH * i : 0];
    }
    pre.b = (tid < D) ? a.b_ckpt[(bh * a.n_ckpt + ckp) * D + tid] : 0.f;
    pre.lr = (tid < K) ? IO::load1(static_cast<const elem*>(a.lr) + bh * (size_t)a.seq_stride + (size_t)stage * K + tid) : 0.f;
    fetch_tile(pre.q, a.xq, stage);
    fetch_tile(pre.k, a.xk, stage);
    fetch_tile(pre.v, a.xv, stage);
    fetch_tile(pre.o, a.d_out, stage);
  };
  auto commit_state = [&]() {
    if constexpr (!WG) {
#pragma unroll
      for (int i = 0; i < WP; ++i) {
        const int idx = (tid + NTH * i) * 4;
        if (WALL || idx < D * D) *reinterpret_cast<f32x4*>(sW + (idx / D) * LD + (idx % D)) = pre.w[i];
      }
    }
    if (tid < D) sb[tid] = pre.b;
  };
  auto commit_tiles = [&]() {
#pragma unroll
    for (int e = 0; e < EP; ++e) {
      lds[L::XQ + pt * LD + pc + e] = pre.q[e];
      lds[L::XK + pt * LD + pc + e] = pre.k[e];
      lds[L::TG + pt * LD + pc + e] = pre.v[e] - pre.k[e];
      lds[L::DO + pt * LD + pc + e] = pre.o[e];
    }
    if (tid < KT) slr[tid] = pre.lr;
  };
  fetch_stage(a.n_stages - 1);

  for (int st = a.n_stages - 1; st >= 0; --st) {
    // ================= state entering stage st: checkpoint + re-simulated updates
    const int ck = st / a.ckpt_interval;
    if constexpr (WG) Wp = a.W_ckpt + (bh * a.n_ckpt + st) * (size_t)D * D;  // checkpoint_interval is 1
    commit_state();
    for (int s2 = ck * a.ckpt_interval; s2 < st; ++s2) {
      bar();
      load_tile(lds + L::XK, a.xk, s2);
      load_tile(lds + L::TG, a.xv, s2);
      load_lr(s2);
      bar();
#pragma unroll
      for (int j = 0; j < NJ; ++j) lds[L::TG + t * LD + cg + 16 * j] -= lds[L::XK + t * LD + cg + 16 * j];
      E::template lds<0, NW>(lds + L::XH, LD, lds + L::XK, LD, 1, sW, LD, 1, MT, NJ, D, wave, lane);
      bar();
      {
        float xh[NJ], Gv[NJ], rstd;
        ln1(lds + L::XH, lds + L::TG, xh, Gv, rstd);
        const float last = te_last * slr[t];
#pragma unroll
        for (int j = 0; j < NJ; ++j) lds[L::G + t * LD + cg + 16 * j] = Gv[j] * last;
      }
      bar();
      // W -= XK^T (last * G) ; b -= colsum(last * G)      (linear.rs:134-144)
      E::template lds<2, NW, NJ, 4>(sW, LD, lds + L::XK, 1, LD, lds + L::G, LD, 1, NJ, NJ, KT, wave, lane);
      if (tid < D) {
        float s = 0.f;
        for (int r = 0; r < KT; ++r) s += lds[L::G + r * LD + tid];
        sb[tid] -= s;
      }
    }
    if (ck * a.ckpt_interval < st) bar();  // the re-simulation used the XK / target tiles

    // ================= this stage's tiles (target = XV - XK formed on the way), then prefetch the next
    commit_tiles();
    bar();
    if (st > 0) fetch_stage(st - 1);
    // Z1 = XK W ; Zq = XQ W ; A = XQ XK^T
    // every product is cut into jobs of NB2 tile columns: two or more accumulator chains per wave keep the
    // matrix pipe busy (a single chain waits out the full MFMA latency between dependent steps)
    E::template lds<0, NW, NB2>(lds + L::XH, LD, lds + L::XK, LD, 1, Wp, wld, 1, MT, NJ, D, wave, lane, 0);
    E::template lds<0, NW, NB2>(lds + L::XH2, LD, lds + L::XQ, LD, 1, Wp, wld, 1, MT, NJ, D, wave, lane, 2);
    E::template lds<0, NW>(lds + L::A, LK, lds + L::XQ, LD, 1, lds + L::XK, 1, LD, MT, MT, D, wave, lane, 1);
    bar();

    // ================= forward intermediates: x_hat, rstd, G; eta, A (tril), M = eta (1 + A)
    float xh[NJ], Gv[NJ], rstd1;
    ln1(lds + L::XH, lds + L::TG, xh, Gv, rstd1);
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      lds[L::XH + t * LD + cg + 16 * j] = xh[j];
      lds[L::G + t * LD + cg + 16 * j] = Gv[j];
    }
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const int s = cg + 16 * i;  // (t, s) entry of the [KT x KT] matrices
      const bool low = s <= t;
      const float at = low ? lds[L::A + t * LK + s] : 0.f;
      const float et = low ? ste[t] * slr[s] : 0.f;
      lds[L::A + t * LK + s] = at;
      lds[L::ETA + t * LK + s] = et;
      lds[L::M + t * LK + s] = et * (1.f + at);
    }
    bar();
    // Zb = XQ W - M G  (+ b added when read)
    E::template lds<2, NW, 1, 4>(lds + L::XH2, LD, lds + L::M, LK, 1, lds + L::G, LD, 1, MT, NJ, KT, wave, lane);
    bar();

    // ================= output LayerNorm and its backward (stage 4)
    {
      float zv[NJ], s = 0.f;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        zv[j] = lds[L::XH2 + t * LD + cg + 16 * j] + sb[cg + 16 * j];
        s += zv[j];
      }
      const float mu = row16_sum(s) * inv_d;
      float v = 0.f;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        zv[j] -= mu;
        v += zv[j] * zv[j];
      }
      const float rstd2 = __builtin_amdgcn_rsqf(row16_sum(v) * inv_d + a.eps);
      float gx2[NJ], s1 = 0.f, s2 = 0.f;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const float x2 = zv[j] * rstd2;
        const float dO = lds[L::DO + t * LD + cg + 16 * j];
        dgam_acc[j] += dO * x2;
        dbet_acc[j] += dO;
        gx2[j] = dO * sgam[cg + 16 * j];
        s1 += gx2[j];
        s2 += gx2[j] * x2;
        zv[j] = x2;
      }
      s1 = row16_sum(s1) * inv_d;
      s2 = row16_sum(s2) * inv_d;
#pragma unroll
      for (int j = 0; j < NJ; ++j) lds[L::DZB + t * LD + cg + 16 * j] = (gx2[j] - s1 - zv[j] * s2) * rstd2;
    }
    bar();

    // ================= P = dZb G^T ; dQ = dZb W^T ; S = XK dW ; TMP = G dW^T
    // a transposed matrix in global memory is contiguous along k: loaded four lanes to a row (BG)
    E::template lds<0, NW, NB2, 4, WG>(lds + L::DQ, LD, lds + L::DZB, LD, 1, Wp, 1, wld, MT, NJ, D, wave, lane, 0);
    E::template lds<0, NW, NB2, 4, DG>(lds + L::TMP, LD, lds + L::G, LD, 1, sdW, 1, dld, MT, NJ, D, wave, lane, 0);
    E::template lds<0, NW, NB2>(lds + L::S, LD, lds + L::XK, LD, 1, sdW, dld, 1, MT, NJ, D, wave, lane, 2);
    E::template lds<0, NW>(lds + L::P, LK, lds + L::DZB, LD, 1, lds + L::G, 1, LD, MT, MT, D, wave, lane, 3);
    bar();

    // ================= dA, d eta ; S += db ; dlast
    {
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const int s = cg + 16 * i;
        const bool low = s <= t;
        const float p = lds[L::P + t * LK + s];
        lds[L::DA + t * LK + s] = low ? -p * lds[L::ETA + t * LK + s] : 0.f;
        lds[L::DETA + t * LK + s] = low ? -p * (1.f + lds[L::A + t * LK + s]) : 0.f;
      }
      float dl = 0.f;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const float sv = lds[L::S + t * LD + cg + 16 * j] + sdb[cg + 16 * j];
        lds[L::S + t * LD + cg + 16 * j] = sv;
        dl += Gv[j] * sv;
      }
      dl = row16_sum(dl);
      if (cg == 0) lds[L::dlast + t] = -dl;
    }
    bar();

    // ================= dQ += dA XK ; dK = dA^T XQ ; DGM = M^T dZb ; dW += XQ^T dZb ; db += colsum(dZb)
    E::template lds<1, NW, NJ, 4>(lds + L::DQ, LD, lds + L::DA, LK, 1, lds + L::XK, LD, 1, MT, NJ, KT, wave, lane, 0);
    E::template lds<0, NW, NJ, 4>(lds + L::DK, LD, lds + L::DA, 1, LK, lds + L::XQ, LD, 1, MT, NJ, KT, wave, lane, 1);
    E::template lds<0, NW, NJ, 4>(lds + L::DGM, LD, lds + L::M, 1, LK, lds + L::DZB, LD, 1, MT, NJ, KT, wave, lane, 2);
    E::template lds<1, NW, NJ, 4>(sdW, dld, lds + L::XQ, 1, LD, lds + L::DZB, LD, 1, NJ, NJ, KT, wave, lane);
    if (tid < D) {
      float s = 0.f;
      for (int r = 0; r < KT; ++r) s += lds[L::DZB + r * LD + tid];
      sdb[tid] += s;
    }
    // d lr and d token_eta (KT threads each, in different waves)
    if (tid < KT) {
      float s = 0.f;
      for (int r = 0; r < KT; ++r) s += lds[L::DETA + r * LK + tid] * ste[r];
      s += te_last * lds[L::dlast + tid];
      if (tid < K) IO::store1(static_cast<elem*>(a.d_lr) + bh * (size_t)a.seq_stride + (size_t)st * K + tid, s);
    } else if (tid >= 64 && tid < 64 + KT) {
      const int tt = tid - 64;
      float s = 0.f;
      for (int r = 0; r < KT; ++r) s += lds[L::DETA + tt * LK + r] * slr[r];
      if (tt == K - 1)
        for (int r = 0; r < KT; ++r) s += lds[L::dlast + r] * slr[r];
      if (tt < K) atomicAdd(a.d_token_eta + (size_t)st * K + tt, s);
    }
    bar();

    // ================= through G: second-order LayerNorm (stage 2), token-local
    {
      const float last = te_last * slr[t];
      float dG[NJ], u[NJ], gO[NJ], gx[NJ], s1 = 0.f, s2 = 0.f, sgx = 0.f;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int o = cg + 16 * j;
        dG[j] = -lds[L::DGM + t * LD + o] - last * lds[L::S + t * LD + o];
        u[j] = -dG[j] * rstd1;
        gO[j] = sgam[o] * xh[j] + sbet[o] - lds[L::TG + t * LD + o];
        gx[j] = gO[j] * sgam[o];
        s1 += u[j];
        s2 += u[j] * xh[j];
        sgx += gx[j] * xh[j];
      }
      s1 = row16_sum(s1) * inv_d;
      s2 = row16_sum(s2) * inv_d;
      sgx = row16_sum(sgx) * inv_d;
      float dxh[NJ], dy[NJ], q1 = 0.f, q2 = 0.f;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int o = cg + 16 * j;
        const float dgx = -u[j] + s1 + xh[j] * s2;
        dy[j] = sgam[o] * dgx;
        dgam_acc[j] += gO[j] * dgx + dy[j] * xh[j];
        dbet_acc[j] += dy[j];
        dxh[j] = dy[j] * sgam[o] + gx[j] * s2 + u[j] * sgx;
        q1 += dxh[j];
        q2 += dxh[j] * xh[j] + dG[j] * Gv[j];
      }
      q1 = row16_sum(q1) * inv_d;
      const float dsig = -row16_sum(q2) * rstd1;  // d loss / d sigma
      elem* pv = static_cast<elem*>(a.d_xv) + (bh * (size_t)a.seq_stride + (size_t)st * K + t) * D;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int o = cg + 16 * j;
        lds[L::DZ1 + t * LD + o] = (dxh[j] - q1) * rstd1 + xh[j] * dsig * inv_d;
        // dXV = dT = -dy ; dXK collects dA^T XQ - last (G dW'^T) - dT
        if (t < K) IO::store1(pv + o, -dy[j]);
        lds[L::DK + t * LD + o] += dy[j] - last * lds[L::TMP + t * LD + o];
      }
    }
    bar();

    // ================= dK += dZ1 W^T ; dW += XK^T dZ1 ; db += colsum(dZ1)
    E::template lds<1, NW, NB2, 4, WG>(lds + L::DK, LD, lds + L::DZ1, LD, 1, Wp, 1, wld, MT, NJ, D, wave, lane, 2);
    E::template lds<1, NW, NJ, 4>(sdW, dld, lds + L::XK, 1, LD, lds + L::DZ1, LD, 1, NJ, NJ, KT, wave, lane);
    if (tid < D) {
      float s = 0.f;
      for (int r = 0; r < KT; ++r) s += lds[L::DZ1 + r * LD + tid];
      sdb[tid] += s;
    }
    bar();

    // ================= store dXQ = dO + dQ, dXK
    if (t < K) {
      elem* pq = static_cast<elem*>(a.d_xq) + (bh * (size_t)a.seq_stride + (size_t)st * K + t) * D;
      elem* pk = static_cast<elem*>(a.d_xk) + (bh * (size_t)a.seq_stride + (size_t)st * K + t) * D;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int o = cg + 16 * j;
        IO::store1(pq + o, lds[L::DQ + t * LD + o] + lds[L::DO + t * LD + o]);
        IO::store1(pk + o, lds[L::DK + t * LD + o]);
      }
    }
    bar();
  }

  // ---- results carried over the whole scan
  if constexpr (!DG) {
    for (int i = tid; i < D * D; i += NTH) {
      const int r = i / D, cc = i - r * D;
      a.d_W0[bh * D * D + i] = sdW[r * LD + cc];
    }
  }
  if (tid < D) a.d_b0[bh * D + tid] = sdb[tid];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    lds[L::XQ + t * LD + cg + 16 * j] = dgam_acc[j];
    lds[L::XK + t * LD + cg + 16 * j] = dbet_acc[j];
  }
  __syncthreads();
  if (tid < D) {
    float sg = 0.f, sbt = 0.f;
    for (int r = 0; r < KT; ++r) {
      sg += lds[L::XQ + r * LD + tid];
      sbt += lds[L::XK + r * LD + tid];
    }
    atomicAdd(a.d_gamma + h * D + tid, sg);
    atomicAdd(a.d_beta + h * D + tid, sbt);
  }
}

}  // namespace ttt
