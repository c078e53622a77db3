// TTT-MLP multi-stage forward for gfx950 with the whole state resident in registers.
//
// Arithmetic: reference rust/core/src/mlp.rs:127-208 (one mini-batch) looped over the sequence as
// rust/core/src/inner.rs:25-50; GELU constants rust/thundercube/src/unary_ops.rs:136-173.
//
// One workgroup of eight waves per (batch, head).  The hidden axis (4 d units) is cut into eight
// slices; wave w keeps, as MFMA accumulator tiles in VGPRs for the whole sequence,
//     W1[:, slice]  (d x 4d/8)   rows (d features) in registers, hidden units across lanes
//     W2[slice, :]  (4d/8 x d)   hidden units in registers, d features across lanes
//     b1[slice]
// which is 2 * (d/16) * (d/32) tiles = 144 VGPRs at d = 96.  Everything that is elementwise in the
// hidden axis (Z1, GELU, G1, Zbar1, Xbar2, both state updates) stays inside the wave.  The three
// contractions OVER the hidden axis (Z2 = X2 W2, Zbar2 = Xbar2 W2, A2 = Xbar2 X2^T) are split-k:
// every wave writes its partial tiles to LDS and wave I < d/16 (a "reducer") adds up d-feature
// tile I, owns b2 / gamma / beta of those sixteen features and does the LayerNorm work on them.
//
// Per mini-batch there are three barriers on the recurrence W -> Z1 -> X2 -> Z2 -> G2 -> G1 -> W':
//   B1  partial Z2 tiles (and last mini-batch's partial Zbar2 / A2) are in LDS
//   B2  the reducers' row moments (six for the LN-L2 gradient of this mini-batch, two for the output
//       LayerNorm of the previous one) are in LDS
//   B3  G2 (as both operand orientations, already scaled by -eta_last) is in LDS
// The output of mini-batch t needs nothing the recurrence waits for, so it is finished one
// mini-batch late, inside the reducers' part of mini-batch t+1, and shares its barriers.
//
// An odd hidden tile at the end of a split-k chain is issued as a k = 32 MFMA with a zero second
// half, not as a k = 16 one: a 16x16x16 bf16 MFMA accumulating straight onto the result of a
// 16x16x32 one was measured to give wrong sums on gfx950 with this toolchain.
//
// Contractions over the d axis against W2 (G1 = G2 W2^T) need W2 tiles with d in the k position;
// the accumulator layout has it across lanes, so those operand tiles are transposed on the matrix
// pipe (one 16x16x16 MFMA against an identity fragment each).
#pragma once
#include "ttt_engine_fwd.hip.h"
#include "ttt_linear_fwd_mw.hip.h"

namespace ttt {

template <int D, int ES>
struct MlpRrLds {
  static constexpr int NW = 8, NT = D / 16;
  static constexpr int TILE = 16 * D * ES;    // one [16 x d] input tile, rows unpadded
  static constexpr int IN1 = 3 * TILE;        // xq, xk, xv tiles of one mini-batch
  static constexpr int IN = 0;                // [3 buffers][3][16][d]
  static constexpr int LR = IN + 3 * IN1;     // [3][16] floats
  static constexpr int P1 = LR + 3 * 64 + 64;  // [NW][NT][64] f32x4: partial Z2^T tiles
  static constexpr int P2 = P1 + NW * NT * 1024;  // partial Zbar2^T tiles
  static constexpr int PA = P2 + NW * NT * 1024;  // [NW][64] f32x4: partial A2^T
  static constexpr int EX = PA + NW * 1024;       // [8 sums][2][16 tokens] f32x4 (reducer index % 4)
  static constexpr int GT = EX + 8 * 2 * 16 * 16;  // [NT][64] frag: G2^T tiles (d along k)
  static constexpr int GD = GT + NT * 64 * 4 * ES;  // [NT][64] frag: G2 tiles (tokens along k)
  static constexpr int KD = GD + NT * 64 * 4 * ES;  // [2][NT][64] frag: XK tiles (tokens along k)
  static constexpr int PRM = KD + 2 * NT * 64 * 4 * ES;  // gamma[d], beta[d], b1[4d] floats
  static constexpr int EXO = PRM + (2 * D + 4 * D) * 4;    // [2 sums][2][16 tokens] f32x4 (output tile % 4)
  static constexpr int BYTES = EXO + 2 * 2 * 16 * 16;
  static_assert(BYTES <= 160 * 1024, "exceeds the 160 KiB of LDS of a gfx950 CU");
  static_assert(NT <= NW && D % 32 == 0, "one reducer wave per d-feature tile");
  static_assert(TILE % 1024 == 0 && P1 % 16 == 0, "input tiles are staged in 1 KiB wave blocks");
};

// Makes the compiler forget what it knows about v.  The bf16 operand copies of the W2 tiles are
// needed at three places of a mini-batch; without this the compiler keeps the converted copies
// (36 VGPRs at d = 96) alive across the barriers and spills state tiles to scratch instead.
__device__ __forceinline__ void forget(f32x4& v) { asm volatile("" : "+v"(v)); }
// Orders memory accesses around the point where v is complete: keeps a reduction loop from issuing
// all its LDS loads (four VGPRs each) before the first add.
__device__ __forceinline__ void pin(f32x4& v) { asm volatile("" : "+v"(v)::"memory"); }
__device__ __forceinline__ void pin(float& v) { asm volatile("" : "+v"(v)::"memory"); }

// ---- Centred second layer.  The TTT-MLP loop looks at W2 and b2 only through LayerNorm (Z2 = X2 W2 + b2 feeds the
// LN-L2 gradient, Zbar2 the output LayerNorm) and through G1 = (G2 W2^T) gelu'(Z1), where the rows of G2 sum to zero.
// So, exactly as for the TTT-Linear state (centre_state in ttt_linear_fwd_mw.hip.h), the kernels carry
// W2 - m 1^T (m_i = mean over the d columns of row i) and b2 - mean(b2): the dropped part shifts every feature of a
// token by the same amount (discarded by both LayerNorms) and meets only zero row sums in G2 W2^T; the updates
// W2 += X2^T G2'', b2 += colsum G2'' do not move m or mean(b2).  Z2 and Zbar2 then have row means at rounding
// level, which keeps the one-pass statistics and the bf16 operand images of W2 accurate for any offset of its rows.
//
// Mean of each of the four rows (4g + r of a 16-row tile) of a [16 x d] tile held as NT accumulator tiles
// (columns: tile I, lane c), the same float in all sixteen lanes of a row.  Made opaque so that the subtraction
// that follows is a subtraction of this rounded number wherever it is repeated (no fused multiply-add).
template <int NT>
__device__ __forceinline__ f32x4 row_means16(const f32x4 (&t)[NT], float inv_d) {
  f32x4 m;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    float p = 0.f;
#pragma unroll
    for (int I = 0; I < NT; ++I) p += t[I][r];
    m[r] = row16_first(row16_sum_dpp(p)) * inv_d;
  }
  asm volatile("" : "+v"(m));
  return m;
}
// mean of d floats in global memory, the same float in every lane, opaque as above
__device__ __forceinline__ float mean_of(const float* p, int d, float inv_d) {
  float s = 0.f;
  for (int f = 0; f < d; ++f) s += p[f];
  s *= inv_d;
  asm volatile("" : "+v"(s));
  return s;
}

// The LDS addresses derived from the lane index are many (the regions span 150 KiB, beyond the
// 64 KiB reach of an instruction offset) and all loop-invariant: hoisted out of the loop they are
// spilled and reloaded from scratch.  Hiding the lane index from the optimiser at the start of each
// phase makes them cheap phase-local recomputations instead.
#define RELANE() asm volatile("" : "+v"(lane))

template <class T, int D>
__global__ void __launch_bounds__(512) ttt_mlp_fwd_rr_kernel(Problems<MlpFwdArgs> problems) {
  const MlpFwdArgs& a = problems.p[blockIdx.y];
  using IO = Io<T>;
  using frag = typename IO::frag;
  using elem = typename IO::elem;
  constexpr int ES = sizeof(elem);
  using L = MlpRrLds<D, ES>;
  constexpr int NW = 8, NT = D / 16, F = 4 * D, HT = F / 16 / NW;
  constexpr float inv_d = 1.0f / D;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  // the wave index is read through an SGPR so that everything keyed on it is scalar control flow
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6);
  int lane = tid & 63;  // refreshed (see RELANE) at every phase of the main loop
  const int c = lane & 15, g = lane >> 4;
  const size_t bh = blockIdx.x;
  const int h = (int)(bh % a.H), K = a.K;
  const bool red = w < NT;  // this wave reduces d-feature tile w

  f32x4* const P1 = reinterpret_cast<f32x4*>(smem + L::P1);
  f32x4* const P2 = reinterpret_cast<f32x4*>(smem + L::P2);
  f32x4* const PA = reinterpret_cast<f32x4*>(smem + L::PA);
  float* const EX = reinterpret_cast<float*>(smem + L::EX);
  float* const EXO = reinterpret_cast<float*>(smem + L::EXO);
  frag* const GT = reinterpret_cast<frag*>(smem + L::GT);
  frag* const GD = reinterpret_cast<frag*>(smem + L::GD);
  frag* const KD = reinterpret_cast<frag*>(smem + L::KD);
  uint32_t* const LRs = reinterpret_cast<uint32_t*>(smem + L::LR);
  float* const GAM = reinterpret_cast<float*>(smem + L::PRM);
  float* const BET = GAM + D;
  float* const B1s = BET + D;  // b1: each wave reads and updates only its own slice

  // scale folding as in the TTT-Linear kernels: G'' = -sc lr G, M'' = (token_eta[t] / sc)(1 + A)
  const float te_last = a.token_eta[K - 1];
  const bool upd = te_last != 0.f;
  const float sc = upd ? te_last : 1.f;
  const float rho_c = (c < K) ? a.token_eta[c] / sc : 0.f;
  const frag ident = identity_frag<T>(c, g);
  const frag ones = splat_frag<T>(1.f);
  const size_t sb = a.state_per_batch ? bh : (size_t)h;
  const int own = own_offset<1>(red ? w : 0, 0, g);  // first of this lane's four features of tile w

  // ---- state and parameters
  f32x4 W1c[NT][HT], W2c[HT][NT];
  {
    const float* W1 = a.W1_0 + sb * (size_t)D * F;
    const float* W2 = a.W2_0 + sb * (size_t)D * F;
#pragma unroll
    for (int j = 0; j < HT; ++j) {
      const int hb = 16 * (w * HT + j);
#pragma unroll
      for (int I = 0; I < NT; ++I)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          W1c[I][j][r] = W1[(size_t)feat(I, 4 * g + r) * F + hb + c];
          W2c[j][I][r] = W2[(size_t)(hb + 4 * g + r) * D + feat(I, c)];
        }
    }
  }
  f32x4 b2T;
  float sum_a = 0.f;
#pragma unroll
  for (int r = 0; r < 4; ++r) b2T[r] = a.b2_0[sb * D + own + r];
  // the second layer is carried centred (see row_means16)
#pragma unroll
  for (int j = 0; j < HT; ++j) {
    const f32x4 m = row_means16<NT>(W2c[j], inv_d);
#pragma unroll
    for (int I = 0; I < NT; ++I) W2c[j][I] -= m;
  }
  b2T -= mean_of(a.b2_0 + sb * D, D, inv_d);
  for (int f = 0; f < D; ++f) sum_a += a.gamma[h * D + f] * a.gamma[h * D + f];
  for (int i = tid; i < D; i += 512) {
    GAM[i] = a.gamma[h * D + i];
    BET[i] = a.beta[h * D + i];
  }
  for (int i = tid; i < F; i += 512) B1s[i] = a.b1_0[sb * F + i];

  // ---- staging of the xq / xk / xv rows of a mini-batch: global -> LDS without passing through
  // registers, in wave blocks of 64 lanes x 16 bytes.  A block never straddles two tensors; lanes
  // whose token is past a short mini-batch are masked off and their LDS rows keep the zeros
  // written below.  Three buffers: mini-batch st+1 is fetched while st is computed, and rows of
  // st are still read (for the W1 update) after the slowest wave has started st+1's fetch.
  constexpr int NBLK = L::IN1 / 1024, NBI = (NBLK + NW - 1) / NW;
  int goff[NBI];
#pragma unroll
  for (int it = 0; it < NBI; ++it) {
    const int rem = (1024 * (w + NW * it) + 16 * lane) % L::TILE, tok = rem / (D * ES);
    goff[it] = (tok < K) ? rem : -1;
  }
  auto fetch = [&](int stage) {
    if (stage >= a.n_stages) return;
    unsigned char* dst = smem + L::IN + (stage % 3) * L::IN1;
    const size_t tok0 = (bh * (size_t)a.seq_stride + (size_t)stage * K) * D * ES;
#pragma unroll
    for (int it = 0; it < NBI; ++it) {
      const int b = w + NW * it;  // wave-uniform
      if (b < NBLK) {
        const int ten = (1024 * b) / L::TILE;
        const unsigned char* src =
            static_cast<const unsigned char*>(ten == 0 ? a.xq : ten == 1 ? a.xk : a.xv) + tok0;
        if (goff[it] >= 0)
          lds_dma16(src, (unsigned)goff[it], (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)(dst + 1024 * b));
      }
    }
    // lr as zero-extended bf16 words, copied like the tiles (a register load here would make the compiler
    // wait for every copy in flight); absent tokens read a clamped position and are zeroed at use
    if (tid < 16)
      lds_dma2(static_cast<const elem*>(a.lr) + bh * (size_t)a.seq_stride + (size_t)stage * K, 2u * (unsigned)(tid < K ? tid : K - 1),
               (unsigned)(size_t)(__attribute__((address_space(3))) uint32_t*)(LRs + (stage % 3) * 16));
  };
  // staged row of token c of tensor ten (0 xq, 1 xk, 2 xv)
  auto row = [&](int buf, int ten) -> const elem* {
    return reinterpret_cast<const elem*>(smem + L::IN + buf * L::IN1 + ten * L::TILE) + c * D;
  };

  for (int i = tid; i < (L::P1 - L::IN) / 4; i += 512) reinterpret_cast<float*>(smem)[i] = 0.f;
  for (int i = tid; i < 8 * 2 * 16 * 4; i += 512) EX[i] = 0.f;
  if (tid < 2 * 2 * 16 * 4) EXO[tid] = 0.f;
  __syncthreads();
  fetch(0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  // pending output of the previous mini-batch (reducers)

  // ---- reducers: lane group g publishes sums g and g + 4 (six in all) of reducer w
  auto publish = [&](const float (&S)[6]) {
    const float v0 = xg_sum4_scatter(S[0], S[1], S[2], S[3]);
    const float v1 = xg_sum4_scatter(S[4], S[5], 0.f, 0.f);
    EX[(((g)*2 + (w >> 2)) * 16 + c) * 4 + (w & 3)] = v0;
    if (g < 2) EX[(((g + 4) * 2 + (w >> 2)) * 16 + c) * 4 + (w & 3)] = v1;
  };
  auto collect = [&](int i) -> float {
    const f32x4 lo = *reinterpret_cast<const f32x4*>(EX + ((i * 2 + 0) * 16 + c) * 4);
    float s = (lo[0] + lo[1]) + (lo[2] + lo[3]);
    if (NT > 4) {
      const f32x4 hi = *reinterpret_cast<const f32x4*>(EX + ((i * 2 + 1) * 16 + c) * 4);
      s += (hi[0] + hi[1]) + (hi[2] + hi[3]);
    }
    return s;
  };

  // ---- output path: finishing the OUTPUT of the previous mini-batch is spread over the waves with
  // the most slack: d-feature tile I goes to wave (NT + I) % NW, i.e. first to the waves that reduce
  // no Z2 tile, then to reducers 0, 1, ...  Each wave has at most one output tile.
  const int otile = (w - NT + NW) % NW;  // this wave's output tile
  const bool outw = otile < NT;
  const int ooff = own_offset<1>(outw ? otile : 0, 0, g);
  f32x4 zb = {0.f, 0.f, 0.f, 0.f};
  // part 1 (before B2): Zbar2^T tile from the split-k partials, causal correction, row moments
  auto output_reduce = [&]() {
    f32x4 at = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ww = 0; ww < NW; ++ww) at += PA[ww * 64 + lane];
    pin(at);
    f32x4 m;
#pragma unroll
    for (int r = 0; r < 4; ++r) m[r] = (4 * g + r <= c) ? rho_c * (1.f + at[r]) : 0.f;
    zb = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ww = 0; ww < NW; ++ww) zb += P2[(ww * NT + otile) * 64 + lane];
    pin(zb);
    IO::mma(zb, GD[otile * 64 + lane], IO::to_frag(m));  // GD still holds the previous mini-batch's G2
    float s0 = 0.f, s1 = 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      s0 += zb[r];
      s1 += zb[r] * zb[r];
    }
    s0 = xg_sum(s0);
    s1 = xg_sum(s1);
    if (g == 0) {
      EXO[((0 * 2 + (otile >> 2)) * 16 + c) * 4 + (otile & 3)] = s0;
      EXO[((1 * 2 + (otile >> 2)) * 16 + c) * 4 + (otile & 3)] = s1;
    }
  };
  auto collect_o = [&](int i) -> float {
    const f32x4 lo = *reinterpret_cast<const f32x4*>(EXO + ((i * 2 + 0) * 16 + c) * 4);
    float s = (lo[0] + lo[1]) + (lo[2] + lo[3]);
    if (NT > 4) {
      const f32x4 hi = *reinterpret_cast<const f32x4*>(EXO + ((i * 2 + 1) * 16 + c) * 4);
      s += (hi[0] + hi[1]) + (hi[2] + hi[3]);
    }
    return s;
  };
  // part 2 (after B2): out = xq + gamma (zbar - mu) rstd + beta
  auto output_emit = [&](int stage) {
    const float mu = collect_o(0) * inv_d;
    const float rstd = __builtin_amdgcn_rsqf(fmaxf(collect_o(1) * inv_d - mu * mu, 0.f) + a.eps);
    if (c < K) {
      const f32x4 gam = *reinterpret_cast<const f32x4*>(GAM + ooff), bet = *reinterpret_cast<const f32x4*>(BET + ooff);
      const frag qo = load4<T>(row(stage % 3, 0) + ooff);
      elem* po = static_cast<elem*>(a.out) + (bh * (size_t)a.seq_stride + (size_t)stage * K + c) * D + ooff;
      store4<T>(po, IO::to_f32(qo) + bet + gam * ((zb - mu) * rstd));
    }
  };

  for (int st = 0; st < a.n_stages; ++st) {
    const int buf = st % 3, par = st & 1;
    RELANE();
    fetch(st + 1);

    // ================= phase A: everything that needs only W1, W2 and the inputs
    f32x4 z1[HT];
    // XK tile w with tokens along k, for everybody's W1 update
    if (red) {
      f32x4 t = {0.f, 0.f, 0.f, 0.f};
      IO::mma(t, load4<T>(row(buf, 1) + own), ident);
      KD[(par * NT + w) * 64 + lane] = IO::to_frag(t);
    }
    // Z1^T for this wave's hidden units
#pragma unroll
    for (int j = 0; j < HT; ++j) z1[j] = *reinterpret_cast<const f32x4*>(B1s + 16 * (w * HT + j) + 4 * g);
#pragma unroll
    for (int q = 0; q < NT / 2; ++q) {
      frag k0, k1;
      IO::load8(row(buf, 1) + 32 * q + 8 * g, true, k0, k1);
#pragma unroll
      for (int j = 0; j < HT; ++j)
        IO::mma2(z1[j], IO::to_frag(W1c[2 * q][j]), IO::to_frag(W1c[2 * q + 1][j]), k0, k1);
      __builtin_amdgcn_sched_barrier(0);
    }
    const float lrc = (c < K) ? __uint_as_float(LRs[buf * 16 + c] << 16) : 0.f;
    // X2 = gelu(Z1), gelu'(Z1)
    frag x2f[HT];
    f32x4 dg[HT];
#pragma unroll
    for (int j = 0; j < HT; ++j) {
      f32x4 y, dy;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float yy, dd;
        gelu_fast_pair(z1[j][r], yy, dd);
        y[r] = yy;
        dy[r] = dd;
      }
      x2f[j] = IO::to_frag(y);
      dg[j] = dy;
      // materialise both now: left to itself the compiler postpones gelu' to its use after the
      // barriers and keeps (or spills) twice as many intermediates until then
      asm volatile("" : "+v"(x2f[j]), "+v"(dg[j]));
      __builtin_amdgcn_sched_barrier(0);
    }
    // partial Z2^T over this wave's hidden units
#pragma unroll
    for (int I = 0; I < NT; ++I) {
      f32x4 p = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j + 1 < HT; j += 2)
        IO::mma2(p, IO::to_frag(W2c[j][I]), IO::to_frag(W2c[j + 1][I]), x2f[j], x2f[j + 1]);
      if (HT & 1) IO::mma2(p, IO::to_frag(W2c[HT - 1][I]), IO::zero(), x2f[HT - 1], IO::zero());
      P1[(w * NT + I) * 64 + lane] = p;
      __builtin_amdgcn_sched_barrier(0);
    }
    lds_barrier();  // ---- B1
    RELANE();

    // ================= phase B: reducers: full Z2 tile and its row moments;
    //                          output waves: Zbar2 tiles of the previous mini-batch and their moments
    f32x4 z = {0.f, 0.f, 0.f, 0.f}, bq = z;
    if (red) {
      z = b2T;
#pragma unroll
      for (int ww = 0; ww < NW; ++ww) {
        z += P1[(ww * NT + w) * 64 + lane];
        if ((ww & 3) == 3) pin(z);
      }
      const frag ko = load4<T>(row(buf, 1) + own), vo = load4<T>(row(buf, 2) + own);
      const f32x4 gam = *reinterpret_cast<const f32x4*>(GAM + own), bet = *reinterpret_cast<const f32x4*>(BET + own);
      bq = gam * (bet - (IO::to_f32(vo) - IO::to_f32(ko)));
      float S[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      const f32x4 az = gam * gam * z;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        S[0] += z[r];
        S[1] += z[r] * z[r];
        S[2] += az[r];
        S[3] += az[r] * z[r];
        S[4] += bq[r];
        S[5] += bq[r] * z[r];
      }
      publish(S);
    }
    if (outw && st > 0) output_reduce();
    lds_barrier();  // ---- B2
    RELANE();

    // ================= phase C: reducers: G2'' in both orientations; output waves: store the output
    frag g2_saved = IO::zero();
    if (red) {
      float S[6];
#pragma unroll
      for (int i = 0; i < 6; ++i) {
        S[i] = collect(i);
      }
      const float mu = S[0] * inv_d;
      const float var = S[1] * inv_d - mu * mu;
      const float rstd = __builtin_amdgcn_rsqf(fmaxf(var, 0.f) + a.eps);
      const float s1 = rstd * (S[2] - mu * sum_a) + S[4];
      const float s2 = rstd * rstd * (S[3] - 2.f * mu * S[2] + mu * mu * sum_a) + rstd * (S[5] - mu * S[4]);
      const float p = -sc * lrc * rstd;
      const float c1 = p * rstd, c2 = -c1 * s2 * inv_d, c3 = -p * s1 * inv_d;
      const f32x4 gam = *reinterpret_cast<const f32x4*>(GAM + own);
      const f32x4 G = (z - mu) * (gam * gam * c1 + c2) + (bq * p + c3);
      const frag gt = IO::to_frag(G);
      f32x4 t = {0.f, 0.f, 0.f, 0.f};
      IO::mma(t, gt, ident);
      GT[w * 64 + lane] = gt;
      GD[w * 64 + lane] = IO::to_frag(t);
      g2_saved = gt;
    }
    if (outw && st > 0) output_emit(st - 1);
    // the next mini-batch's rows must have landed before anybody passes B3; the output store just issued
    // (the only memory operation younger than the copies, which retire in order) may stay in flight
    if (outw && st > 0)
      asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
    else
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    lds_barrier();  // ---- B3
    RELANE();

    // ================= phase D: G1, Zbar1, Xbar2, split-k partials of the output path, updates
    // The factors of this mini-batch's state update for ttt_mlp_bwd, eta_last * G1 [16 x 4d] and eta_last * G2
    // [16 x d] (row = token), exactly as the update applies them: rounded to the operand type, sign undone
    // (G'' = -eta_last * lr * G); zeros when token_eta[K-1] = 0 switches the update off.  Stored behind B3 so
    // that the counted waits of phase C see the same memory operations as without them.
    const size_t save_row = (bh * (size_t)a.n_stages + st) * 16 + c;
    if (a.G2_save != nullptr && red) {
      const f32x4 v = upd ? -IO::to_f32(g2_saved) : f32x4{0.f, 0.f, 0.f, 0.f};
      *reinterpret_cast<f32x4*>(a.G2_save + save_row * D + own) = v;
    }
#pragma unroll
    for (int j = 0; j < HT; ++j)
#pragma unroll
      for (int I = 0; I < NT; ++I) forget(W2c[j][I]);
    frag G1d[HT];
#pragma unroll
    for (int j = 0; j < HT; ++j) {
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int q = 0; q < NT / 2; ++q) {
        f32x4 t0 = {0.f, 0.f, 0.f, 0.f}, t1 = {0.f, 0.f, 0.f, 0.f};
        IO::mma(t0, IO::to_frag(W2c[j][2 * q]), ident);
        IO::mma(t1, IO::to_frag(W2c[j][2 * q + 1]), ident);
        IO::mma2(acc, IO::to_frag(t0), IO::to_frag(t1), GT[(2 * q) * 64 + lane], GT[(2 * q + 1) * 64 + lane]);
      }
      f32x4 t = {0.f, 0.f, 0.f, 0.f};
      const frag g1b = IO::to_frag(acc * dg[j]);
      IO::mma(t, g1b, ident);
      G1d[j] = IO::to_frag(t);
      if (a.G1_save != nullptr) {
        const f32x4 v = upd ? -IO::to_f32(g1b) : f32x4{0.f, 0.f, 0.f, 0.f};
        *reinterpret_cast<f32x4*>(a.G1_save + save_row * F + 16 * (w * HT + j) + 4 * g) = v;
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // Zbar1^T = (XQ W1 + b1)^T + G1''^T M1, with M1[s][t] = (token_eta[t] / sc)(1 + A1[t][s]) for s <= t.
    // Computed here rather than next to Z1 so that it does not occupy registers across the barriers.
#pragma unroll
    for (int j = 0; j < HT; ++j)
#pragma unroll
      for (int I = 0; I < NT; ++I) forget(W1c[I][j]);
    f32x4 zq[HT], At = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < HT; ++j) zq[j] = *reinterpret_cast<const f32x4*>(B1s + 16 * (w * HT + j) + 4 * g);
#pragma unroll
    for (int q = 0; q < NT / 2; ++q) {
      frag k0, k1, q0, q1;
      IO::load8(row(buf, 1) + 32 * q + 8 * g, true, k0, k1);
      IO::load8(row(buf, 0) + 32 * q + 8 * g, true, q0, q1);
#pragma unroll
      for (int j = 0; j < HT; ++j)
        IO::mma2(zq[j], IO::to_frag(W1c[2 * q][j]), IO::to_frag(W1c[2 * q + 1][j]), q0, q1);
      IO::mma2(At, k0, k1, q0, q1);
      __builtin_amdgcn_sched_barrier(0);
    }
    {
      f32x4 m;
#pragma unroll
      for (int r = 0; r < 4; ++r) m[r] = (4 * g + r <= c) ? rho_c * (1.f + At[r]) : 0.f;
      const frag Mf = IO::to_frag(m);
#pragma unroll
      for (int j = 0; j < HT; ++j) IO::mma(zq[j], G1d[j], Mf);
    }
    frag xbf[HT];
#pragma unroll
    for (int j = 0; j < HT; ++j) {
      f32x4 y;
#pragma unroll
      for (int r = 0; r < 4; ++r) y[r] = gelu_fast(zq[j][r]);
      xbf[j] = IO::to_frag(y);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int j = 0; j < HT; ++j)
#pragma unroll
      for (int I = 0; I < NT; ++I) forget(W2c[j][I]);
    {
      f32x4 p = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j + 1 < HT; j += 2) IO::mma2(p, x2f[j], x2f[j + 1], xbf[j], xbf[j + 1]);
      if (HT & 1) IO::mma2(p, x2f[HT - 1], IO::zero(), xbf[HT - 1], IO::zero());
      PA[w * 64 + lane] = p;
    }
#pragma unroll
    for (int I = 0; I < NT; ++I) {
      f32x4 p = (I == w) ? b2T : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j + 1 < HT; j += 2)
        IO::mma2(p, IO::to_frag(W2c[j][I]), IO::to_frag(W2c[j + 1][I]), xbf[j], xbf[j + 1]);
      if (HT & 1) IO::mma2(p, IO::to_frag(W2c[HT - 1][I]), IO::zero(), xbf[HT - 1], IO::zero());
      P2[(w * NT + I) * 64 + lane] = p;
      __builtin_amdgcn_sched_barrier(0);
    }
    if (upd) {
      frag x2d[HT];
#pragma unroll
      for (int j = 0; j < HT; ++j) {
        f32x4 t = {0.f, 0.f, 0.f, 0.f};
        IO::mma(t, x2f[j], ident);
        x2d[j] = IO::to_frag(t);
        f32x4 b = *reinterpret_cast<const f32x4*>(B1s + 16 * (w * HT + j) + 4 * g);
        IO::mma(b, G1d[j], ones);
        if (c == 0) *reinterpret_cast<f32x4*>(B1s + 16 * (w * HT + j) + 4 * g) = b;
      }
#pragma unroll
      for (int I = 0; I < NT; ++I) {
        const frag kd = KD[(par * NT + I) * 64 + lane], g2d = GD[I * 64 + lane];
#pragma unroll
        for (int j = 0; j < HT; ++j) {
          IO::mma(W1c[I][j], kd, G1d[j]);
          IO::mma(W2c[j][I], x2d[j], g2d);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if (red) IO::mma(b2T, GD[w * 64 + lane], ones);
    }
  }

  // ---- the last mini-batch's output
  lds_barrier();
  if (outw) output_reduce();
  lds_barrier();
  if (outw) output_emit(a.n_stages - 1);

  // ---- final state.  Second layer: initial value + (centred value now - centred value at the start), the start
  // value formed again exactly as above, so a sequence that never updates the state returns it bit for bit.
  {
    float* W1 = a.W1 + bh * (size_t)D * F;
    float* W2 = a.W2 + bh * (size_t)D * F;
    const float* W2i = a.W2_0 + sb * (size_t)D * F;
#pragma unroll
    for (int j = 0; j < HT; ++j) {
      const int hb = 16 * (w * HT + j);
      f32x4 w0[NT];
#pragma unroll
      for (int I = 0; I < NT; ++I)
#pragma unroll
        for (int r = 0; r < 4; ++r) w0[I][r] = W2i[(size_t)(hb + 4 * g + r) * D + feat(I, c)];
      const f32x4 m = row_means16<NT>(w0, inv_d);
#pragma unroll
      for (int I = 0; I < NT; ++I) {
        const f32x4 start = w0[I] - m;
        const f32x4 fin = w0[I] + (W2c[j][I] - start);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          W1[(size_t)feat(I, 4 * g + r) * F + hb + c] = W1c[I][j][r];
          W2[(size_t)(hb + 4 * g + r) * D + feat(I, c)] = fin[r];
        }
      }
      if (c == 0) store4<F32>(a.b1 + bh * F + hb + 4 * g, *reinterpret_cast<const f32x4*>(B1s + hb + 4 * g));
    }
    if (red) {
      const float bb = mean_of(a.b2_0 + sb * D, D, inv_d);
      const f32x4 v0 = *reinterpret_cast<const f32x4*>(a.b2_0 + sb * D + own);
      const f32x4 start = v0 - bb;
      if (c == 0) store4<F32>(a.b2 + bh * D + own, v0 + (b2T - start));
    }
  }
}

#undef RELANE

}  // namespace ttt
