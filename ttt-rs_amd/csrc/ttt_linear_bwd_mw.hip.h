// TTT-Linear fused backward for gfx950, checkpoint interval 1, NW wavefronts per (batch, head): the
// register-resident scheme of ttt_linear_bwd_rr.hip.h with the feature axis cut into NW slices.
//
// Arithmetic: the reverse scan of ttt_linear_bwd.hip.h (reference
// rust/fused/src/linear_fused_tile/backward/kernel.rs:253-429, backward/stage.rs:42-1006, second-order
// LayerNorm layer_norm.rs:428-709).
//
// Wave w owns TPW = (d/16)/NW feature tiles.  Of every [16 x d] tile it holds its own features (transposed:
// value r of lane (c, g) is feature feat(J, 4g+r) of token c); of the state gradient it holds the column
// slice dW[:, own] (dWc) and the row slice dW[own, :] transposed (DT), each fed back as an A operand without
// data movement.  What a wave needs of the other slices crosses through LDS at four points per mini-batch:
//   X1  six raw moments of Z1 (mean, variance and both sums of the LN-L2 gradient follow from them), the
//       partial attention blocks, XK^T / XQ^T fragments (tokens along k);
//   X2  four raw moments of Zbar and of the output-LayerNorm backward; G fragments;
//   X3  partial P = dZbar G^T, dZbar fragments in both forms, and the six sums of the second-order LayerNorm
//       (all its statistics are linear in them; none needs P, so one exchange carries both);
//   X4  dZ1 fragments in both forms.
// All matrix products with a d-deep contraction over the OTHER slices' features take those fragments as B
// operands; products over tokens (rank-16) are local.  f32 I/O computes in true-f32 MFMA
// (v_mfma_f32_16x16x4_f32), bf16 I/O in bf16 MFMA with f32 accumulation.
// Staging: checkpoint, bias, lr and the four activation tiles of a mini-batch are copied global -> LDS
// (one buffer: everything is moved to registers at the top of the mini-batch, the copies for the next one
// are issued behind the first exchange).
#pragma once
#include "ttt_linear_bwd.hip.h"
#include "ttt_linear_fwd_mw.hip.h"

namespace ttt {

// PK: the W checkpoint arrives packed (bf16 fragments in accumulator order, see store_ckpt_packed)
// FM: no states were saved but the update factors and the final state (see store_factor): the f32 state lives in
//     the registers of the waves (each its column tiles, as in the forward), is walked back by one mini-batch per
//     pass, and its packed image is written where a packed checkpoint would have been copied to
template <int D, int NW, int ES, bool PK = false, bool FM = false>
struct LinBwdMwLds {
  static constexpr int NT = D / 16, TPW = NT / NW;
  static constexpr int XS = (ES == 2) ? NT / 2 : NT;  // 1 KiB slots per activation tensor
  static constexpr int FT = 64 * 4 * ES;              // bytes of one fragment tile
  static constexpr int W = 0;                         // NT*NT slots: slot I*NT+J, lane (c,g): W[feat(I,c)][feat(J,4g..4g+3)]
                                                      // packed: NT*NT/2 slots: slot I*NT/2+q = tiles (I,2q), (I,2q+1)
  static constexpr int WSLOTS = (PK && ES == 2) ? NT * NT / 2 : NT * NT;
  static constexpr int Bv = W + WSLOTS * 1024;        // NT slots: b[feat(J,4g..4g+3)]
  static constexpr int X = Bv + NT * 1024;            // 4 tensors x XS slots
  static constexpr int LR = X + 4 * XS * 1024;        // 16 dwords: lr of token c (bf16 zero-extended, or f32)
  static constexpr int SUM = LR + 256;                // 3 exchanges x [8 sums][16 tokens][NW]
  static constexpr int PT = SUM + 3 * 8 * 16 * NW * 4;  // 4 kinds x [NW][64] f32x4: partial [16 x 16] blocks
  static constexpr int FR = PT + 4 * NW * 1024;       // 9 kinds x [NT][64] fragments
  static constexpr int M0 = FR + 9 * NT * FT;         // D row means of the initial W, then mean(b): the centred state
  static constexpr int GDS = M0 + (D + 4) * 4;         // FM: NT half slots: the factor fragments of tile J
  static constexpr int BYTES = GDS + (FM ? NT * 512 : 0);
  static_assert(!FM || (PK && ES == 2), "factors: bf16 I/O, packed image of the state");
  static_assert(GDS % 16 == 0, "copy targets are 16-byte aligned");
  static_assert(NT % NW == 0 && WSLOTS % NW == 0, "feature tiles must divide among the waves");
  static_assert(BYTES <= 160 * 1024, "exceeds the 160 KiB of LDS of a gfx950 CU");
};

// FULL: mini_batch == 16, every lane's token exists: the stores and copies of a mini-batch need no lane mask (and no
// branch around them, which would also end the block the scheduler can reorder within)
// Up to d = 64 with one feature tile per wave the kernel is held to 256 registers: two workgroups then share a compute
// unit (two waves per SIMD), which is what 257 registers would silently halve (f32 I/O with f32 row-major checkpoints
// excepted: it needs 265 and would spill).
template <class T, int D, int NW, bool PK = false, bool FM = false, bool FULL = false>
__global__ void __launch_bounds__(64 * NW, (D <= 64 && D / 16 == NW && (PK || sizeof(typename Io<T>::elem) == 2)) ? 2 : 1)
    ttt_linear_bwd_mw_kernel(LinearBwdArgs a) {
  using IO = Io<T>;
  using frag = typename IO::frag;
  using elem = typename IO::elem;
  constexpr int ES = sizeof(elem);
  constexpr bool BF = ES == 2;
  using L = LinBwdMwLds<D, NW, ES, PK, FM>;
  constexpr int NT = D / 16, TPW = NT / NW, NQ = NT / 2, XS = L::XS;
  constexpr float inv_d = 1.0f / D;
  enum { KD = 0, QD, GF, ZF, ZD, Z1F, Z1D, GL, ZL };
  enum { P_AT = 0, P_AT2, P_P, P_P2 };
  // bf16, d <= 96: the [16 x 16] blocks that contract over all d features (attention, P = dZbar G^T) are formed
  // whole by every wave on the matrix pipe, from fragments that cross LDS anyway, instead of per-wave partial
  // blocks that are written, read NW times and added up on the VALU
  constexpr bool FULL_AT = BF && D <= 96;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int lane = threadIdx.x & 63, c = lane & 15, g = lane >> 4;
  const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const size_t bh = blockIdx.x;
  const int h = (int)(bh % a.H);
  const int K = a.K;

  float* const SUMp = reinterpret_cast<float*>(smem + L::SUM);
  f32x4* const PTp = reinterpret_cast<f32x4*>(smem + L::PT);
  frag* const FRp = reinterpret_cast<frag*>(smem + L::FR);
  auto fr = [&](int kind, int J) -> frag& { return FRp[(kind * NT + J) * 64 + lane]; };
  auto pt = [&](int kind, int ww) -> f32x4& { return PTp[(kind * NW + ww) * 64 + lane]; };

  const float te_c = (c < K) ? a.token_eta[c] : 0.f;
  const float te_last = a.token_eta[K - 1];
  f32x4 te_s;
#pragma unroll
  for (int r = 0; r < 4; ++r) te_s[r] = (4 * g + r < K) ? a.token_eta[4 * g + r] : 0.f;
  const frag ident = identity_frag<T>(c, g);
  const frag ones = splat_frag<T>(1.f);
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  f32x4 gam[TPW], bet[TPW], a2[TPW], dgam[TPW], dbet[TPW], dbT[TPW];
  float sum_a = 0.f;
  for (int f = 0; f < D; ++f) sum_a += a.gamma[h * D + f] * a.gamma[h * D + f];
#pragma unroll
  for (int jj = 0; jj < TPW; ++jj) {
    const int f = own_offset<TPW>(w, jj, g);
    gam[jj] = *reinterpret_cast<const f32x4*>(a.gamma + h * D + f);
    bet[jj] = *reinterpret_cast<const f32x4*>(a.beta + h * D + f);
    a2[jj] = gam[jj] * gam[jj];
    dgam[jj] = dbet[jj] = zero4;
    dbT[jj] = a.d_b_out ? *reinterpret_cast<const f32x4*>(a.d_b_out + bh * D + f) : zero4;
  }
  // dWc[I][jj]: rows i = feat(I, 4g+r), columns j = feat(own jj, c)
  // DT[J][ii]:  rows j = feat(J, 4g+r), columns i = feat(own ii, c)   (= dW[own rows][all columns], transposed)
  f32x4 dWc[NT][TPW], DT[NT][TPW];
#pragma unroll
  for (int I = 0; I < NT; ++I)
#pragma unroll
    for (int jj = 0; jj < TPW; ++jj) {
      const int Jo = w * TPW + jj;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        dWc[I][jj][r] = a.d_W_out ? a.d_W_out[bh * D * D + feat(I, 4 * g + r) * D + feat(Jo, c)] : 0.f;
        DT[I][jj][r] = a.d_W_out ? a.d_W_out[bh * D * D + feat(Jo, c) * D + feat(I, 4 * g + r)] : 0.f;
      }
    }

  // rows of absent tokens (c >= K) are never fetched: they stay zero
  for (int i = threadIdx.x; i < L::BYTES / 16; i += 64 * NW) reinterpret_cast<u32x4*>(smem)[i] = u32x4{0u, 0u, 0u, 0u};
  __syncthreads();

  // ---- the scan works on the centred state Wc = W - m 1^T, bc = b - mean(b), as the forward does (centre_state in
  // ttt_linear_fwd_mw.hip.h): every product with W either feeds a LayerNorm (Z1, Zbar: a common shift of a row is
  // discarded) or multiplies a LayerNorm gradient from the right (dZbar W^T, dZ1 W^T: the rows of dZbar and dZ1 sum
  // to zero, so the m 1^T part contributes nothing).  m and mean(b) are those of the initial state (checkpoint 0):
  // the forward's updates do not move them.  A packed checkpoint holds the centred matrix already.
  float* const M0p = reinterpret_cast<float*>(smem + L::M0);
  {
    const size_t c0 = bh * (size_t)a.n_ckpt;
    if (!PK) {
      for (int i = threadIdx.x; i < D; i += 64 * NW) {
        const f32x4* row = reinterpret_cast<const f32x4*>(a.W_ckpt + c0 * D * D + (size_t)i * D);
        float sum = 0.f;
        for (int j = 0; j < D / 4; ++j) {
          const f32x4 v = row[j];
          sum += (v[0] + v[1]) + (v[2] + v[3]);
        }
        M0p[i] = sum * inv_d;
      }
    }
    if (!FM && threadIdx.x == 0) {
      float sum = 0.f;
      for (int f = 0; f < D; ++f) sum += a.b_ckpt[c0 * D + f];
      M0p[D] = sum * inv_d;
    }
    __syncthreads();
  }
  float mrow[NT];  // m of row feat(I, c)
#pragma unroll
  for (int I = 0; I < NT; ++I) mrow[I] = PK ? 0.f : M0p[feat(I, c)];
  float mrowo[TPW];  // the same for the wave's own row tiles
#pragma unroll
  for (int ii = 0; ii < TPW; ++ii) mrowo[ii] = PK ? 0.f : M0p[feat(w * TPW + ii, c)];
  const float bbar = M0p[D];

  // ---- copies of one mini-batch, dealt round-robin to the waves
  const unsigned stg = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)smem;
  // FM: the unit's share of the W checkpoint buffer holds the final state and, behind it, one factor per mini-batch
  const unsigned char* const fac0 =
      reinterpret_cast<const unsigned char*>(a.W_ckpt + bh * (size_t)a.n_ckpt * (D * D)) + D * D * 4;
  auto fetch = [&](int stage) {
    if (stage < 0) return;
    if constexpr (FM) {
      // the factor of the mini-batch: tile J is 512 bytes, copied by half a wave
      const unsigned char* fp = fac0 + (size_t)stage * (32 * D);
#pragma unroll
      for (int it = 0; it < TPW; ++it) {
        const int J = w + NW * it;
        if (lane < 32) lds_dma16(fp, (unsigned)(J * 512 + lane * 16), stg + L::GDS + J * 512);
      }
    } else {
      const size_t ci = bh * (size_t)a.n_ckpt + stage;
      const float* Wg = a.W_ckpt + ci * D * D;
#pragma unroll
      for (int it = 0; it < L::WSLOTS / NW; ++it) {
        const int n = w + NW * it, I = n / NT, J = n - I * NT;
        if (PK)  // whole 1 KiB rows
          lds_dma16(Wg, (unsigned)(n * 1024 + lane * 16), stg + L::W + n * 1024);
        else
          lds_dma16(Wg, (unsigned)(feat(I, c) * D + 32 * (J >> 1) + 8 * g + 4 * (J & 1)) * 4u, stg + L::W + n * 1024);
      }
      if (w == 1 % NW) {
        const float* bg = a.b_ckpt + ci * D;
#pragma unroll
        for (int J = 0; J < NT; ++J) lds_dma16(bg, (unsigned)(32 * (J >> 1) + 8 * g + 4 * (J & 1)) * 4u, stg + L::Bv + J * 1024);
      }
    }
    const size_t tok0 = (bh * (size_t)a.seq_stride + (size_t)stage * K) * D;
#pragma unroll
    for (int ten = 0; ten < 4; ++ten) {
      if (ten % NW != w) continue;
      const elem* src = static_cast<const elem*>(ten == 0 ? a.xq : ten == 1 ? a.xk : ten == 2 ? a.xv : a.d_out) + tok0;
      if (FULL || c < K) {
#pragma unroll
        for (int s = 0; s < XS; ++s) {
          // bf16: 8 features of tiles 2s, 2s+1; f32: the 4 features of tile s
          const unsigned off = BF ? (unsigned)(c * D + 32 * s + 8 * g) * 2u
                                  : (unsigned)(c * D + 32 * (s >> 1) + 8 * g + 4 * (s & 1)) * 4u;
          lds_dma16(src, off, stg + L::X + (ten * XS + s) * 1024);
        }
      }
    }
    if (w == NW - 1 && lane < 16) {
      const elem* lrp = static_cast<const elem*>(a.lr) + bh * (size_t)a.seq_stride + (size_t)stage * K;
      const unsigned li = (unsigned)(c < K ? c : K - 1);
      if (BF)
        lds_dma2(lrp, 2u * li, stg + L::LR);
      else
        lds_dma4(lrp, 4u * li, stg + L::LR);
    }
  };
  // partial sums of this wave's features -> totals in every wave, in two steps: publish, then (behind the
  // exchange barrier) collect.  Issue is in order, so work that does not depend on the exchange is placed
  // between the two: it runs while the LDS write, the barrier and the LDS reads are in flight.
  auto xpub = [&](int region, const float (&S)[8]) {
    const float v0 = xg_sum4_scatter(S[0], S[1], S[2], S[3]);
    const float v1 = xg_sum4_scatter(S[4], S[5], S[6], S[7]);
    float* e = SUMp + region * 8 * 16 * NW;
    e[(g * 16 + c) * NW + w] = v0;
    e[((g + 4) * 16 + c) * NW + w] = v1;
  };
  auto xcol = [&](int region, float (&S)[8]) {
    const float* e = SUMp + region * 8 * 16 * NW;
    lds_barrier();
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float s = 0.f;
#pragma unroll
      for (int ww = 0; ww < NW; ++ww) s += e[(i * 16 + c) * NW + ww];
      S[i] = s;
    }
  };
  auto ptsum = [&](int kind) {
    f32x4 s = pt(kind, 0);
#pragma unroll
    for (int ww = 1; ww < NW; ++ww) s += pt(kind, ww);
    return s;
  };
  // byte offset (without the lane's 16) of tile (I, J) of a packed checkpoint in the staging area
  auto pk_off = [&](int I, int J) { return BF ? L::W + (I * NQ + (J >> 1)) * 1024 + 8 * (J & 1) : L::W + (I * NT + J) * 1024; };
  auto tokens_k = [&](frag x) {
    f32x4 t = {0.f, 0.f, 0.f, 0.f};
    IO::mma(t, x, ident);
    return IO::to_frag(t);
  };
  // acc += sum over the NT tiles of A[J] B[J]
  auto mma_all = [&](f32x4& acc, const frag (&A)[NT], const frag (&B)[NT]) {
#pragma unroll
    for (int qq = 0; qq < NQ; ++qq) IO::mma2(acc, A[2 * qq], A[2 * qq + 1], B[2 * qq], B[2 * qq + 1]);
  };
  // acc += sum over this wave's tiles
  auto mma_own = [&](f32x4& acc, const frag (&A)[TPW], const frag (&B)[TPW]) {
    if (TPW % 2 == 0) {
#pragma unroll
      for (int qq = 0; qq < TPW / 2; ++qq) IO::mma2(acc, A[2 * qq], A[2 * qq + 1], B[2 * qq], B[2 * qq + 1]);
    } else {
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) IO::mma(acc, A[jj], B[jj]);
    }
  };
  // The counted waits of the scan.  Memory operations of a wave retire in the order they were issued, stores
  // included, so "s_waitcnt vmcnt(n)" with n = the number of operations a wave is KNOWN to have issued behind its
  // global->LDS copies waits for the copies and not for those younger operations.  Counted are the row stores of the
  // three activation gradients, one store_own per tensor, wave and pass, issued by every wave on every path: the
  // guard in front of each is a lane mask (c < K), never a wave-uniform branch, so a mini-batch shorter than 16 tokens
  // still issues it, and store_own is at least one instruction for TPW <= 2 (an f32 store of two tiles is two: more
  // operations than counted only make the wait longer).  Operations that only some waves issue (d_lr by the first
  // wave, the d_token_eta atomics by the last) are not counted.  Fewer operations than counted would let the loop
  // read staged rows before they have landed, so whoever moves a store_own across one of the two waits, or makes one
  // conditional at wave level, changes these numbers with it.
  //   loop top: d_xq, d_xv and d_xk of the pass before lie behind the copies (issued before the first of them)
  //   X4 barrier (FM only; the walk back reads the staged rows): d_xq and d_xv lie behind the copies
  static_assert(TPW <= 2, "store_own must stay one store instruction (bf16) per tensor and wave");
  constexpr int kStoresBehindCopiesAtLoopTop = 3;
  constexpr int kStoresBehindCopiesAtX4 = 2;
  auto store_own = [&](void* base, size_t tokoff, const f32x4 (&x)[TPW]) {
    elem* p = static_cast<elem*>(base) + tokoff;
    if (TPW == 1) {
      store4<T>(p + own_offset<TPW>(w, 0, g), x[0]);
    } else {
#pragma unroll
      for (int qq = 0; qq < TPW / 2; ++qq) IO::store8(p + own_offset<TPW>(w, 2 * qq, g), x[2 * qq], x[2 * qq + 1]);
    }
  };

  // FM: the state after the last mini-batch (centred, as the forward carried it) is where the walk back starts
  f32x4 bTm[TPW], Wm[FM ? NT : 1][TPW];  // bias of the own features; W[all row tiles][own column tiles]
  const bool upd = te_last != 0.f;  // the forward leaves the state alone when token_eta[K-1] is zero
  if constexpr (FM) {
    const unsigned char* Wl = reinterpret_cast<const unsigned char*>(a.W_ckpt + bh * (size_t)a.n_ckpt * (D * D));
    const float* bl = a.b_ckpt + bh * (size_t)a.n_ckpt * D;
#pragma unroll
    for (int I = 0; I < NT; ++I)
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj)
        Wm[I][jj] = *reinterpret_cast<const f32x4*>(Wl + (I * NT + w * TPW + jj) * 1024 + lane * 16);
#pragma unroll
    for (int ii = 0; ii < TPW; ++ii) bTm[ii] = *reinterpret_cast<const f32x4*>(bl + own_offset<TPW>(w, ii, g));
  }
  fetch(a.n_stages - 1);

  // FM: the state entering the mini-batch whose copies are staged: W_t = W_{t+1} - XK_t^T G''_t and
  // b_t = b_{t+1} - colsum G''_t, with the operands the forward multiplied (XK as staged, G'' as saved).  This wave's
  // column tiles of the f32 state are updated in its registers and their packed image is written where the products
  // of the next pass read it.  Runs at the end of the pass before (the staged rows have all been moved to registers, the
  // packed image of the current state is no longer read), so it is off the chain of dependent exchanges.
  auto walk_back = [&]() {
    if constexpr (FM) {
      const unsigned char* sl = smem + lane * 16;
      frag kda[NT];
#pragma unroll
      for (int s = 0; s < XS; ++s) {
        const u32x4 rk = *reinterpret_cast<const u32x4*>(sl + L::X + (1 * XS + s) * 1024);
        kda[2 * s] = tokens_k(__builtin_bit_cast(frag, u32x2{rk[0], rk[1]}));
        kda[2 * s + 1] = tokens_k(__builtin_bit_cast(frag, u32x2{rk[2], rk[3]}));
      }
      frag nG[TPW];
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) {
        u32x2 raw = *reinterpret_cast<const u32x2*>(smem + L::GDS + (w * TPW + jj) * 512 + lane * 8);
        raw[0] = upd ? raw[0] ^ 0x80008000u : 0u;
        raw[1] = upd ? raw[1] ^ 0x80008000u : 0u;
        nG[jj] = __builtin_bit_cast(frag, raw);
        IO::mma(bTm[jj], nG[jj], ones);
      }
#pragma unroll
      for (int I = 0; I < NT; ++I)
#pragma unroll
        for (int jj = 0; jj < TPW; ++jj) {
          IO::mma(Wm[I][jj], kda[I], nG[jj]);
          *reinterpret_cast<frag*>(smem + lane * 16 + pk_off(I, w * TPW + jj)) = IO::to_frag(Wm[I][jj]);
        }
    }
  };
  if constexpr (FM) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    lds_barrier();
    walk_back();
  }

  for (int st = a.n_stages - 1; st >= 0; --st) {
    // ---- the mini-batch's copies have landed (every wave waits for its own, then all meet)
    // Memory operations complete in the order they were issued, stores included (they count until the cache has
    // acknowledged them).  Behind the copies of this mini-batch (issued early in the previous pass of the loop) every
    // wave has issued at least three stores (its d_xq, d_xv and d_xk rows); waiting for everything would wait for
    // those as well, a store latency per mini-batch, so all but the three youngest operations are waited for.  The
    // first pass has no stores behind its copies.
    if (st == a.n_stages - 1)
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kStoresBehindCopiesAtLoopTop) : "memory");
    lds_barrier();
    const unsigned char* sl = smem + lane * 16;
    frag q[NT], k[NT], qo[TPW], ko[TPW], vo[TPW], oo[TPW];  // full rows of xq, xk; own features of all four
    if constexpr (BF) {
#pragma unroll
      for (int s = 0; s < XS; ++s) {
        const u32x4 rq = *reinterpret_cast<const u32x4*>(sl + L::X + (0 * XS + s) * 1024);
        const u32x4 rk = *reinterpret_cast<const u32x4*>(sl + L::X + (1 * XS + s) * 1024);
        q[2 * s] = __builtin_bit_cast(frag, u32x2{rq[0], rq[1]});
        q[2 * s + 1] = __builtin_bit_cast(frag, u32x2{rq[2], rq[3]});
        k[2 * s] = __builtin_bit_cast(frag, u32x2{rk[0], rk[1]});
        k[2 * s + 1] = __builtin_bit_cast(frag, u32x2{rk[2], rk[3]});
      }
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) {
        const int Jo = w * TPW + jj;
        qo[jj] = *reinterpret_cast<const frag*>(sl + L::X + (0 * XS + (Jo >> 1)) * 1024 + 8 * (Jo & 1));
        ko[jj] = *reinterpret_cast<const frag*>(sl + L::X + (1 * XS + (Jo >> 1)) * 1024 + 8 * (Jo & 1));
        vo[jj] = *reinterpret_cast<const frag*>(sl + L::X + (2 * XS + (Jo >> 1)) * 1024 + 8 * (Jo & 1));
        oo[jj] = *reinterpret_cast<const frag*>(sl + L::X + (3 * XS + (Jo >> 1)) * 1024 + 8 * (Jo & 1));
      }
    } else {
#pragma unroll
      for (int s = 0; s < NT; ++s) {
        q[s] = *reinterpret_cast<const frag*>(sl + L::X + (0 * XS + s) * 1024);
        k[s] = *reinterpret_cast<const frag*>(sl + L::X + (1 * XS + s) * 1024);
      }
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) {
        qo[jj] = *reinterpret_cast<const frag*>(sl + L::X + (0 * XS + w * TPW + jj) * 1024);
        ko[jj] = *reinterpret_cast<const frag*>(sl + L::X + (1 * XS + w * TPW + jj) * 1024);
        vo[jj] = *reinterpret_cast<const frag*>(sl + L::X + (2 * XS + w * TPW + jj) * 1024);
        oo[jj] = *reinterpret_cast<const frag*>(sl + L::X + (3 * XS + w * TPW + jj) * 1024);
      }
    }
    float lr_c;
    f32x4 lr_s;
    {
      const uint32_t* lrw = reinterpret_cast<const uint32_t*>(smem + L::LR);
      const u32x4 w4 = *reinterpret_cast<const u32x4*>(lrw + 4 * g);
      auto cv = [&](uint32_t x) { return BF ? __uint_as_float(x << 16) : __uint_as_float(x); };
      lr_c = (FULL || c < K) ? cv(lrw[c]) : 0.f;
#pragma unroll
      for (int r = 0; r < 4; ++r) lr_s[r] = (FULL || 4 * g + r < K) ? cv(w4[r]) : 0.f;
    }
    f32x4 bT[TPW];
    frag Wn[TPW][NT], kdo[TPW], qdo[TPW];
#pragma unroll
    for (int ii = 0; ii < TPW; ++ii) {
      const int Io = w * TPW + ii;
      if constexpr (FM)
        bT[ii] = bTm[ii];
      else
        bT[ii] = *reinterpret_cast<const f32x4*>(sl + L::Bv + Io * 1024) - bbar;
#pragma unroll
      for (int J = 0; J < NT; ++J) {
        if constexpr (PK)  // stored as (m = j, k = i): transposed on the matrix pipe
          Wn[ii][J] = tokens_k(*reinterpret_cast<const frag*>(sl + pk_off(Io, J)));
        else
          Wn[ii][J] = IO::to_frag(*reinterpret_cast<const f32x4*>(sl + L::W + (Io * NT + J) * 1024) - mrowo[ii]);
      }
      kdo[ii] = tokens_k(ko[ii]);
      qdo[ii] = tokens_k(qo[ii]);
      fr(KD, Io) = kdo[ii];
      fr(QD, Io) = qdo[ii];
    }

    // ---- forward intermediates of the own features: Z1 = XK W + b, Zq = XQ W + b; partial attention blocks
    f32x4 z1[TPW], zb[TPW];
#pragma unroll
    for (int jj = 0; jj < TPW; ++jj) {
      const int Jo = w * TPW + jj;
      z1[jj] = zb[jj] = bT[jj];
#pragma unroll
      for (int qq = 0; qq < NQ; ++qq) {
        // W tiles (rows 2qq / 2qq+1, own column tile), transposed on the matrix pipe: (m = j, k = i)
        frag wa0, wa1;
        if constexpr (PK) {
          wa0 = *reinterpret_cast<const frag*>(sl + pk_off(2 * qq, Jo));
          wa1 = *reinterpret_cast<const frag*>(sl + pk_off(2 * qq + 1, Jo));
        } else {
          wa0 = tokens_k(IO::to_frag(*reinterpret_cast<const f32x4*>(sl + L::W + ((2 * qq) * NT + Jo) * 1024) - mrow[2 * qq]));
          wa1 = tokens_k(IO::to_frag(*reinterpret_cast<const f32x4*>(sl + L::W + ((2 * qq + 1) * NT + Jo) * 1024) - mrow[2 * qq + 1]));
        }
        IO::mma2(z1[jj], wa0, wa1, k[2 * qq], k[2 * qq + 1]);
        IO::mma2(zb[jj], wa0, wa1, q[2 * qq], q[2 * qq + 1]);
      }
    }
    // bf16: every wave forms the whole attention block itself (it holds the full rows of XQ and XK anyway, and the
    // matrix pipe has room): two k = 32 instructions per orientation instead of one partial block per wave that
    // crosses LDS (a write, NW reads and NW - 1 vector additions per orientation).  f32 products are bound by the
    // matrix pipe, there the waves share the work; so they do at d = 128, where the register file is full.
    f32x4 at = zero4, at2 = zero4;
    if constexpr (FULL_AT) {
      mma_all(at, k, q);   // [s = 4g+r][t = c]
      mma_all(at2, q, k);  // [t = 4g+r][s = c]
    } else {
      mma_own(at, ko, qo);
      mma_own(at2, qo, ko);
      pt(P_AT, w) = at;
      pt(P_AT2, w) = at2;
    }
    // ---- X1: raw moments of Z1
    f32x4 bq[TPW];
    float S1[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int jj = 0; jj < TPW; ++jj) {
      bq[jj] = gam[jj] * (bet[jj] - (IO::to_f32(vo[jj]) - IO::to_f32(ko[jj])));
      const f32x4 az = a2[jj] * z1[jj];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        S1[0] += z1[jj][r];
        S1[1] += z1[jj][r] * z1[jj][r];
        S1[2] += az[r];
        S1[3] += az[r] * z1[jj][r];
        S1[4] += bq[jj][r];
        S1[5] += bq[jj][r] * z1[jj][r];
      }
    }
    xpub(0, S1);
    // window: S = XK dW + db (own features) needs nothing of this mini-batch but XK
    f32x4 S[TPW];
#pragma unroll
    for (int ii = 0; ii < TPW; ++ii) {
      S[ii] = dbT[ii];
#pragma unroll
      for (int qq = 0; qq < NQ; ++qq)
        IO::mma2(S[ii], IO::to_frag(dWc[2 * qq][ii]), IO::to_frag(dWc[2 * qq + 1][ii]), k[2 * qq], k[2 * qq + 1]);
    }
    xcol(0, S1);
    // every wave has moved the staged mini-batch to registers: the next one may be copied in
    fetch(st - 1);

    const float mu1 = S1[0] * inv_d;
    const float rstd1 = __builtin_amdgcn_rsqf(fmaxf(S1[1] * inv_d - mu1 * mu1, 0.f) + a.eps);
    const float sa_xh = rstd1 * (S1[2] - mu1 * sum_a);                                    // sum a2 xh
    const float sa_xh2 = rstd1 * rstd1 * (S1[3] - 2.f * mu1 * S1[2] + mu1 * mu1 * sum_a);  // sum a2 xh^2
    const float s_gx = sa_xh + S1[4];                                                     // sum gx
    const float s_gxxh = sa_xh2 + rstd1 * (S1[5] - mu1 * S1[4]);                          // sum gx xh
    const float mgx = s_gx * inv_d, sgx = s_gxxh * inv_d;
    f32x4 xh[TPW], gx[TPW], G[TPW];
#pragma unroll
    for (int jj = 0; jj < TPW; ++jj) {
      xh[jj] = (z1[jj] - mu1) * rstd1;
      gx[jj] = a2[jj] * xh[jj] + bq[jj];
      G[jj] = (gx[jj] - mgx - xh[jj] * sgx) * rstd1;
    }
    // ---- eta, tril(A), M = eta (1 + A) in both orientations
    f32x4 eta, onepA, eta2, onepA2, nM, M2;
    {
      const f32x4 At = FULL_AT ? at : ptsum(P_AT), At2 = FULL_AT ? at2 : ptsum(P_AT2);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const bool low = 4 * g + r <= c;
        eta[r] = low ? te_c * lr_s[r] : 0.f;
        onepA[r] = low ? 1.f + At[r] : 0.f;
        nM[r] = -eta[r] * onepA[r];
        const bool low2 = c <= 4 * g + r;
        eta2[r] = low2 ? te_s[r] * lr_c : 0.f;
        onepA2[r] = low2 ? 1.f + At2[r] : 0.f;
        M2[r] = eta2[r] * onepA2[r];
      }
    }
    // ---- Zb = XQ W + b - M G ; X2: raw moments of Zb and of the output-LayerNorm backward
    frag Gf[TPW];
    f32x4 gx2[TPW];
    float S2[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    {
      const frag nMf = IO::to_frag(nM);
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) {
        Gf[jj] = IO::to_frag(G[jj]);
        fr(GF, w * TPW + jj) = Gf[jj];
        IO::mma(zb[jj], tokens_k(Gf[jj]), nMf);
        gx2[jj] = IO::to_f32(oo[jj]) * gam[jj];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          S2[0] += zb[jj][r];
          S2[1] += zb[jj][r] * zb[jj][r];
          S2[2] += gx2[jj][r];
          S2[3] += gx2[jj][r] * zb[jj][r];
        }
      }
    }
    xpub(1, S2);
    xcol(1, S2);
    frag Zf[TPW], Zd[TPW];
    {
      const float mu2 = S2[0] * inv_d;
      const float rstd2 = __builtin_amdgcn_rsqf(fmaxf(S2[1] * inv_d - mu2 * mu2, 0.f) + a.eps);
      const float m1 = S2[2] * inv_d, m2 = rstd2 * (S2[3] - mu2 * S2[2]) * inv_d;
      f32x4 P = zero4, P2 = zero4;
      frag Gl[TPW], Zl[TPW];
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) {
        const f32x4 x2 = (zb[jj] - mu2) * rstd2;
        const f32x4 dO = IO::to_f32(oo[jj]);
        dgam[jj] += dO * x2;
        dbet[jj] += dO;
        const f32x4 dzb = (gx2[jj] - m1 - x2 * m2) * rstd2;
        Zf[jj] = IO::to_frag(dzb);
        Zd[jj] = tokens_k(Zf[jj]);
        fr(ZF, w * TPW + jj) = Zf[jj];
        fr(ZD, w * TPW + jj) = Zd[jj];
        if (BF) {
          // P feeds the gradients of eta (small differences of large sums): bf16 head + tail of both factors
          Gl[jj] = IO::to_frag(G[jj] - IO::to_f32(Gf[jj]));
          Zl[jj] = IO::to_frag(dzb - IO::to_f32(Zf[jj]));
          if constexpr (FULL_AT) {
            fr(GL, w * TPW + jj) = Gl[jj];
            fr(ZL, w * TPW + jj) = Zl[jj];
          }
        }
      }
      // ---- partial P = dZb G^T in both orientations (FULL_AT: formed whole behind the next exchange)
      if constexpr (!FULL_AT) {
        mma_own(P, Gf, Zf);   // [s][t]
        mma_own(P2, Zf, Gf);  // [t][s]
        if (BF) {
          mma_own(P, Gl, Zf);
          mma_own(P, Gf, Zl);
          mma_own(P2, Zl, Gf);
          mma_own(P2, Zf, Gl);
        }
        pt(P_P, w) = P;
        pt(P_P2, w) = P2;
      }
    }
    // ---- DGM = M^T dZb (own features) ; X3: the partial P blocks and dZb / G fragments travel with the six
    //      sums of the second-order LayerNorm, none of which needs P
    const bool tok_ok = FULL || c < K;
    const size_t tokoff = (bh * (size_t)a.seq_stride + (size_t)st * K + c) * D;
    f32x4 dK[TPW], DGM[TPW], TMP[TPW];
    {
      const frag M2f = IO::to_frag(M2);
#pragma unroll
      for (int ii = 0; ii < TPW; ++ii) {
        DGM[ii] = zero4;
        IO::mma(DGM[ii], Zd[ii], M2f);
      }
    }
    const float last = te_last * lr_c;
    f32x4 u[TPW];
    float S4[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int jj = 0; jj < TPW; ++jj) {
      u[jj] = (DGM[jj] + last * S[jj]) * rstd1;  // u = -dG rstd1
      const f32x4 au = a2[jj] * u[jj];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        S4[0] += u[jj][r];
        S4[1] += u[jj][r] * xh[jj][r];
        S4[2] += au[r];
        S4[3] += au[r] * xh[jj][r];
        S4[4] += u[jj][r] * gx[jj][r];
        S4[5] += G[jj][r] * S[jj][r];
      }
    }
    xpub(2, S4);
    // window: TMP = G dW^T (own features) needs the G fragments of every wave, published one exchange ago
    frag Gfa[NT];
#pragma unroll
    for (int J = 0; J < NT; ++J) Gfa[J] = fr(GF, J);
#pragma unroll
    for (int ii = 0; ii < TPW; ++ii) {
      TMP[ii] = zero4;
#pragma unroll
      for (int qq = 0; qq < NQ; ++qq)
        IO::mma2(TMP[ii], IO::to_frag(DT[2 * qq][ii]), IO::to_frag(DT[2 * qq + 1][ii]), Gfa[2 * qq], Gfa[2 * qq + 1]);
    }
    xcol(2, S4);
    frag Zfa[NT];
#pragma unroll
    for (int J = 0; J < NT; ++J) Zfa[J] = fr(ZF, J);
    f32x4 dA, dEta, dA2, dEta2;
    {
      f32x4 P, P2;
      if constexpr (FULL_AT) {
        frag Gla[NT], Zla[NT];
#pragma unroll
        for (int J = 0; J < NT; ++J) {
          Gla[J] = fr(GL, J);
          Zla[J] = fr(ZL, J);
        }
        P = P2 = zero4;
        mma_all(P, Gfa, Zfa);   // [s][t]
        mma_all(P2, Zfa, Gfa);  // [t][s]
        mma_all(P, Gla, Zfa);
        mma_all(P2, Zla, Gfa);
        mma_all(P, Gfa, Zla);
        mma_all(P2, Zfa, Gla);
      } else {
        P = ptsum(P_P);
        P2 = ptsum(P_P2);
      }
      dA = -P * eta;
      dEta = -P * onepA;
      dA2 = -P2 * eta2;
      dEta2 = -P2 * onepA2;
    }
    // ---- dXQ = dO + dZb W^T + dA XK   (own features)
    {
      const frag dAf = IO::to_frag(dA);
      f32x4 dQ[TPW];
#pragma unroll
      for (int ii = 0; ii < TPW; ++ii) {
        dQ[ii] = IO::to_f32(oo[ii]);
        mma_all(dQ[ii], Wn[ii], Zfa);
        // bf16: a k = 16 instruction accumulating straight onto the result of a k = 32 one has given wrong
        // sums, so the rank-16 term is issued as k = 32 with a zero half
        if (BF)
          IO::mma2(dQ[ii], kdo[ii], IO::zero(), dAf, IO::zero());
        else
          IO::mma(dQ[ii], kdo[ii], dAf);
      }
      if (tok_ok) store_own(a.d_xq, tokoff, dQ);
    }
    // ---- dK = dA^T XQ   (own features)
    {
      const frag dA2f = IO::to_frag(dA2);
#pragma unroll
      for (int ii = 0; ii < TPW; ++ii) {
        dK[ii] = zero4;
        IO::mma(dK[ii], qdo[ii], dA2f);
      }
    }
    const float dl = -S4[5];
    frag Z1f[TPW], Z1d[TPW];
    {
      const float s1 = S4[0] * inv_d, s2 = S4[1] * inv_d;
      const float q1 = (s1 * sum_a + s2 * sa_xh - S4[2] + s2 * s_gx + sgx * S4[0]) * inv_d;
      const float q2 = s1 * sa_xh + s2 * sa_xh2 - S4[3] + s2 * s_gxxh + sgx * S4[1];  // sum dxh xh
      const float s_uG = rstd1 * (S4[4] - mgx * S4[0] - sgx * S4[1]);                  // sum u G
      const float dsig = -(q2 * rstd1 - s_uG);
      f32x4 ndy[TPW];
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) {
        const f32x4 dgx = s1 + xh[jj] * s2 - u[jj];
        const f32x4 dy = gam[jj] * dgx;
        // gO = gamma xh + beta - target = gx / gamma, kept as gamma-free form through bq
        const f32x4 gO = gam[jj] * xh[jj] + bet[jj] - (IO::to_f32(vo[jj]) - IO::to_f32(ko[jj]));
        dgam[jj] += gO * dgx + dy * xh[jj];
        dbet[jj] += dy;
        const f32x4 dxh = dy * gam[jj] + gx[jj] * s2 + u[jj] * sgx;
        Z1f[jj] = IO::to_frag((dxh - q1) * rstd1 + xh[jj] * (dsig * inv_d));
        Z1d[jj] = tokens_k(Z1f[jj]);
        fr(Z1F, w * TPW + jj) = Z1f[jj];
        fr(Z1D, w * TPW + jj) = Z1d[jj];
        dK[jj] += dy - last * TMP[jj];
        ndy[jj] = -dy;
      }
      if (tok_ok) store_own(a.d_xv, tokoff, ndy);
    }
    // ---- X4: dZ1 fragments
    // FM: the copies of the next mini-batch (issued behind X1; two stores, d_xq and d_xv, are younger) have to be
    // visible to every wave behind this barrier: the walk back at the end of the pass reads them
    if constexpr (FM) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kStoresBehindCopiesAtX4) : "memory");
    lds_barrier();
    {
      frag Z1fa[NT];
#pragma unroll
      for (int J = 0; J < NT; ++J) Z1fa[J] = fr(Z1F, J);
#pragma unroll
      for (int ii = 0; ii < TPW; ++ii) mma_all(dK[ii], Wn[ii], Z1fa);
      if (tok_ok) store_own(a.d_xk, tokoff, dK);
    }
    // ---- d lr (first wave), d token_eta (last wave): work of a single wave is skew at the next barrier.  Where it
    // goes is a matter of measurement: in front of the state-gradient products when the walk back follows them
    // (451 against 454 us at B = 32, 335 against 350 at B = 16), behind them otherwise (packed states 450 -> 438 us,
    // f32 741 -> 726 us)
    auto single_wave_outputs = [&]() {
      if (w == 0) {
        float e2 = 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) e2 += dEta2[r] * te_s[r];
        const float dlr = xg_sum(e2) + te_last * dl;
        if (g == 0 && tok_ok)
          IO::store1(static_cast<elem*>(a.d_lr) + bh * (size_t)a.seq_stride + (size_t)st * K + c, dlr);
      }
      if (w == NW - 1) {
        float e1 = 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) e1 += dEta[r] * lr_s[r];
        float dte = xg_sum(e1);
        const float tail = row16_sum_dpp(dl * lr_c);
        if (c == K - 1) dte += tail;
        if (g == 0 && tok_ok) atomicAdd(a.d_token_eta + (size_t)st * K + c, dte);
      }
    };
    if constexpr (FM) single_wave_outputs();
    // ---- state gradient: dW += XQ^T dZb + XK^T dZ1 (column slice and transposed row slice), db
#pragma unroll
    for (int I = 0; I < NT; ++I) {
      const frag qa = fr(QD, I), ka = fr(KD, I), za = fr(ZD, I), z1a = fr(Z1D, I);
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) {
        IO::mma2(dWc[I][jj], qa, ka, Zd[jj], Z1d[jj]);
        IO::mma2(DT[I][jj], za, z1a, qdo[jj], kdo[jj]);
      }
    }
#pragma unroll
    for (int jj = 0; jj < TPW; ++jj) IO::mma2(dbT[jj], Zd[jj], Z1d[jj], ones, ones);
    if constexpr (!FM) single_wave_outputs();
    // FM: the state entering the next mini-batch of the scan.  Placed last: its short dependent chain (transposes,
    // products, conversions, LDS writes) then runs behind the state-gradient products instead of in front of the
    // dXK products and stores (measured 479 -> 463 us).  Behind the first mini-batch of the sequence nothing new is
    // staged: the walk then works on stale rows, its result is never read, and the loop keeps one shape.
    if constexpr (FM) walk_back();
  }

  // ---- results carried over the whole scan
#pragma unroll
  for (int I = 0; I < NT; ++I)
#pragma unroll
    for (int jj = 0; jj < TPW; ++jj)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        a.d_W0[bh * D * D + feat(I, 4 * g + r) * D + feat(w * TPW + jj, c)] = dWc[I][jj][r];
#pragma unroll
  for (int jj = 0; jj < TPW; ++jj) {
    const int f = own_offset<TPW>(w, jj, g);
    if (c == 0) store4<F32>(a.d_b0 + bh * D + f, dbT[jj]);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float sg = row16_sum_dpp(dgam[jj][r]), sbt = row16_sum_dpp(dbet[jj][r]);
      if (c == 0) {
        atomicAdd(a.d_gamma + h * D + f + r, sg);
        atomicAdd(a.d_beta + h * D + f + r, sbt);
      }
    }
  }
}

}  // namespace ttt
