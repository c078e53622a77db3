// TTT-Linear fused backward for gfx950, bf16 I/O, checkpoint interval 1: ONE wavefront per
// (batch, head), everything that lives across mini-batches in registers, no barrier at all.
//
// Arithmetic: the reverse scan of ttt_linear_bwd.hip.h (reference
// rust/fused/src/linear_fused_tile/backward/kernel.rs:253-429, backward/stage.rs:42-1006, second-order
// LayerNorm layer_norm.rs:428-709).  With a checkpoint per mini-batch the state W_t entering stage t is
// read, not recomputed, so the only chain through the scan is the state gradient dW, db.
//
// Layouts (see ttt_frag.hip.h): every [16 tokens x d] tile is held transposed, tile J of the feature axis
// as one f32x4 per lane: value r of lane (c, g) is (feature feat(J, 4g+r), token c).  A row statistic is
// in-lane adds plus one sum over the four lane groups.  The same registers, converted to bf16, are both
// the A operand (m = token, k = feature) and the B operand (k = feature, n = token) of the matrix
// instructions; the form with tokens along k comes from one multiplication by an identity fragment.
//   W_t     read from the checkpoint as A operand (m = row i, k = column j) for dQ = dZb W^T and
//           dK += dZ1 W^T; its transpose (m = j, k = i), for Z1 = XK W and Zq = XQ W, is made on the matrix
//           pipe (identity multiplication, exact for bf16 values).
//   dW      f32 accumulator tiles dWc[I][J] (rows i in registers), updated by one rank-32 product
//           [XQ; XK]^T [dZb; dZ1] per mini-batch.  Its bf16 image is an A operand as it stands (m = j, k = i)
//           for S = XK dW; for G dW^T the image is transposed tile by tile on the matrix pipe.
//   [16 x 16] causal matrices are computed in both orientations (operands swapped) instead of transposed.
// Staging: the checkpoint (16 KiB at d = 64), its bias and the four activation tiles of the next
// mini-batch are copied global -> LDS without passing registers (global_load_lds_dwordx4), each lane
// fetching exactly the 16-byte pieces it will read back itself, so LDS acts as a per-lane queue.
#pragma once
#include "ttt_linear_bwd.hip.h"
#include "ttt_linear_fwd_mw.hip.h"

namespace ttt {

// PK: the W checkpoint arrives packed (bf16 fragments in accumulator order, see store_ckpt_packed)
template <int D, bool PK = false>
struct LinBwdRrLds {
  static constexpr int NT = D / 16;
  static constexpr int W = 0;                       // NT*NT slots of 1 KiB: slot I*NT+J, lane (c,g): W[feat(I,c)][feat(J,4g..4g+3)]
                                                    // packed: NT*NT/2 slots: slot I*NT/2+q = tiles (I,2q), (I,2q+1)
  static constexpr int Bv = W + (PK ? NT * NT / 2 : NT * NT) * 1024;  // NT slots: b[feat(J,4g..4g+3)]
  static constexpr int X = Bv + NT * 1024;          // 4 tensors x NT/2 slots: X[token c][32q + 8g .. +7] (bf16)
  static constexpr int LR = X + 4 * (NT / 2) * 1024;  // 16 dwords: lr of token c, zero-extended bf16
  static constexpr int STAGE = LR + 256;
  static constexpr int M0 = 2 * STAGE;             // D row means of the initial W, then mean(b): the centred state
  static constexpr int BYTES = M0 + (D + 4) * 4;
};

template <class T, int D, bool PK = false>
__global__ void __launch_bounds__(64) ttt_linear_bwd_rr_kernel(LinearBwdArgs a) {
  using IO = Io<T>;
  using frag = typename IO::frag;
  using elem = typename IO::elem;
  using L = LinBwdRrLds<D, PK>;
  static_assert(sizeof(elem) == 2, "bf16 I/O only");
  constexpr int NT = D / 16, NQ = NT / 2;
  constexpr float inv_d = 1.0f / D;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int lane = threadIdx.x, c = lane & 15, g = lane >> 4;
  const size_t bh = blockIdx.x;
  const int h = (int)(bh % a.H);
  const int K = a.K;

  const float te_c = (c < K) ? a.token_eta[c] : 0.f;
  const float te_last = a.token_eta[K - 1];
  f32x4 te_s;
#pragma unroll
  for (int r = 0; r < 4; ++r) te_s[r] = (4 * g + r < K) ? a.token_eta[4 * g + r] : 0.f;
  const frag ident = identity_frag<T>(c, g);
  const frag ones = splat_frag<T>(1.f);
  f32x4 gam[NT], bet[NT], dgam[NT], dbet[NT], dbT[NT];
#pragma unroll
  for (int J = 0; J < NT; ++J) {
    const int f = own_offset<NT>(0, J, g);
    gam[J] = *reinterpret_cast<const f32x4*>(a.gamma + h * D + f);
    bet[J] = *reinterpret_cast<const f32x4*>(a.beta + h * D + f);
    dgam[J] = dbet[J] = f32x4{0.f, 0.f, 0.f, 0.f};
    dbT[J] = a.d_b_out ? *reinterpret_cast<const f32x4*>(a.d_b_out + bh * D + f) : f32x4{0.f, 0.f, 0.f, 0.f};
  }
  // state gradient: dWc[I][J], rows i = feat(I, 4g+r) in registers, columns j = feat(J, c) on lanes
  f32x4 dWc[NT][NT];
#pragma unroll
  for (int I = 0; I < NT; ++I)
#pragma unroll
    for (int J = 0; J < NT; ++J)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        dWc[I][J][r] = a.d_W_out ? a.d_W_out[bh * D * D + feat(I, 4 * g + r) * D + feat(J, c)] : 0.f;
      }

  // rows of absent tokens (c >= K) are never fetched: they stay zero
  for (int i = lane; i < L::BYTES / 16; i += 64) reinterpret_cast<u32x4*>(smem)[i] = u32x4{0u, 0u, 0u, 0u};
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");

  // The scan works on the centred state Wc = W - m 1^T, bc = b - mean(b), as the forward does (centre_state in
  // ttt_linear_fwd_mw.hip.h): Z1 and Zbar feed LayerNorms, which discard a common shift of a row, and dZbar W^T,
  // dZ1 W^T multiply LayerNorm gradients, whose rows sum to zero.  m, mean(b): those of checkpoint 0 (the forward's
  // updates do not move them); a packed checkpoint holds the centred matrix already.
  float* const M0p = reinterpret_cast<float*>(smem + L::M0);
  {
    const size_t c0 = bh * (size_t)a.n_ckpt;
    if (!PK) {
      for (int i = lane; i < D; i += 64) {
        const f32x4* row = reinterpret_cast<const f32x4*>(a.W_ckpt + c0 * D * D + (size_t)i * D);
        float sum = 0.f;
        for (int j = 0; j < D / 4; ++j) {
          const f32x4 v = row[j];
          sum += (v[0] + v[1]) + (v[2] + v[3]);
        }
        M0p[i] = sum * inv_d;
      }
    }
    if (lane == 0) {
      float sum = 0.f;
      for (int f = 0; f < D; ++f) sum += a.b_ckpt[c0 * D + f];
      M0p[D] = sum * inv_d;
    }
    __syncthreads();
  }
  float mrow[NT];  // m of row feat(I, c)
#pragma unroll
  for (int I = 0; I < NT; ++I) mrow[I] = PK ? 0.f : M0p[feat(I, c)];
  const float bbar = M0p[D];

  // The copies of one mini-batch are issued in NPART portions spread over the previous mini-batch's
  // arithmetic: the memory pipeline accepts only so many requests at a time, and a wave that issues a
  // whole mini-batch at once (29 KiB) sits in the issue for thousands of cycles while all other units do
  // the same.  Everything goes through LDS, nothing through registers: a load the compiler knows of would
  // make it place a wait for ALL outstanding memory operations, these copies included, before its first use.
  constexpr int NPART = NT + 3;
  auto fetch = [&](int stage, int part) {
    if (stage < 0) return;
    unsigned char* dst = smem + (stage & 1) * L::STAGE;
    const size_t ci = bh * (size_t)a.n_ckpt + stage;
    const float* Wg = a.W_ckpt + ci * D * D;
    const float* bg = a.b_ckpt + ci * D;
    const unsigned dst_lds = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)dst;
    // wave-uniform base + 32-bit lane offset: one address register per copy
    auto dma = [&](const void* base, unsigned lane_off, int off) { lds_dma16(base, lane_off, dst_lds + off); };
    const size_t tok0 = (bh * (size_t)a.seq_stride + (size_t)stage * K) * D;
    const unsigned xoff = (unsigned)(c * D + 8 * g) * 2u;
    if (part < NT) {
      const int I = part;
      if (PK) {
#pragma unroll
        for (int q = 0; q < NQ; ++q) dma(Wg, (unsigned)((I * NQ + q) * 1024 + lane * 16), L::W + (I * NQ + q) * 1024);
      } else {
#pragma unroll
        for (int J = 0; J < NT; ++J)
          dma(Wg, (unsigned)(feat(I, c) * D + own_offset<NT>(0, J, g)) * 4u, L::W + (I * NT + J) * 1024);
      }
    } else if (part == NT) {
#pragma unroll
      for (int J = 0; J < NT; ++J) dma(bg, (unsigned)own_offset<NT>(0, J, g) * 4u, L::Bv + J * 1024);
      // lr of the 16 tokens (absent ones: a clamped position, zeroed at use), one 2-byte element per lane
      if (lane < 16)
        lds_dma2(static_cast<const elem*>(a.lr) + bh * (size_t)a.seq_stride + (size_t)stage * K,
                 2u * (unsigned)(c < K ? c : K - 1), dst_lds + L::LR);
    } else if (c < K) {
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        if (part == NT + 1) {
          dma(static_cast<const elem*>(a.xq) + tok0, xoff + 64u * q, L::X + (0 * NQ + q) * 1024);
          dma(static_cast<const elem*>(a.xk) + tok0, xoff + 64u * q, L::X + (1 * NQ + q) * 1024);
        } else {
          dma(static_cast<const elem*>(a.xv) + tok0, xoff + 64u * q, L::X + (2 * NQ + q) * 1024);
          dma(static_cast<const elem*>(a.d_out) + tok0, xoff + 64u * q, L::X + (3 * NQ + q) * 1024);
        }
      }
    }
  };
  auto rowsum = [&](const f32x4 (&x)[NT]) {
    float s = 0.f;
#pragma unroll
    for (int J = 0; J < NT; ++J) s += (x[J][0] + x[J][1]) + (x[J][2] + x[J][3]);
    return xg_sum(s);
  };
  auto rowdot = [&](const f32x4 (&x)[NT], const f32x4 (&y)[NT]) {
    float s = 0.f;
#pragma unroll
    for (int J = 0; J < NT; ++J)
#pragma unroll
      for (int r = 0; r < 4; ++r) s += x[J][r] * y[J][r];
    return xg_sum(s);
  };
  // tile with tokens along k: A operand (m = feature, k = token) or B operand (k = token, n = feature)
  auto tokens_k = [&](frag x) {
    f32x4 t = {0.f, 0.f, 0.f, 0.f};
    IO::mma(t, x, ident);
    return IO::to_frag(t);
  };
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};

#pragma unroll
  for (int part = 0; part < NPART; ++part) fetch(a.n_stages - 1, part);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  for (int st = a.n_stages - 1; st >= 0; --st) {
    fetch(st - 1, 0);
    const unsigned char* sb = smem + (st & 1) * L::STAGE + lane * 16;
    float lr_c;
    f32x4 lr_s;
    {
      const uint32_t* lrw = reinterpret_cast<const uint32_t*>(smem + (st & 1) * L::STAGE + L::LR);
      lr_c = (c < K) ? __uint_as_float(lrw[c] << 16) : 0.f;
      const u32x4 w4 = *reinterpret_cast<const u32x4*>(lrw + 4 * g);
#pragma unroll
      for (int r = 0; r < 4; ++r) lr_s[r] = (4 * g + r < K) ? __uint_as_float(w4[r] << 16) : 0.f;
    }

    // ---- this mini-batch's tiles and the state entering it
    frag q[NT], k[NT], v[NT], o[NT];
#pragma unroll
    for (int qq = 0; qq < NQ; ++qq) {
      auto get = [&](int ten, frag& lo, frag& hi) {
        const u32x4 raw = *reinterpret_cast<const u32x4*>(sb + L::X + (ten * NQ + qq) * 1024);
        lo = __builtin_bit_cast(frag, u32x2{raw[0], raw[1]});
        hi = __builtin_bit_cast(frag, u32x2{raw[2], raw[3]});
      };
      get(0, q[2 * qq], q[2 * qq + 1]);
      get(1, k[2 * qq], k[2 * qq + 1]);
      get(2, v[2 * qq], v[2 * qq + 1]);
      get(3, o[2 * qq], o[2 * qq + 1]);
    }
    f32x4 bT[NT];
#pragma unroll
    for (int J = 0; J < NT; ++J) bT[J] = *reinterpret_cast<const f32x4*>(sb + L::Bv + J * 1024) - bbar;
    frag Wn[NT][NT], kd[NT], qd[NT];
#pragma unroll
    for (int I = 0; I < NT; ++I) {
      kd[I] = tokens_k(k[I]);
      qd[I] = tokens_k(q[I]);
    }

    if (1 < NPART) fetch(st - 1, 1);
    // ---- forward intermediates: Z1 = XK W + b, Zq = XQ W + b, attention block in both orientations
    f32x4 z1[NT], zb[NT], At = zero4, At2 = zero4;
#pragma unroll
    for (int J = 0; J < NT; ++J) z1[J] = zb[J] = bT[J];
#pragma unroll
    for (int qq = 0; qq < NQ; ++qq) {
      frag Wa[2][NT];
#pragma unroll
      for (int e = 0; e < 2; ++e)
#pragma unroll
        for (int J = 0; J < NT; ++J) {
          const int I = 2 * qq + e;
          if constexpr (PK) {
            Wa[e][J] = *reinterpret_cast<const frag*>(sb + L::W + (I * NQ + (J >> 1)) * 1024 + 8 * (J & 1));
            Wn[I][J] = tokens_k(Wa[e][J]);
          } else {
            Wn[I][J] = IO::to_frag(*reinterpret_cast<const f32x4*>(sb + L::W + (I * NT + J) * 1024) - mrow[I]);
            Wa[e][J] = tokens_k(Wn[I][J]);  // tile transpose: (m = j, k = i)
          }
        }
#pragma unroll
      for (int J = 0; J < NT; ++J) {
        IO::mma2(z1[J], Wa[0][J], Wa[1][J], k[2 * qq], k[2 * qq + 1]);
        IO::mma2(zb[J], Wa[0][J], Wa[1][J], q[2 * qq], q[2 * qq + 1]);
      }
      IO::mma2(At, k[2 * qq], k[2 * qq + 1], q[2 * qq], q[2 * qq + 1]);   // [s = 4g+r][t = c]
      IO::mma2(At2, q[2 * qq], q[2 * qq + 1], k[2 * qq], k[2 * qq + 1]);  // [t = 4g+r][s = c]
    }

    if (2 < NPART) fetch(st - 1, 2);
    // ---- first LayerNorm and the gradient of the reconstruction loss
    f32x4 xh[NT], G[NT], gO[NT];
    float rstd1, sgx;
    {
      const float mu = rowsum(z1) * inv_d;
      const float var = rowdot(z1, z1) * inv_d - mu * mu;
      rstd1 = __builtin_amdgcn_rsqf(fmaxf(var, 0.f) + a.eps);
#pragma unroll
      for (int J = 0; J < NT; ++J) {
        xh[J] = (z1[J] - mu) * rstd1;
        gO[J] = gam[J] * xh[J] + bet[J] - (IO::to_f32(v[J]) - IO::to_f32(k[J]));
        G[J] = gO[J] * gam[J];  // gx for now
      }
      const float mgx = rowsum(G) * inv_d;
      sgx = rowdot(G, xh) * inv_d;
#pragma unroll
      for (int J = 0; J < NT; ++J) G[J] = (G[J] - mgx - xh[J] * sgx) * rstd1;
    }
    // ---- eta, tril(A), M = eta (1 + A) in both orientations
    f32x4 eta, onepA, eta2, onepA2, nM, M2;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const bool low = 4 * g + r <= c;   // s <= t with s = 4g+r, t = c
      eta[r] = low ? te_c * lr_s[r] : 0.f;
      onepA[r] = low ? 1.f + At[r] : 0.f;
      nM[r] = -eta[r] * onepA[r];
      const bool low2 = c <= 4 * g + r;  // s <= t with t = 4g+r, s = c
      eta2[r] = low2 ? te_s[r] * lr_c : 0.f;
      onepA2[r] = low2 ? 1.f + At2[r] : 0.f;
      M2[r] = eta2[r] * onepA2[r];
    }
    if (3 < NPART) fetch(st - 1, 3);
    // ---- Zb = XQ W + b - M G
    frag Gf[NT];
    {
      const frag nMf = IO::to_frag(nM);
#pragma unroll
      for (int J = 0; J < NT; ++J) {
        Gf[J] = IO::to_frag(G[J]);
        IO::mma(zb[J], tokens_k(Gf[J]), nMf);
      }
    }
    if (4 < NPART) fetch(st - 1, 4);
    // ---- output LayerNorm and its backward: dZb
    frag Zf[NT], Zd[NT];
    f32x4 DZB[NT];
    {
      const float mu = rowsum(zb) * inv_d;
      const float var = rowdot(zb, zb) * inv_d - mu * mu;
      const float rstd2 = __builtin_amdgcn_rsqf(fmaxf(var, 0.f) + a.eps);
      f32x4 gx2[NT];
#pragma unroll
      for (int J = 0; J < NT; ++J) {
        zb[J] = (zb[J] - mu) * rstd2;  // x2
        const f32x4 dO = IO::to_f32(o[J]);
        dgam[J] += dO * zb[J];
        dbet[J] += dO;
        gx2[J] = dO * gam[J];
      }
      const float m1 = rowsum(gx2) * inv_d, m2 = rowdot(gx2, zb) * inv_d;
#pragma unroll
      for (int J = 0; J < NT; ++J) {
        DZB[J] = (gx2[J] - m1 - zb[J] * m2) * rstd2;
        Zf[J] = IO::to_frag(DZB[J]);
        Zd[J] = tokens_k(Zf[J]);
      }
    }
    if (5 < NPART) fetch(st - 1, 5);
    // ---- P = dZb G^T in both orientations; dA = -P eta, d eta = -P (1 + A)
    f32x4 dA, dEta, dA2, dEta2;
    {
      // P feeds the gradients of eta, which are small differences of large sums: both factors are split
      // into a bf16 head and a bf16 tail and the three leading partial products are kept
      f32x4 P = zero4, P2 = zero4;
#pragma unroll
      for (int qq = 0; qq < NQ; ++qq) {
        const int J0 = 2 * qq, J1 = 2 * qq + 1;
        const frag Gl0 = IO::to_frag(G[J0] - IO::to_f32(Gf[J0])), Gl1 = IO::to_frag(G[J1] - IO::to_f32(Gf[J1]));
        const frag Zl0 = IO::to_frag(DZB[J0] - IO::to_f32(Zf[J0])), Zl1 = IO::to_frag(DZB[J1] - IO::to_f32(Zf[J1]));
        IO::mma2(P, Gf[J0], Gf[J1], Zf[J0], Zf[J1]);   // [s][t]
        IO::mma2(P, Gl0, Gl1, Zf[J0], Zf[J1]);
        IO::mma2(P, Gf[J0], Gf[J1], Zl0, Zl1);
        IO::mma2(P2, Zf[J0], Zf[J1], Gf[J0], Gf[J1]);  // [t][s]
        IO::mma2(P2, Zl0, Zl1, Gf[J0], Gf[J1]);
        IO::mma2(P2, Zf[J0], Zf[J1], Gl0, Gl1);
      }
      dA = -P * eta;
      dEta = -P * onepA;
      dA2 = -P2 * eta2;
      dEta2 = -P2 * onepA2;
    }
    if (6 < NPART) fetch(st - 1, 6);
    const bool tok_ok = c < K;
    const size_t tok = (bh * (size_t)a.seq_stride + (size_t)st * K + c) * D + 8 * g;
    // ---- dXQ = dO + dZb W^T + dA XK
    {
      const frag dAf = IO::to_frag(dA);
      f32x4 dQ[NT];
#pragma unroll
      for (int I = 0; I < NT; ++I) {
        dQ[I] = IO::to_f32(o[I]);
#pragma unroll
        for (int qq = 0; qq < NQ; ++qq) IO::mma2(dQ[I], Wn[I][2 * qq], Wn[I][2 * qq + 1], Zf[2 * qq], Zf[2 * qq + 1]);
        // a k = 16 instruction accumulating straight onto the result of a k = 32 one has given wrong sums:
        // the rank-16 term is issued as k = 32 with a zero half
        IO::mma2(dQ[I], kd[I], IO::zero(), dAf, IO::zero());
      }
      if (tok_ok)
#pragma unroll
        for (int qq = 0; qq < NQ; ++qq)
          IO::store8(static_cast<elem*>(a.d_xq) + tok + 32 * qq, dQ[2 * qq], dQ[2 * qq + 1]);
    }
    // ---- dK = dA^T XQ ; DGM = M^T dZb ; S = XK dW + db ; TMP = G dW^T
    f32x4 dK[NT], DGM[NT], S[NT], TMP[NT];
    {
      const frag dA2f = IO::to_frag(dA2), M2f = IO::to_frag(M2);
#pragma unroll
      for (int I = 0; I < NT; ++I) {
        dK[I] = DGM[I] = TMP[I] = zero4;
        S[I] = dbT[I];
        IO::mma(dK[I], qd[I], dA2f);
        IO::mma(DGM[I], Zd[I], M2f);
      }
      // dW tiles as A operands: as they are (m = column j, k = row i) for S, transposed on the matrix pipe
      // (m = i, k = j) for G dW^T
#pragma unroll
      for (int qq = 0; qq < NQ; ++qq) {
        frag t0[NT], t1[NT];
#pragma unroll
        for (int J = 0; J < NT; ++J) {
          const frag f0 = IO::to_frag(dWc[2 * qq][J]), f1 = IO::to_frag(dWc[2 * qq + 1][J]);
          IO::mma2(S[J], f0, f1, k[2 * qq], k[2 * qq + 1]);
          t0[J] = tokens_k(f0);
          t1[J] = tokens_k(f1);
        }
#pragma unroll
        for (int pj = 0; pj < NQ; ++pj) {
          IO::mma2(TMP[2 * qq], t0[2 * pj], t0[2 * pj + 1], Gf[2 * pj], Gf[2 * pj + 1]);
          IO::mma2(TMP[2 * qq + 1], t1[2 * pj], t1[2 * pj + 1], Gf[2 * pj], Gf[2 * pj + 1]);
        }
      }
    }
    // ---- through G: second-order LayerNorm, token-local
    const float last = te_last * lr_c;
    const float dl = -rowdot(G, S);
    frag Z1f[NT], Z1d[NT];
    {
      f32x4 u[NT];
#pragma unroll
      for (int J = 0; J < NT; ++J) u[J] = (DGM[J] + last * S[J]) * rstd1;  // u = -dG rstd1
      const float s1 = rowsum(u) * inv_d, s2 = rowdot(u, xh) * inv_d;
      f32x4 dxh[NT], dy[NT];
      float q2 = 0.f;
#pragma unroll
      for (int J = 0; J < NT; ++J) {
        const f32x4 dgx = s1 + xh[J] * s2 - u[J];
        dy[J] = gam[J] * dgx;
        dgam[J] += gO[J] * dgx + dy[J] * xh[J];
        dbet[J] += dy[J];
        dxh[J] = dy[J] * gam[J] + (gO[J] * gam[J]) * s2 + u[J] * sgx;
#pragma unroll
        for (int r = 0; r < 4; ++r) q2 += dxh[J][r] * xh[J][r];
      }
      // sum(dG G) = -sum(u G) / rstd1
      const float q1 = rowsum(dxh) * inv_d;
      const float dsig = -(xg_sum(q2) * rstd1 - rowdot(u, G));
#pragma unroll
      for (int J = 0; J < NT; ++J) {
        Z1f[J] = IO::to_frag((dxh[J] - q1) * rstd1 + xh[J] * (dsig * inv_d));
        Z1d[J] = tokens_k(Z1f[J]);
        dK[J] += dy[J] - last * TMP[J];
        dy[J] = -dy[J];
      }
      if (tok_ok)
#pragma unroll
        for (int qq = 0; qq < NQ; ++qq)
          IO::store8(static_cast<elem*>(a.d_xv) + tok + 32 * qq, dy[2 * qq], dy[2 * qq + 1]);
    }
    // ---- dK += dZ1 W^T
#pragma unroll
    for (int I = 0; I < NT; ++I)
#pragma unroll
      for (int qq = 0; qq < NQ; ++qq) IO::mma2(dK[I], Wn[I][2 * qq], Wn[I][2 * qq + 1], Z1f[2 * qq], Z1f[2 * qq + 1]);
    if (tok_ok)
#pragma unroll
      for (int qq = 0; qq < NQ; ++qq)
        IO::store8(static_cast<elem*>(a.d_xk) + tok + 32 * qq, dK[2 * qq], dK[2 * qq + 1]);
    // ---- d lr, d token_eta
    {
      float e2 = 0.f, e1 = 0.f;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        e2 += dEta2[r] * te_s[r];  // sum over t of d eta[t][s = c] token_eta[t]
        e1 += dEta[r] * lr_s[r];   // sum over s of d eta[t = c][s] lr[s]
      }
      const float dlr = xg_sum(e2) + te_last * dl;
      float dte = xg_sum(e1);
      const float tail = row16_sum_dpp(dl * lr_c);
      if (c == K - 1) dte += tail;
      if (g == 0 && tok_ok) {
        IO::store1(static_cast<elem*>(a.d_lr) + bh * (size_t)a.seq_stride + (size_t)st * K + c, dlr);
        atomicAdd(a.d_token_eta + (size_t)st * K + c, dte);
      }
    }
    // ---- state gradient: dW += XQ^T dZb + XK^T dZ1 (one rank-32 update), db += colsum(dZb + dZ1)
#pragma unroll
    for (int I = 0; I < NT; ++I)
#pragma unroll
      for (int J = 0; J < NT; ++J) {
        IO::mma2(dWc[I][J], qd[I], kd[I], Zd[J], Z1d[J]);
      }
#pragma unroll
    for (int J = 0; J < NT; ++J) IO::mma2(dbT[J], Zd[J], Z1d[J], ones, ones);
    // The next mini-batch's copies to LDS must have landed; this mini-batch's stores and atomics, all issued
    // after them, need not have (the atomics of all units meet on one cache line and take long).  Vector
    // memory operations retire in order on this counter, so the wait leaves exactly those outstanding:
    // 3 tensors x NQ stores, the d_lr store and the d_token_eta atomic.
    static_assert(NQ == 1 || NQ == 2, "counted wait below");
    if (NQ == 2)
      asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else
      asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
  }

  // ---- results carried over the whole scan
#pragma unroll
  for (int I = 0; I < NT; ++I)
#pragma unroll
    for (int J = 0; J < NT; ++J)
#pragma unroll
      for (int r = 0; r < 4; ++r) a.d_W0[bh * D * D + feat(I, 4 * g + r) * D + feat(J, c)] = dWc[I][J][r];
#pragma unroll
  for (int J = 0; J < NT; ++J) {
    const int f = own_offset<NT>(0, J, g);
    if (c == 0) store4<F32>(a.d_b0 + bh * D + f, dbT[J]);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float sg = row16_sum(dgam[J][r]), sbt = row16_sum(dbet[J][r]);
      if (c == 0) {
        atomicAdd(a.d_gamma + h * D + f + r, sg);
        atomicAdd(a.d_beta + h * D + f + r, sbt);
      }
    }
  }
}

}  // namespace ttt
