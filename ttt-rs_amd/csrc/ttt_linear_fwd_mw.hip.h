// TTT-Linear multi-stage forward for gfx950, one workgroup of NW wavefronts per (batch, head):
// wave w owns TPW = (d/16)/NW output-feature tiles (16*TPW features).  NW = 1 needs no LDS and no
// barrier; NW = d/16 gives every wave one tile.
//
// Arithmetic as ttt_linear_fwd.hip.h (reference rust/core/src/linear.rs:91-149 looped as
// rust/core/src/inner.rs:25-50; checkpoints as
// rust/fused/src/linear_fused_tile/forward/kernel.rs:143-150).
//
// What is split and what is not:
//  * Wave w keeps the column slice W[:, own tiles] (NT*TPW accumulator tiles), its slice of
//    b, gamma, beta, and computes its 16 features of Z1, G, Zbar and of the output.  The state
//    update of that slice needs only the wave's own G tile, so W never crosses waves.
//  * Every wave loads the full XK and XQ rows (they are the k-side operands of its products)
//    and recomputes the [16 x 16] attention block; HBM sees each byte once, the repeats hit L1.
//  * LayerNorm statistics need all d features of a token.  Each wave reduces raw moments of its
//    own 16 features and the waves exchange them through LDS: ONE exchange (six sums) for the
//    LN-L2 gradient, one (two sums) for the output LayerNorm, so two barriers per mini-batch.
//    With z the pre-norm row, a = gamma^2 and q = gamma*(beta - target), the six sums
//    sum z, sum z^2, sum a z, sum a z^2, sum q, sum q z  give mean, variance and both reductions of
//    the gradient formula (reference rust/core/src/util.rs:171-179).
#pragma once
#include "ttt_linear_fwd.hip.h"

namespace ttt {

template <class T, int NT, int TPW>
struct StageInMw {
  typename Io<T>::frag q[NT], k[NT];               // full rows: k-side operands
  typename Io<T>::frag qo[TPW], ko[TPW], vo[TPW];  // this wave's features of xq, xk, xv
  float lr;
};

template <class T>
__device__ __forceinline__ typename Io<T>::frag load4(const typename Io<T>::elem* p);
template <>
__device__ __forceinline__ Io<F32>::frag load4<F32>(const float* p) {
  return *reinterpret_cast<const f32x4*>(p);
}
template <>
__device__ __forceinline__ Io<BF16>::frag load4<BF16>(const uint16_t* p) {
  return __builtin_bit_cast(bf16x4, *reinterpret_cast<const u32x2*>(p));
}
template <class T>
__device__ __forceinline__ void store4(typename Io<T>::elem* p, f32x4 v);
template <>
__device__ __forceinline__ void store4<F32>(float* p, f32x4 v) {
  *reinterpret_cast<f32x4*>(p) = v;
}
template <>
__device__ __forceinline__ void store4<BF16>(uint16_t* p, f32x4 v) {
  *reinterpret_cast<u32x2*>(p) = __builtin_bit_cast(u32x2, Io<BF16>::to_frag(v));
}

// Offset (in elements) of the features of own tile jj held by lane group g: four contiguous
// features feat(J, 4g .. 4g+3), J = w*TPW + jj.
template <int TPW>
__device__ __forceinline__ int own_offset(int w, int jj, int g) {
  const int J = w * TPW + jj;
  return 32 * (J >> 1) + 8 * g + 4 * (J & 1);
}

// Packed W checkpoint: the image of the CENTRED state (see centre_state; the backward works on the centred state
// too, so the row means are not needed again) in accumulator order, in the operand type of the I/O mode (bf16).  Tile (I, J) is the fragment a
// lane holds of it (value r of lane (c, g) is W[feat(I, 4g+r)][feat(J, c)]); the tiles (I, 2q) and (I, 2q+1)
// share the 1 KiB row I * (d/32) + q, 16 bytes per lane.  This wave writes its TPW column tiles of every I.
// f32 I/O keeps f32: tile (I, J) is the 1 KiB row I * (d/16) + J, 16 bytes per lane.
template <class T, int NT, int TPW>
__device__ __forceinline__ void store_ckpt_packed(float* slot, const f32x4 (&Wc)[NT][TPW], int w, int lane) {
  unsigned char* base = reinterpret_cast<unsigned char*>(slot) + lane * 16;
#pragma unroll
  for (int I = 0; I < NT; ++I) {
    if (sizeof(typename Io<T>::elem) == 4) {
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) *reinterpret_cast<f32x4*>(base + (I * NT + w * TPW + jj) * 1024) = Wc[I][jj];
    } else if (TPW % 2 == 0) {
#pragma unroll
      for (int qq = 0; qq < TPW / 2; ++qq) {
        const u32x2 lo = __builtin_bit_cast(u32x2, Io<BF16>::to_frag(Wc[I][2 * qq]));
        const u32x2 hi = __builtin_bit_cast(u32x2, Io<BF16>::to_frag(Wc[I][2 * qq + 1]));
        *reinterpret_cast<u32x4*>(base + (I * (NT / 2) + w * (TPW / 2) + qq) * 1024) = u32x4{lo[0], lo[1], hi[0], hi[1]};
      }
    } else {
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) {
        const int J = w * TPW + jj;
        *reinterpret_cast<u32x2*>(base + (I * (NT / 2) + (J >> 1)) * 1024 + 8 * (J & 1)) =
            __builtin_bit_cast(u32x2, Io<BF16>::to_frag(Wc[I][jj]));
      }
    }
  }
}

// Where the next checkpoint of a (batch, head) unit goes and when it is due.  A checkpoint is written before every
// ckpt_interval-th mini-batch; the slot pointers advance by one checkpoint each time and a counter says how many
// mini-batches are left until the next one, so the loop needs neither the division st / ckpt_interval nor the
// products (bh * n_ckpt + st / ckpt_interval) * d * d.
template <int D>
struct CkptCursor {
  float* W;      // next W slot (null: no checkpoints)
  float* b;      // next b slot
  int every;     // ckpt_interval
  int left;      // mini-batches until the next checkpoint (0: due now)
  bool packed;
  __device__ __forceinline__ CkptCursor(const LinearFwdArgs& a, size_t bh) {
    const bool on = a.W_ckpt != nullptr && a.ckpt_packed != kCkptFactors;
    W = on ? a.W_ckpt + bh * (size_t)a.n_ckpt * (D * D) : nullptr;
    b = on ? a.b_ckpt + bh * (size_t)a.n_ckpt * D : nullptr;
    every = on ? a.ckpt_interval : 1;
    left = 0;
    packed = a.ckpt_packed != 0;
  }
  // true when a checkpoint is due before this mini-batch; call once per mini-batch, then advance() if it was
  __device__ __forceinline__ bool due() const { return W != nullptr && left == 0; }
  __device__ __forceinline__ void advance() {
    W += D * D;
    b += D;
    left = every;
  }
  __device__ __forceinline__ void next_stage() {
    if (W != nullptr) --left;
  }
};

// ---- Update factors instead of states (ckpt_packed == kCkptFactors; bf16 I/O, two or more mini-batches) ---------
// The state changes by W += XK^T G'' and b += colsum G'' per mini-batch, with G'' rounded to the operand type and
// XK an input: the [16 x d] factor G'' (2 KiB at d = 64) says as much as the [d x d] state entering the mini-batch
// (8 KiB packed), given the state at the END of the sequence.  The backward then walks the states back:
// W_t = W_{t+1} - XK_t^T G''_t with the very operands the forward multiplied, so it recovers W_t up to the rounding
// of one f32 addition per element and mini-batch.
// Layout of a unit's share of the W checkpoint buffer (n_ckpt * d * d floats, as for the other formats):
//   bytes [0, 4 d^2)                       the centred state after the last mini-batch, f32, tile (I, J) = 1 KiB
//                                          row I * (d/16) + J, 16 bytes per lane (accumulator order)
//   bytes [4 d^2 + t * 32 d, + 32 d)       factor of mini-batch t: tile J = 512 bytes, 8 per lane: the fragment
//                                          Gd of the wave that owns feature tile J (tokens along k)
// and of the b checkpoint buffer: the centred bias after the last mini-batch (d floats).
template <int D>
__device__ __forceinline__ unsigned char* factor_base(float* W_ckpt, int n_ckpt, size_t bh) {
  return reinterpret_cast<unsigned char*>(W_ckpt + bh * (size_t)n_ckpt * (D * D)) + D * D * 4;
}
template <int TPW>
__device__ __forceinline__ void store_factor(unsigned char* slot, const bf16x4 (&Gd)[TPW], int w, int lane) {
#pragma unroll
  for (int jj = 0; jj < TPW; ++jj)
    *reinterpret_cast<u32x2*>(slot + ((w * TPW + jj) * 64 + lane) * 8) = __builtin_bit_cast(u32x2, Gd[jj]);
}
template <int D, int TPW>
__device__ __forceinline__ void store_state_tiles(float* Wd, float* bd, const f32x4 (&Wc)[D / 16][TPW],
                                                  const f32x4 (&bT)[TPW], int w, int lane) {
  constexpr int NT = D / 16;
  unsigned char* base = reinterpret_cast<unsigned char*>(Wd) + lane * 16;
#pragma unroll
  for (int I = 0; I < NT; ++I)
#pragma unroll
    for (int jj = 0; jj < TPW; ++jj) *reinterpret_cast<f32x4*>(base + (I * NT + w * TPW + jj) * 1024) = Wc[I][jj];
  if ((lane & 15) == 0) {
#pragma unroll
    for (int jj = 0; jj < TPW; ++jj) *reinterpret_cast<f32x4*>(bd + own_offset<TPW>(w, jj, lane >> 4)) = bT[jj];
  }
}

// ---- State centring -------------------------------------------------------------------------------------------
// LayerNorm does not see a shift common to all d features of a row, and the inner loop looks at the state only
// through LayerNorm: Z1 = XK W + b feeds the LN-L2 gradient, Zbar = XQ W + b - (...) G the output LayerNorm.  With
//   W = Wc + m 1^T   (m_i = mean over the columns of row i)      b = bc + mean(b) 1
// Z = X Wc + bc + (X m + mean b) 1^T, and the last term is a per-token constant that both LayerNorms discard.  The
// update W += XK^T G'' keeps the split: the rows of G'' sum to zero (G is the gradient of a function that ignores a
// common shift), and so do the columns it adds to b.  So m and mean(b) of the INITIAL state hold for the whole
// sequence, and the kernels carry Wc and bc.  Z1 and Zbar then have row means at rounding level, which is what
// makes the one-pass statistics (var = E z^2 - (E z)^2, where the reference takes two passes: var_mean_bias,
// rust/core/src/util.rs:141-150) safe for states whose rows sit far from zero, and keeps the bf16 operand images of
// W accurate whatever offset its rows carry.  No instruction is added to the loop.
//
// centre_state: centres the wave's column slice Wc[I][jj] and its bias features in place.  m0s (LDS, D + 1 floats)
// receives m at index 16 I + p for row feat(I, p), and mean(b) at index D.  Every lane subtracts the numbers it
// reads back from m0s, so a whole row is shifted by one and the same float.  xch: LDS scratch of NW * D floats.
// Ends with a workgroup barrier.
template <int D, int NW, int TPW>
__device__ __forceinline__ void centre_state(f32x4 (&Wc)[D / 16][TPW], f32x4 (&bT)[TPW], const float* b0, float* m0s,
                                             float* xch, int w, int c, int g) {
  constexpr int NT = D / 16;
#pragma unroll
  for (int I = 0; I < NT; ++I)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float p = 0.f;
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) p += Wc[I][jj][r];
      p = row16_sum_dpp(p);
      if (c == 0) xch[(I * 16 + 4 * g + r) * NW + w] = p;
    }
  __syncthreads();
  for (int i = threadIdx.x; i < D; i += 64 * NW) {
    float s = 0.f;
#pragma unroll
    for (int ww = 0; ww < NW; ++ww) s += xch[i * NW + ww];
    m0s[i] = s * (1.0f / D);
  }
  if (threadIdx.x == 0) {
    float s = 0.f;
    for (int f = 0; f < D; ++f) s += b0[f];
    m0s[D] = s * (1.0f / D);
  }
  __syncthreads();
#pragma unroll
  for (int I = 0; I < NT; ++I) {
    const f32x4 m = *reinterpret_cast<const f32x4*>(m0s + I * 16 + 4 * g);
#pragma unroll
    for (int jj = 0; jj < TPW; ++jj) Wc[I][jj] -= m;
  }
  const float bb = m0s[D];
#pragma unroll
  for (int jj = 0; jj < TPW; ++jj) bT[jj] -= bb;
  __syncthreads();
}

// The state as f32 row-major matrices from the centred registers (checkpoints): W = Wc + m 1^T, b = bc + mean(b).
template <int D, int TPW>
__device__ __forceinline__ void store_state_f32(float* Wd, float* bd, const f32x4 (&Wc)[D / 16][TPW],
                                                const f32x4 (&bT)[TPW], const float* m0s, int w, int c, int g) {
  constexpr int NT = D / 16;
#pragma unroll
  for (int I = 0; I < NT; ++I) {
    const f32x4 m = *reinterpret_cast<const f32x4*>(m0s + I * 16 + 4 * g);
#pragma unroll
    for (int jj = 0; jj < TPW; ++jj)
#pragma unroll
      for (int r = 0; r < 4; ++r) Wd[feat(I, 4 * g + r) * D + feat(w * TPW + jj, c)] = Wc[I][jj][r] + m[r];
  }
  if (c == 0) {
    const float bb = m0s[D];
#pragma unroll
    for (int jj = 0; jj < TPW; ++jj) {
      f32x4 v = bT[jj];
      v += bb;
      *reinterpret_cast<f32x4*>(bd + own_offset<TPW>(w, jj, g)) = v;
    }
  }
}

// b = bc + mean(b) alone (the packed W checkpoint keeps the centred matrix; the bias checkpoint is always the true bias).
template <int D, int TPW>
__device__ __forceinline__ void store_bias_true(float* bd, const f32x4 (&bT)[TPW], float bb, int w, int c, int g) {
  if (c == 0) {
#pragma unroll
    for (int jj = 0; jj < TPW; ++jj) {
      f32x4 v = bT[jj];
      v += bb;
      *reinterpret_cast<f32x4*>(bd + own_offset<TPW>(w, jj, g)) = v;
    }
  }
}

// The final state: initial state + (centred state now - centred state at the start).  The start value is formed
// again exactly as centre_state formed it, so a sequence that never updates the state (lr = 0, token_eta[K-1] = 0)
// returns the initial state bit for bit.
template <int D, int TPW>
__device__ __forceinline__ void store_state_final(float* Wd, float* bd, const float* W0, const float* b0,
                                                  const f32x4 (&Wc)[D / 16][TPW], const f32x4 (&bT)[TPW],
                                                  const float* m0s, int w, int c, int g) {
  constexpr int NT = D / 16;
#pragma unroll
  for (int I = 0; I < NT; ++I) {
    const f32x4 m = *reinterpret_cast<const f32x4*>(m0s + I * 16 + 4 * g);
#pragma unroll
    for (int jj = 0; jj < TPW; ++jj)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int at = feat(I, 4 * g + r) * D + feat(w * TPW + jj, c);
        const float w0 = W0[at];
        const float start = w0 - m[r];
        Wd[at] = w0 + (Wc[I][jj][r] - start);
      }
  }
  if (c == 0) {
    const float bb = m0s[D];
#pragma unroll
    for (int jj = 0; jj < TPW; ++jj) {
      const int f = own_offset<TPW>(w, jj, g);
      const f32x4 v0 = *reinterpret_cast<const f32x4*>(b0 + f);
      f32x4 start = v0;
      start -= bb;
      *reinterpret_cast<f32x4*>(bd + f) = v0 + (bT[jj] - start);
    }
  }
}

// Where one (batch, head) unit's rows start, as wave-uniform byte pointers formed once; a token's row is then a
// 32-bit byte offset from them (a unit spans at most seq_stride * d * 4 bytes), which is what the addressing of
// global loads and stores takes directly: scalar base plus 32-bit lane offset, no 64-bit arithmetic and no renewed
// fetch of the kernel arguments per mini-batch.
template <class T, int D>
struct UnitBase {
  using elem = typename Io<T>::elem;
  const unsigned char *xq, *xk, *xv, *lr, *xin;
  unsigned char* out;
  __device__ __forceinline__ UnitBase(const LinearFwdArgs& a, size_t bh) {
    const size_t row0 = bh * (size_t)a.seq_stride;
    xin = static_cast<const unsigned char*>(a.xin) + row0 * (D * sizeof(elem));
    xq = static_cast<const unsigned char*>(a.xq) + row0 * (D * sizeof(elem));
    xk = static_cast<const unsigned char*>(a.xk) + row0 * (D * sizeof(elem));
    xv = static_cast<const unsigned char*>(a.xv) + row0 * (D * sizeof(elem));
    lr = static_cast<const unsigned char*>(a.lr) + row0 * sizeof(elem);
    out = static_cast<unsigned char*>(a.out) + row0 * (D * sizeof(elem));
  }
  // byte offset of token (stage * K + c) of the unit
  static __device__ __forceinline__ unsigned row_off(int stage, int K, int c) {
    return ((unsigned)stage * (unsigned)K + (unsigned)c) * (unsigned)(D * sizeof(elem));
  }
};

template <class T, int D, int NW, bool FULL>
__device__ __forceinline__ void load_stage_mw(StageInMw<T, D / 16, D / 16 / NW>& s, const UnitBase<T, D>& ub, int K,
                                              int n_stages, int stage, int c, int g, int w) {
  using IO = Io<T>;
  using elem = typename IO::elem;
  constexpr int NT = D / 16, TPW = NT / NW;
  if (FULL) stage = min(stage, n_stages - 1);
  const bool ok = FULL || ((c < K) && (stage < n_stages));
  const unsigned off = UnitBase<T, D>::row_off(stage, K, c);
  const elem* pq = reinterpret_cast<const elem*>(ub.xq + off);
  const elem* pk = reinterpret_cast<const elem*>(ub.xk + off);
  const elem* pv = reinterpret_cast<const elem*>(ub.xv + off);
#pragma unroll
  for (int q = 0; q < NT / 2; ++q) {
    IO::load8(pq + 32 * q + 8 * g, ok, s.q[2 * q], s.q[2 * q + 1]);
    IO::load8(pk + 32 * q + 8 * g, ok, s.k[2 * q], s.k[2 * q + 1]);
  }
  if (NW == 1) {
    // the wave owns every feature: xq/xk are already there, only xv is extra
#pragma unroll
    for (int q = 0; q < NT / 2; ++q) IO::load8(pv + 32 * q + 8 * g, ok, s.vo[2 * q], s.vo[2 * q + 1]);
  } else if (TPW == 1) {
    const int off1 = own_offset<TPW>(w, 0, g);
    if (ok) {
      s.qo[0] = load4<T>(pq + off1);
      s.ko[0] = load4<T>(pk + off1);
      s.vo[0] = load4<T>(pv + off1);
    } else {
      s.qo[0] = s.ko[0] = s.vo[0] = IO::zero();
    }
  } else {
#pragma unroll
    for (int qq = 0; qq < TPW / 2; ++qq) {
      const int off2 = own_offset<TPW>(w, 2 * qq, g);  // eight contiguous features: tiles 2qq, 2qq+1
      IO::load8(pq + off2, ok, s.qo[2 * qq], s.qo[2 * qq + 1]);
      IO::load8(pk + off2, ok, s.ko[2 * qq], s.ko[2 * qq + 1]);
      IO::load8(pv + off2, ok, s.vo[2 * qq], s.vo[2 * qq + 1]);
    }
  }
  const unsigned tok = (unsigned)stage * (unsigned)K + (unsigned)c;
  s.lr = ok ? IO::load1(reinterpret_cast<const elem*>(ub.lr + tok * (unsigned)sizeof(elem))) : 0.f;
}

// Sum over the four lane groups.  MF: one f32 MFMA against a ones operand (keeps the VALU free);
// otherwise the lane-swap reduction.
template <bool MF>
__device__ __forceinline__ float xg_reduce(float v) {
  if (MF) {
    f32x4 z = {0.f, 0.f, 0.f, 0.f};
    z = __builtin_amdgcn_mfma_f32_16x16x4f32(1.0f, v, z, 0, 0, 0);
    return z[0];
  }
  return xg_sum(v);
}

template <class T, int D, int NW, int PF, bool FULL, bool FAC = false>
__global__ void __launch_bounds__(64 * NW) ttt_linear_fwd_mw_kernel(Problems<LinearFwdArgs> problems) {
  const LinearFwdArgs& a = problems.p[blockIdx.y];
  using IO = Io<T>;
  using frag = typename IO::frag;
  using elem = typename IO::elem;
  constexpr int NT = D / 16, TPW = NT / NW;
  constexpr bool BF = sizeof(elem) == 2;  // bf16 storage: MFMA pipe has room for helper products
  constexpr float inv_d = 1.0f / D;
  __shared__ float ex1[6 * 16 * NW];
  __shared__ float ex2[2 * 16 * NW];

  const int lane = threadIdx.x & 63, w = (threadIdx.x >> 6) % NW;
  const int c = lane & 15, g = lane >> 4;
  const size_t bh = blockIdx.x;
  const int h = (int)(bh % a.H);
  const int K = a.K;

  // eta_last = token_eta[K-1] * lr is folded into G itself: G'' = -sc * lr * G with
  // sc = token_eta[K-1], so the state update is W += XK^T G'' with no further scaling and the
  // causal matrix becomes (token_eta[t] / sc) (1 + A[t][s]).  sc == 0 (no state update at all)
  // falls back to sc = 1 and skips the update.
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
  // Wc[I][jj][r] = W[feat(I,4g+r)][feat(w*TPW+jj, c)]
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
  // the kernel carries the centred state (see centre_state)
  __shared__ __attribute__((aligned(16))) float m0s[D + 4];
  __shared__ float cxch[NW * D];
  centre_state<D, NW, TPW>(Wc, bT, a.b0 + sb * D, m0s, cxch, w, c, g);

  // Ring of R = PF+1 register sets, loop unrolled by R: step u consumes set u and refills the set
  // that step u-1 consumed, so every set has fixed registers and a load is never copied (a copy
  // at the loop back-edge would have to wait for the load, i.e. undo the prefetch).
  constexpr int R = PF + 1;
  StageInMw<T, NT, TPW> buf[R];
  const UnitBase<T, D> ub(a, bh);
  const int K_ = a.K, n_stages_ = a.n_stages;
#pragma unroll
  for (int u = 0; u < PF; ++u) load_stage_mw<T, D, NW, FULL>(buf[u], ub, K_, n_stages_, u, c, g, w);
  CkptCursor<D> ck(a, bh);
  const float b_mean = __builtin_amdgcn_readfirstlane(m0s[D]);  // mean of the initial bias (split off by centre_state)
  static_assert(!FAC || BF, "update factors are saved with bf16 I/O only");
  unsigned char* fac = FAC ? factor_base<D>(a.W_ckpt, a.n_ckpt, bh) : nullptr;

  for (int st0 = 0; st0 < a.n_stages; st0 += R) {
#pragma unroll
    for (int u = 0; u < R; ++u) {
      const int st = st0 + u;
      load_stage_mw<T, D, NW, FULL>(buf[(u + PF) % R], ub, K_, n_stages_, st + PF, c, g, w);
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
      // ---- raw moments of this wave's features
      f32x4 bq[TPW];
      float S[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int jj = 0; jj < TPW; ++jj) {
        const frag ko = (NW == 1) ? cur.k[jj] : cur.ko[jj];
        f32x4 uu;  // beta - (xv - xk)
        if (BF) {
          uu = bet[jj];
          IO::mma2(uu, nident, ident, cur.vo[jj], ko);
        } else {
          uu = bet[jj] - (IO::to_f32(cur.vo[jj]) - IO::to_f32(ko));
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
#pragma unroll
      for (int i = 0; i < 6; ++i) S[i] = xg_reduce<BF>(S[i]);
      if (NW > 1) {
        // lane group g publishes sums g and g+4; every lane then adds up the waves
        float v0 = S[0], v1 = S[4];
        if (g == 1) { v0 = S[1]; v1 = S[5]; }
        if (g == 2) v0 = S[2];
        if (g == 3) v0 = S[3];
        ex1[(g * 16 + c) * NW + w] = v0;
        if (g < 2) ex1[((g + 4) * 16 + c) * NW + w] = v1;
        lds_barrier();
#pragma unroll
        for (int i = 0; i < 6; ++i) {
          float s = 0.f;
#pragma unroll
          for (int ww = 0; ww < NW; ++ww) s += ex1[(i * 16 + c) * NW + ww];
          S[i] = s;
        }
      }
      f32x4 G[TPW];
      {
        const float mu = S[0] * inv_d;
        const float var = S[1] * inv_d - mu * mu;
        const float rstd = __builtin_amdgcn_rsqf(fmaxf(var, 0.f) + a.eps);
        const float s1 = rstd * (S[2] - mu * sum_a) + S[4];
        const float s2 = rstd * rstd * (S[3] - 2.f * mu * S[2] + mu * mu * sum_a) + rstd * (S[5] - mu * S[4]);
        // G'' = p (gx - s1/d - xh s2/d), gx = a2 xh + bq, xh = (z - mu) rstd, p = -sc lr rstd
        //     = (z - mu) (c1 a2 + c2) + (p bq + c3)
        const float p = -sc * cur.lr * rstd;
        const float c1 = p * rstd, c2 = -c1 * s2 * inv_d, c3 = -p * s1 * inv_d;
#pragma unroll
        for (int jj = 0; jj < TPW; ++jj) G[jj] = (z1[jj] - mu) * (a2[jj] * c1 + c2) + (bq[jj] * p + c3);
      }
      // ---- G'' with tokens along k; causal correction Zbar^T += G''^T M''^T
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
      // ---- output LayerNorm
      {
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int jj = 0; jj < TPW; ++jj)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            s0 += zb[jj][r];
            s1 += zb[jj][r] * zb[jj][r];
          }
        s0 = xg_reduce<BF>(s0);
        s1 = xg_reduce<BF>(s1);
        if (NW > 1) {
          if (g < 2) ex2[(g * 16 + c) * NW + w] = (g == 0) ? s0 : s1;
          lds_barrier();
          s0 = s1 = 0.f;
#pragma unroll
          for (int ww = 0; ww < NW; ++ww) {
            s0 += ex2[c * NW + ww];
            s1 += ex2[(16 + c) * NW + ww];
          }
        }
        const float mu = s0 * inv_d;
        const float rstd = __builtin_amdgcn_rsqf(fmaxf(s1 * inv_d - mu * mu, 0.f) + a.eps);
        if (FULL || c < K) {
          elem* po = reinterpret_cast<elem*>(ub.out + UnitBase<T, D>::row_off(st, K, c));
          f32x4 o[TPW];
#pragma unroll
          for (int jj = 0; jj < TPW; ++jj) {
            const frag qo = (NW == 1) ? cur.q[jj] : cur.qo[jj];
            f32x4 qb;  // xq + beta
            if (BF) {
              qb = bet[jj];
              IO::mma(qb, ident, qo);
            } else {
              qb = IO::to_f32(qo) + bet[jj];
            }
            o[jj] = qb + gam[jj] * ((zb[jj] - mu) * rstd);
          }
          if (TPW == 1) {
            store4<T>(po + own_offset<TPW>(w, 0, g), o[0]);
          } else {
#pragma unroll
            for (int qq = 0; qq < TPW / 2; ++qq)
              IO::store8(po + own_offset<TPW>(w, 2 * qq, g), o[2 * qq], o[2 * qq + 1]);
          }
        }
      }
      // ---- state update of this wave's column slice (linear.rs:134-144): W += XK^T G'', b += colsum G''
      if (upd) {
#pragma unroll
        for (int I = 0; I < NT; ++I) {
          f32x4 t = {0.f, 0.f, 0.f, 0.f};
          IO::mma(t, cur.k[I], ident);  // t[r] = XK[s = 4g+r][feat(I,c)]
          const frag kd = IO::to_frag(t);
#pragma unroll
          for (int jj = 0; jj < TPW; ++jj) IO::mma(Wc[I][jj], kd, Gd[jj]);
        }
#pragma unroll
        for (int jj = 0; jj < TPW; ++jj) IO::mma(bT[jj], Gd[jj], ones);
      }
    }
  }

  store_state_final<D, TPW>(a.W_out + bh * D * D, a.b_out + bh * D, a.W0 + sb * D * D, a.b0 + sb * D, Wc, bT, m0s, w, c, g);
  if constexpr (FAC)
    store_state_tiles<D, TPW>(a.W_ckpt + bh * (size_t)a.n_ckpt * (D * D), a.b_ckpt + bh * (size_t)a.n_ckpt * D, Wc, bT, w, lane);
}

}  // namespace ttt
