// TTT-MLP multi-stage forward for head_dim 128 (and 96) on gfx950: the register-resident kernel of
// ttt_mlp_fwd_rr.hip.h spread over a PAIR of workgroups (two CUs) per (batch, head).
//
// Arithmetic: reference rust/core/src/mlp.rs:127-208 looped as rust/core/src/inner.rs:25-50.
//
// At d = 128 the f32 state (W1 [128,512], W2 [512,128]: 512 KiB) equals the whole register file of
// one CU, so the hidden axis is cut in two: workgroup `cu` of a pair owns hidden units
// [2d cu, 2d cu + 2d), i.e. W1[:, half], W2[half, :], b1[half] (128 VGPRs of state per lane), and
// runs the register-resident scheme on its half.  A workgroup has d/16 waves: one per d-feature tile
// (reducer and output roles) and two hidden tiles each.  At d = 96 (six waves, 96 VGPRs of state) the
// state fits one CU and the pair is an option for launches with at most half as many units as CUs.
// What crosses the pair, once per mini-batch:
//   X1  (recurrence)  each CU's locally reduced Z2^T tiles [d x 16]: both CUs add the two halves
//       (always in the order cu 0 + cu 1, so both hold bit-identical Z2, G2, b2);
//   X2  (output path) CU 1's locally reduced Zbar2^T tiles and A2 tile go to CU 0, which finishes
//       and stores the output.
// The exchange runs through global memory without fences or separate flags: every f32 travels in a
// 64-bit word together with a tag (mini-batch index + 1), written and polled with relaxed agent-scope
// atomics, so a word is either old or complete and the caches are never flushed or invalidated (an
// agent-scope release / acquire pair per mini-batch cost about 30 us here).  Lane l of wave I only
// ever waits for lane l of wave I of the other CU.  There is no workspace argument in ttt_mlp_fwd, so
// the exchange area is the unit's W2_out buffer, which is not needed until the final state is stored:
// everything a CU polls lies in the rows of W2_out that this CU itself overwrites at the end, so its
// final store is ordered after its last read by program order, and the partner never writes there
// again after its last mini-batch.  The host zeroes W2_out (tag 0 = nothing sent) before the launch.
// Pairs are blocks (i, i + 8): with workgroups dealt round-robin to the eight XCDs both land on the
// same XCD (shared L2), and the exchange then never leaves that L2 (workgroup-scope stores, see send_tagged).
// That placement is checked, not assumed: at start the two workgroups tell each other which XCD they run on
// (device-scope words), and a pair that sits on two XCDs stores at device scope for the whole launch -- slower,
// same results.  Every wait is bounded, so a missing partner ends in NaN outputs, never in a hang.
#pragma once
#include "ttt_mlp_fwd_rr.hip.h"

namespace ttt {

template <int D, int ES>
struct MlpCl2Lds {
  static constexpr int NW = D / 16, NT = D / 16, FH = 2 * D;  // FH: hidden units of one CU; one wave per d-feature tile
  static constexpr int TILE = 16 * D * ES;
  static constexpr int IN1 = 3 * TILE;
  static constexpr int IN = 0;                  // [2 buffers][3][16][d]
  static constexpr int LR = IN + 2 * IN1;       // [2][16] floats
  static constexpr int P1 = LR + 2 * 64 + 128;  // [NW][NT][64] f32x4: partial Z2^T tiles
  static constexpr int P2 = P1 + NW * NT * 1024;  // [NW][NT][64] bf16x4: partial Zbar2^T tiles
  static constexpr int PA = P2 + NW * NT * 512;   // [NW][64] f32x4: partial A2^T
  static constexpr int EX = PA + NW * 1024;       // [8 sums][2][16 tokens] f32x4
  static constexpr int GT = EX + 8 * 2 * 16 * 16;
  static constexpr int GD = GT + NT * 64 * 4 * ES;
  static constexpr int KD = GD + NT * 64 * 4 * ES;  // [2][NT][64] frag
  static constexpr int PRM = KD + 2 * NT * 64 * 4 * ES;  // gamma[d], beta[d], b1[FH] floats
  static constexpr int EXO = PRM + (2 * D + FH) * 4;
  static constexpr int LOST = EXO + 2 * 2 * 16 * 16;  // one word: a wait for the partner ran out
  static constexpr int BYTES = LOST + 16;
  static_assert(BYTES <= 160 * 1024, "exceeds the 160 KiB of LDS of a gfx950 CU");
  static_assert(NT == NW && NW <= 8 && D % 32 == 0 && ES == 2, "one reducer and one output tile per wave, bf16 I/O");
  static_assert(FH % (16 * NW) == 0, "whole hidden tiles per wave");
  static_assert(TILE % 1024 == 0 && P1 % 16 == 0, "input tiles are staged in 1 KiB wave blocks");
  // exchange area inside this CU's rows of W2_out (bytes): two parities of X1 tiles, X2 tiles, A2 tile,
  // each tile as 64 lanes x 4 tagged 64-bit words
  static constexpr int XTILE = 2048, XSLOT = (2 * NT + 1) * XTILE;
  static constexpr int XHELLO = 2 * XSLOT;  // one tagged word behind the tiles: the partner's XCD
  static_assert(XHELLO + 16 <= FH * D * 4, "exchange area exceeds this CU's rows of W2_out");
};

// One [16 x 16] f32 tile (this lane's four values) as four (value, tag) words.
// The two workgroups of a pair sit on CUs of one XCD (see the block numbering in the kernel), which share an L2.
// The stores therefore carry workgroup scope: they leave the CU (its L1 writes through) and stay in that L2, where
// the partner's device-scope loads, which bypass its own L1, find them.  Device-scope stores would also be written
// through to memory, every one of them: measured at 2.8 GB of writes per launch of 128 units x 2048 tokens, which
// made the kernel 40 % slower on a full GPU than on a quarter of it.  `same_xcd` is what the two workgroups found
// out about each other at start (see the kernel): a pair on two XCDs stores at device scope.
__device__ __forceinline__ void send_tagged(unsigned long long* slot, f32x4 v, unsigned tag, bool same_xcd) {
  if (same_xcd) {
#pragma unroll
    for (int r = 0; r < 4; ++r)
      __hip_atomic_store(slot + r, ((unsigned long long)tag << 32) | __float_as_uint(v[r]), __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_WORKGROUP);
  } else {
#pragma unroll
    for (int r = 0; r < 4; ++r)
      __hip_atomic_store(slot + r, ((unsigned long long)tag << 32) | __float_as_uint(v[r]), __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
  }
}
// Receives N tiles at once: polls until the four words of every slot carry that slot's tag, all
// loads of a round in flight together (one memory round trip per round, not one per tile).  The wait
// is bounded; after one wait has run out (`alive` cleared) no further wait is attempted: a lost
// partner costs one time-out per wave, not one per mini-batch, and ends in NaNs in b1_out, never in a hang.
template <int N>
__device__ __forceinline__ void recv_tagged(const unsigned long long* const (&slot)[N], const unsigned (&tag)[N],
                                            f32x4 (&out)[N], bool& alive, int spin_limit) {
  unsigned long long wd[N][4];
  int it = 0;
  // light first stage: one lane watches the word stored last of the first slot, so that sixteen
  // waiting waves do not flood the memory system with polls; the full check then usually passes at once
  if (alive && (threadIdx.x & 63) == 0) {
    const unsigned long long* last = slot[0] + 4 * 63 + 3;  // lane 63's fourth word (slot[] is lane 0's here)
    while ((unsigned)(__hip_atomic_load(last, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >> 32) != tag[0]) {
      if (++it >= spin_limit) break;
      __builtin_amdgcn_s_sleep(1);
    }
  }
  it = 0;
  while (true) {
    bool ok = true;
#pragma unroll
    for (int n = 0; n < N; ++n)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        wd[n][r] = __hip_atomic_load(slot[n] + r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int n = 0; n < N; ++n)
#pragma unroll
      for (int r = 0; r < 4; ++r) ok = ok && (unsigned)(wd[n][r] >> 32) == tag[n];
    // the whole wave leaves together: its lanes poll neighbouring words of the same tiles
    if (__all(ok) || !alive) break;
    if (++it >= spin_limit) {
      alive = false;
      break;
    }
    __builtin_amdgcn_s_sleep(1);
  }
#pragma unroll
  for (int n = 0; n < N; ++n)
    out[n] = f32x4{__uint_as_float((unsigned)wd[n][0]), __uint_as_float((unsigned)wd[n][1]),
                   __uint_as_float((unsigned)wd[n][2]), __uint_as_float((unsigned)wd[n][3])};
}

#define RELANE() asm volatile("" : "+v"(lane))

template <class T, int D>
__global__ void __launch_bounds__(64 * (D / 16)) ttt_mlp_fwd_cl2_kernel(Problems<MlpFwdArgs> problems) {
  const MlpFwdArgs& a = problems.p[blockIdx.y];
  using IO = Io<T>;
  using frag = typename IO::frag;
  using elem = typename IO::elem;
  constexpr int ES = sizeof(elem);
  using L = MlpCl2Lds<D, ES>;
  constexpr int NW = L::NW, NT = D / 16, F = 4 * D, FH = L::FH, HT = FH / 16 / NW, NTHR = 64 * NW;
  constexpr float inv_d = 1.0f / D;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6);
  int lane = tid & 63;
  const int c = lane & 15, g = lane >> 4;
  // blocks (i, i + 8) of every group of sixteen form a pair
  const int blk = blockIdx.x;
  const int cu = (blk >> 3) & 1;
  const size_t bh = (size_t)a.unit_base + (size_t)(blk >> 4) * 8 + (blk & 7);
  if (bh >= (size_t)a.B * a.H) return;
  int& lost = *reinterpret_cast<int*>(smem + L::LOST);  // set by a wave whose wait for the partner ran out
  if (tid == 0) lost = 0;
  const int h = (int)(bh % a.H), K = a.K;
  const int hoff = cu * FH;  // first hidden unit of this CU

  f32x4* const P1 = reinterpret_cast<f32x4*>(smem + L::P1);
  frag* const P2 = reinterpret_cast<frag*>(smem + L::P2);
  f32x4* const PA = reinterpret_cast<f32x4*>(smem + L::PA);
  float* const EX = reinterpret_cast<float*>(smem + L::EX);
  float* const EXO = reinterpret_cast<float*>(smem + L::EXO);
  frag* const GT = reinterpret_cast<frag*>(smem + L::GT);
  frag* const GD = reinterpret_cast<frag*>(smem + L::GD);
  frag* const KD = reinterpret_cast<frag*>(smem + L::KD);
  uint32_t* const LRs = reinterpret_cast<uint32_t*>(smem + L::LR);
  float* const GAM = reinterpret_cast<float*>(smem + L::PRM);
  float* const BET = GAM + D;
  float* const B1s = BET + D;  // this CU's half of b1

  // exchange areas: what this CU receives lies in its own rows of W2_out, what it sends in the partner's
  unsigned char* const xin = reinterpret_cast<unsigned char*>(a.W2 + (bh * F + hoff) * (size_t)D);
  unsigned char* const xout = reinterpret_cast<unsigned char*>(a.W2 + (bh * F + (FH - hoff)) * (size_t)D);

  // ---- which XCD does the partner run on?  One device-scope word each way (tag 0xffffffff: no mini-batch uses it),
  // sent before the state is loaded and read after, so the round trip costs nothing.  The answer decides the scope
  // of every later store to the partner.
  unsigned my_xcc;
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(my_xcc));
  my_xcc &= 15u;
  if (tid == 0)
    __hip_atomic_store(reinterpret_cast<unsigned long long*>(xout + L::XHELLO), (0xffffffffull << 32) | my_xcc, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);

  const float te_last = a.token_eta[K - 1];
  const bool upd = te_last != 0.f;
  const float sc = upd ? te_last : 1.f;
  const float rho_c = (c < K) ? a.token_eta[c] / sc : 0.f;
  const frag ident = identity_frag<T>(c, g);
  const frag ones = splat_frag<T>(1.f);
  const size_t sb = a.state_per_batch ? bh : (size_t)h;
  const int own = own_offset<1>(w, 0, g);  // first of this lane's four features of d-feature tile w

  // ---- state and parameters
  f32x4 W1c[NT][HT], W2c[HT][NT];
  {
    const float* W1 = a.W1_0 + sb * (size_t)D * F;
    const float* W2 = a.W2_0 + sb * (size_t)D * F;
#pragma unroll
    for (int j = 0; j < HT; ++j) {
      const int hb = hoff + 16 * (w * HT + j);
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
  // the second layer is carried centred (see row_means16 in ttt_mlp_fwd_rr.hip.h)
#pragma unroll
  for (int j = 0; j < HT; ++j) {
    const f32x4 m = row_means16<NT>(W2c[j], inv_d);
#pragma unroll
    for (int I = 0; I < NT; ++I) W2c[j][I] -= m;
  }
  b2T -= mean_of(a.b2_0 + sb * D, D, inv_d);
  for (int f = 0; f < D; ++f) sum_a += a.gamma[h * D + f] * a.gamma[h * D + f];
  for (int i = tid; i < D; i += NTHR) {
    GAM[i] = a.gamma[h * D + i];
    BET[i] = a.beta[h * D + i];
  }
  for (int i = tid; i < FH; i += NTHR) B1s[i] = a.b1_0[sb * F + hoff + i];

  // ---- staging of the xq / xk / xv rows: global -> LDS, two buffers.  The fetch of mini-batch st+1 is
  // issued after the first barrier of mini-batch st (every wave has then finished reading the buffer it
  // overwrites) and has landed before the third.
  constexpr int NBLK = L::IN1 / 1024, NBI = (NBLK + NW - 1) / NW;
  int goff[NBI];
#pragma unroll
  for (int it = 0; it < NBI; ++it) {
    const int rem = (1024 * (w + NW * it) + 16 * lane) % L::TILE, tok = rem / (D * ES);
    goff[it] = (tok < K) ? rem : -1;
  }
  auto fetch = [&](int stage) {
    if (stage >= a.n_stages) return;
    unsigned char* dst = smem + L::IN + (stage & 1) * L::IN1;
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
               (unsigned)(size_t)(__attribute__((address_space(3))) uint32_t*)(LRs + (stage & 1) * 16));
  };
  auto row = [&](int buf, int ten) -> const elem* {
    return reinterpret_cast<const elem*>(smem + L::IN + buf * L::IN1 + ten * L::TILE) + c * D;
  };

  for (int i = tid; i < (L::P1 - L::IN) / 4; i += NTHR) reinterpret_cast<float*>(smem)[i] = 0.f;
  for (int i = tid; i < 8 * 2 * 16 * 4; i += NTHR) EX[i] = 0.f;
  if (tid < 2 * 2 * 16 * 4) EXO[tid] = 0.f;
  int& partner_xcc = *reinterpret_cast<int*>(smem + L::LOST + 4);  // -1: the partner never said
  if (tid == 0) {
    const unsigned long long* hello = reinterpret_cast<const unsigned long long*>(xin + L::XHELLO);
    unsigned long long wd = 0;
    int it = 0;
    while ((unsigned)((wd = __hip_atomic_load(hello, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) >> 32) != 0xffffffffu) {
      if (++it >= a.spin_limit) break;
      __builtin_amdgcn_s_sleep(1);
    }
    partner_xcc = (unsigned)(wd >> 32) == 0xffffffffu ? (int)(wd & 15u) : -1;
  }
  __syncthreads();
  // a partner that never said where it runs is treated like one on another XCD; the first wait for it will run out
  const bool same_xcd = !a.assume_other_xcd && __builtin_amdgcn_readfirstlane(partner_xcc) == (int)my_xcc;
  fetch(0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  auto publish = [&](const float (&S)[6]) {
    const float v0 = xg_sum4_scatter(S[0], S[1], S[2], S[3]);
    const float v1 = xg_sum4_scatter(S[4], S[5], 0.f, 0.f);
    EX[(((g)*2 + (w >> 2)) * 16 + c) * 4 + (w & 3)] = v0;
    if (g < 2) EX[(((g + 4) * 2 + (w >> 2)) * 16 + c) * 4 + (w & 3)] = v1;
  };
  auto collect = [&](const float* ex, int i) -> float {
    const f32x4 lo = *reinterpret_cast<const f32x4*>(ex + ((i * 2 + 0) * 16 + c) * 4);
    const f32x4 hi = *reinterpret_cast<const f32x4*>(ex + ((i * 2 + 1) * 16 + c) * 4);
    return ((lo[0] + lo[1]) + (lo[2] + lo[3])) + ((hi[0] + hi[1]) + (hi[2] + hi[3]));
  };
  // tile slot `idx` of parity `par`: X1 tiles 0..NT-1, X2 tiles NT..2NT-1, the A2 tile 2NT
  bool alive = a.spin_limit > 0;
  auto send_tile = [&](int par_, int idx, f32x4 v, unsigned tag) {
    send_tagged(reinterpret_cast<unsigned long long*>(xout + par_ * L::XSLOT + idx * L::XTILE) + 4 * lane, v, tag, same_xcd);
  };
  auto slot_in = [&](int par_, int idx) -> const unsigned long long* {
    return reinterpret_cast<const unsigned long long*>(xin + par_ * L::XSLOT + idx * L::XTILE) + 4 * lane;
  };

  // ---- output path (previous mini-batch), wave w owns d-feature tile w.  CU 1 reduces its half and
  // sends it; CU 0 adds both halves, applies the causal correction and finishes the LayerNorm.
  f32x4 zb = {0.f, 0.f, 0.f, 0.f};
  frag qo_pend = IO::zero();  // xq tile of the mini-batch whose output is pending
  f32x4 at2 = {0.f, 0.f, 0.f, 0.f};
  // local half of the pending output: this CU's split-k sums; CU 1 sends them off at once
  auto output_local = [&](int st_out) {  // st_out: the mini-batch the output belongs to
    at2 = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ww = 0; ww < NW; ++ww) at2 += PA[ww * 64 + lane];
    pin(at2);
    zb = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ww = 0; ww < NW; ++ww) zb += IO::to_f32(P2[(ww * NT + w) * 64 + lane]);
    pin(zb);
    if (cu == 1) {
      send_tile(st_out & 1, NT + w, zb, (unsigned)st_out + 1);
      if (w == 0) send_tile(st_out & 1, 2 * NT, at2, (unsigned)st_out + 1);
    }
  };
  // CU 0: add CU 1's half, causal correction, row moments
  auto output_finish = [&](f32x4 zb_part, f32x4 at_part) {
    if (cu == 1) return;
    zb += zb_part;
    at2 += at_part;
    f32x4 m;
#pragma unroll
    for (int r = 0; r < 4; ++r) m[r] = (4 * g + r <= c) ? rho_c * (1.f + at2[r]) : 0.f;
    IO::mma(zb, GD[w * 64 + lane], IO::to_frag(m));  // GD still holds the previous mini-batch's G2
    float s0 = 0.f, s1 = 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      s0 += zb[r];
      s1 += zb[r] * zb[r];
    }
    s0 = xg_sum(s0);
    s1 = xg_sum(s1);
    if (g == 0) {
      EXO[((0 * 2 + (w >> 2)) * 16 + c) * 4 + (w & 3)] = s0;
      EXO[((1 * 2 + (w >> 2)) * 16 + c) * 4 + (w & 3)] = s1;
    }
  };
  auto output_emit = [&](int stage) {
    if (cu == 1) return;
    const float mu = collect(EXO, 0) * inv_d;
    const float rstd = __builtin_amdgcn_rsqf(fmaxf(collect(EXO, 1) * inv_d - mu * mu, 0.f) + a.eps);
    if (c < K) {
      const f32x4 gam = *reinterpret_cast<const f32x4*>(GAM + own), bet = *reinterpret_cast<const f32x4*>(BET + own);
      elem* po = static_cast<elem*>(a.out) + (bh * (size_t)a.seq_stride + (size_t)stage * K + c) * D + own;
      store4<T>(po, IO::to_f32(qo_pend) + bet + gam * ((zb - mu) * rstd));
    }
  };

  for (int st = 0; st < a.n_stages; ++st) {
    const int buf = st & 1, par = st & 1;
    RELANE();

    // ================= phase A: everything that needs only W1, W2 and the inputs
    f32x4 z1[HT];
    {
      f32x4 t = {0.f, 0.f, 0.f, 0.f};
      IO::mma(t, load4<T>(row(buf, 1) + own), ident);
      KD[(par * NT + w) * 64 + lane] = IO::to_frag(t);
    }
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
      asm volatile("" : "+v"(x2f[j]), "+v"(dg[j]));
      __builtin_amdgcn_sched_barrier(0);
    }
    // partial Z2^T over this wave's hidden units (HT is even here)
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

    // ================= phase B: this CU's half of Z2 tile w, exchange with the partner, row moments;
    //                          then the output path of the previous mini-batch
    f32x4 z, bq, zq[HT];
    frag Mf;
    {
      f32x4 zloc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ww = 0; ww < NW; ++ww) {
        zloc += P1[(ww * NT + w) * 64 + lane];
        if ((ww & 3) == 3) pin(zloc);
      }
      send_tile(par, w, zloc, (unsigned)st + 1);
      // everything that does not need the partner goes between the send and the wait
      if (st > 0) output_local(st - 1);
      // (XQ W1 + b1)^T for this wave's hidden units and the causal matrix M1: independent of the partner
#pragma unroll
      for (int j = 0; j < HT; ++j)
#pragma unroll
        for (int I = 0; I < NT; ++I) forget(W1c[I][j]);
#pragma unroll
      for (int j = 0; j < HT; ++j) zq[j] = *reinterpret_cast<const f32x4*>(B1s + 16 * (w * HT + j) + 4 * g);
      {
        f32x4 At = {0.f, 0.f, 0.f, 0.f};
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
        f32x4 m;
#pragma unroll
        for (int r = 0; r < 4; ++r) m[r] = (4 * g + r <= c) ? rho_c * (1.f + At[r]) : 0.f;
        Mf = IO::to_frag(m);
      }
      const frag ko = load4<T>(row(buf, 1) + own), vo = load4<T>(row(buf, 2) + own);
      const f32x4 gam = *reinterpret_cast<const f32x4*>(GAM + own), bet = *reinterpret_cast<const f32x4*>(BET + own);
      bq = gam * (bet - (IO::to_f32(vo) - IO::to_f32(ko)));
      // one wait for everything the partner sends this mini-batch: its half of Z2 tile w and (to CU 0)
      // its half of the pending output
      f32x4 zpart, zb_part = {0.f, 0.f, 0.f, 0.f}, at_part = zb_part;
      if (cu == 0 && st > 0) {
        const unsigned long long* const sl[3] = {slot_in(par, w), slot_in(par ^ 1, NT + w), slot_in(par ^ 1, 2 * NT)};
        const unsigned tg[3] = {(unsigned)st + 1, (unsigned)st, (unsigned)st};
        f32x4 rv[3];
        recv_tagged<3>(sl, tg, rv, alive, a.spin_limit);
        zpart = rv[0];
        zb_part = rv[1];
        at_part = rv[2];
      } else {
        const unsigned long long* const sl[1] = {slot_in(par, w)};
        const unsigned tg[1] = {(unsigned)st + 1};
        f32x4 rv[1];
        recv_tagged<1>(sl, tg, rv, alive, a.spin_limit);
        zpart = rv[0];
      }
      fetch(st + 1);
      z = b2T + (cu == 0 ? zloc + zpart : zpart + zloc);  // same order of the halves on both CUs
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
      if (st > 0) output_finish(zb_part, at_part);
    }
    lds_barrier();  // ---- B2
    RELANE();

    // ================= phase C: G2'' in both orientations; CU 0 stores the previous output
    {
      float S[6];
#pragma unroll
      for (int i = 0; i < 6; ++i) S[i] = collect(EX, i);
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
    }
    if (st > 0) output_emit(st - 1);
    qo_pend = load4<T>(row(buf, 0) + own);
    // the next mini-batch's rows must have landed; CU 0's output store, the only memory operation younger
    // than the copies (which retire in order), may stay in flight
    if (cu == 0 && st > 0)
      asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
    else
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    lds_barrier();  // ---- B3
    RELANE();

    // ================= phase D: G1, Zbar1, Xbar2, split-k partials of the output path, updates
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
      IO::mma(t, IO::to_frag(acc * dg[j]), ident);
      G1d[j] = IO::to_frag(t);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int j = 0; j < HT; ++j) IO::mma(zq[j], G1d[j], Mf);
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
      // b2 enters the sum once: through wave I of CU 0
      f32x4 p = (I == w && cu == 0) ? b2T : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j + 1 < HT; j += 2)
        IO::mma2(p, IO::to_frag(W2c[j][I]), IO::to_frag(W2c[j + 1][I]), xbf[j], xbf[j + 1]);
      if (HT & 1) IO::mma2(p, IO::to_frag(W2c[HT - 1][I]), IO::zero(), xbf[HT - 1], IO::zero());
      P2[(w * NT + I) * 64 + lane] = IO::to_frag(p);
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
      IO::mma(b2T, GD[w * 64 + lane], ones);
    }
  }

  // ---- the last mini-batch's output
  lds_barrier();
  output_local(a.n_stages - 1);
  if (cu == 0) {
    const int lp = (a.n_stages - 1) & 1;
    const unsigned long long* const sl[2] = {slot_in(lp, NT + w), slot_in(lp, 2 * NT)};
    const unsigned tg[2] = {(unsigned)a.n_stages, (unsigned)a.n_stages};
    f32x4 rv[2];
    recv_tagged<2>(sl, tg, rv, alive, a.spin_limit);
    output_finish(rv[0], rv[1]);
  }
  lds_barrier();
  output_emit(a.n_stages - 1);

  // ---- final state: this CU's hidden half.  Its rows of W2_out held the exchange area; every read of
  // it by this workgroup is above, every write of the partner into it was awaited above.
  if (!alive) lost = 1;
  __syncthreads();
  // A wait for the partner that ran out (the two workgroups of a pair were not resident together long enough)
  // must not pass for a result: the workgroup that saw it turns everything it owns of the unit into NaN -- its
  // half of W1, b1, W2, b2 and the whole output of the unit (both workgroups do, as a rule: the partner then finds
  // NaN tags where it polls and times out too).  The caller sees NaN in every output tensor of that unit.
  const float poison = lost ? __builtin_nanf("") : 0.f;
  {
    float* W1 = a.W1 + bh * (size_t)D * F;
    float* W2 = a.W2 + bh * (size_t)D * F;
    const float* W2i = a.W2_0 + sb * (size_t)D * F;
#pragma unroll
    for (int j = 0; j < HT; ++j) {
      const int hb = hoff + 16 * (w * HT + j);
      // second layer: initial value + (centred value now - centred value at the start); see ttt_mlp_fwd_rr.hip.h
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
          W1[(size_t)feat(I, 4 * g + r) * F + hb + c] = W1c[I][j][r] + poison;
          W2[(size_t)(hb + 4 * g + r) * D + feat(I, c)] = fin[r] + poison;
        }
      }
      if (c == 0)
        store4<F32>(a.b1 + bh * F + hb + 4 * g, *reinterpret_cast<const f32x4*>(B1s + 16 * (w * HT + j) + 4 * g) + poison);
    }
    {
      const float bb = mean_of(a.b2_0 + sb * D, D, inv_d);
      const f32x4 v0 = *reinterpret_cast<const f32x4*>(a.b2_0 + sb * D + own);
      const f32x4 start = v0 - bb;
      if ((cu == 0 || lost) && c == 0) store4<F32>(a.b2 + bh * D + own, v0 + (b2T - start) + poison);
    }
    if (lost) {
      if (tid == 0) atomicAdd(&g_mlp_fwd_lost_workgroups, 1u);
      elem* po = static_cast<elem*>(a.out) + bh * (size_t)a.seq_stride * D;
      const size_t n = (size_t)a.n_stages * K * D;
      for (size_t i = tid; i < n; i += NTHR) IO::store1(po + i, poison);
    }
  }
}

#undef RELANE

}  // namespace ttt
