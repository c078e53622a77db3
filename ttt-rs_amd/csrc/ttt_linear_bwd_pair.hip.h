// TTT-Linear fused backward for gfx950 on TWO workgroups per (batch, head): f32 I/O, one checkpoint per mini-batch,
// head_dim 32 / 64, one feature tile per wave (the feature-split scheme of ttt_linear_bwd_mw.hip.h).
//
// With f32 I/O the reverse scan is bound by the f32 matrix instructions of the four SIMDs that hold a unit, and by the
// chain of dependent steps of a mini-batch that one wave per SIMD cannot overlap; a batch of 8 x 12 heads leaves 160 of
// 256 CUs without work.  A mini-batch's work falls into two parts of about equal matrix time (112 and 148
// v_mfma_f32_16x16x4_f32 per wave at head_dim 64, packed checkpoints):
//   producer  everything that needs only the saved state W_t and the inputs: Z1, its LayerNorm and G, the attention
//             block, Zbar, the output-LayerNorm backward dZbar, P = dZbar G^T, dA, d eta, dXQ (final), dA^T XQ, M^T dZbar;
//   consumer  everything that needs the state gradient carried from the later mini-batches: S = XK dW + db, G dW^T,
//             the second-order LayerNorm backward dZ1, dXV, dXK, d lr, d token_eta, and the rank-32 update of dW, db.
// Nothing of the consumer's flows back.  The producer workgroup runs ahead of the consumer; what crosses lies in a
// ring of three slots per unit in global memory (the caller's workspace): the producer stores the consumer's operands
// exactly as the consumer's lanes hold them (1 KiB per wave instruction; 29 KiB per mini-batch at head_dim 64: dZbar^T
// and G of every wave, xhat, gx, gO, M^T dZbar, dA^T XQ of the own features, eight scalars per token), the consumer
// copies a slot global -> LDS without passing registers, one mini-batch ahead, into one of two LDS buffers, together
// with what it takes from the inputs itself (the W tiles of the checkpoint, the rows of XK and XQ).
//
// Each workgroup has a CONTROL WAVE beside its NW compute waves.  It issues every global -> LDS copy, polls the
// partner's counter and raises its own side's, and takes part in every barrier.  A copy costs the wave that issues it
// about a hundred cycles of stalled issue (measured: the same copies dealt to the compute waves, between their matrix
// instructions, made a mini-batch 1 000 - 1 600 cycles longer on either side), a poll is a round trip to the L2; with
// the control wave neither sits in the instruction stream of a wave that feeds the matrix pipe.
//
// Two counters per unit say how far each side has come: the producer raises its own when every store of a slot has
// been acknowledged (every compute wave waits for its stores in front of a barrier, the control wave raises behind it),
// the consumer waits for it and copies -- with device-scope loads, which do not look in the CU's vector cache; the
// consumer raises its own when the copies of a slot have landed, and the producer waits for slot t + 3 to have landed
// before it overwrites that slot.
// Workgroups b and b + 8 of every 16 share a unit: consecutive workgroup ids go to the XCDs in turn, so both run
// behind one L2.  Each publishes its XCD number; the producer publishes with a device-scope release (write-back
// of its L2) until it has read the consumer's number and found it equal to its own, and the consumer puts a
// device-scope acquire in front of its copies until it has found the producer's equal to its own.  Every wait is
// bounded; a side that waits in vain marks its counter, both run to the end without waiting again, the consumer makes
// the unit's d_b0 NaN and the status word g_mlp_fwd_lost_workgroups counts both.
//
// Arithmetic: that of ttt_linear_bwd_mw_kernel<F32, D, D/16, PK> term by term (reference
// rust/fused/src/linear_fused_tile/backward/kernel.rs:253-429, backward/stage.rs:42-1006, layer_norm.rs:428-709).
#pragma once
#include "ttt_linear_bwd_mw.hip.h"

namespace ttt {

// lds_dma16 with a device-scope load (sc1): the load does not look in the CU's vector cache, so it sees what another
// CU behind the same L2 stored and had acknowledged, without the cache being dropped first.
__device__ __forceinline__ void lds_dma16_dev(const void* base, unsigned lane_off, unsigned lds_base) {
  unsigned saved;
  asm volatile(
      "s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 sc1\n\ts_nop 0\n\ts_mov_b32 m0, %0"
      : "=&s"(saved)
      : "v"(lane_off), "s"(uniform_ptr(base)), "s"(lds_base)
      : "memory");
}

// lds_dma16 with a non-temporal load: for rows that nothing reads again (the producer's xv and d_out, everything the
// consumer takes from the inputs, which the producer has read before it).  Lines brought in this way do not push the
// hand-over slots out of the L2, where they are meant to stay between their store and their one read: 170 MB per
// step less between L2 and memory at 8 x 12 units of 2048 tokens.  (Non-temporal on every input copy lost as much as
// it won: the consumer's read of the checkpoint then missed the L2.)
__device__ __forceinline__ void lds_dma16_nt(const void* base, unsigned lane_off, unsigned lds_base) {
  unsigned saved;
  asm volatile(
      "s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt\n\ts_nop 0\n\ts_mov_b32 m0, %0"
      : "=&s"(saved)
      : "v"(lane_off), "s"(uniform_ptr(base)), "s"(lds_base)
      : "memory");
}

struct LinearBwdPairArgs {
  LinearBwdArgs a;
  unsigned char* hand;  // [B*H][kLinBwdPairSlots][LinBwdPair<D>::H_BYTES] hand-over ring
  unsigned* flags;      // [B*H][kLinBwdPairFlagWords] progress words, zero on entry
  unsigned spin_limit;  // polls before a wait for the partner gives up; 0: give up at once (tests of that path)
  int agent_release;    // 1: the producer always publishes with a device-scope release
};

constexpr int kLinBwdPairSlots = 3;
constexpr int kLinBwdPairFlagWords = 16;  // per unit: [0] producer's count, [1] consumer's count, [2], [3] XCD numbers
constexpr unsigned kLinBwdPairPoison = 0xffffffffu;

template <int D, bool PK>
struct LinBwdPair {
  static constexpr int NT = D / 16, NW = NT;
  // ---- a hand-over slot (bytes); every piece is a 1 KiB row: 16 bytes per lane of the wave that holds it.  What the
  // consumer can take from the inputs itself (the state W_t from the checkpoint, XK^T and XQ^T) is not handed over: a
  // slot is written once and read once through the L2, and what does not fit there is written back to memory.
  static constexpr int H_FRK = 0;                         // 2 kinds x NT: dZbar^T fragments, G fragments
  static constexpr int H_OWN = H_FRK + 2 * NT * 1024;     // 5 kinds x NT: xhat, gx, gO, M^T dZbar, dA^T XQ of wave w's features
  static constexpr int H_SC = H_OWN + 5 * NT * 1024;      // 16 kinds x 16 tokens of f32 (8 used)
  static constexpr int H_BYTES = H_SC + 1024;
  static constexpr int H_ROWS = H_BYTES / 1024;
  enum { ZD = 0, GF };
  enum { XH = 0, GX, GO, DGM, DKP };
  enum { S_RSTD = 0, S_AXH, S_AXH2, S_GX, S_GXXH, S_LR, S_E1, S_E2 };
  // ---- consumer LDS: two buffers of (slot image, XK rows, XQ rows, the W tiles of the checkpoint), then its own
  // exchange areas
  static constexpr int C_XK = H_BYTES;                    // NT rows
  static constexpr int C_XQ = C_XK + NT * 1024;           // NT rows
  static constexpr int C_W = C_XQ + NT * 1024;            // NT*NT rows, as the producer stages them
  static constexpr int C_BUF = C_W + NT * NT * 1024;
  static constexpr int C_SUM = 2 * C_BUF;                 // [8 sums][16 tokens][NW]
  static constexpr int C_FR = C_SUM + 8 * 16 * NW * 4;    // 4 kinds x NT rows: dZ1 fragments in both forms, XK^T, XQ^T
  static constexpr int C_M0 = C_FR + 4 * NT * 1024;       // D row means of the initial W, then mean(b)
  static constexpr int C_CTL = C_M0 + (D + 4) * 4;        // control words
  static constexpr int C_BYTES = C_CTL + 16;
  // ---- producer LDS: the staging of ttt_linear_bwd_mw_kernel in two buffers used alternately, its exchange areas
  static constexpr int P_W = 0;
  static constexpr int P_B = P_W + NT * NT * 1024;        // NT rows (row w: the bias of wave w's features)
  static constexpr int P_X = P_B + NT * 1024;             // 4 tensors x NT rows
  static constexpr int P_LR = P_X + 4 * NT * 1024;
  static constexpr int P_BUF = P_LR + 256;
  static constexpr int P_SUM = 2 * P_BUF;                 // 2 exchanges x [8][16][NW]
  static constexpr int P_PT = P_SUM + 2 * 8 * 16 * NW * 4;  // 4 kinds x [NW] partial [16 x 16] blocks
  static constexpr int P_ZF = P_PT + 4 * NW * 1024;       // dZbar fragments of every wave
  static constexpr int P_M0 = P_ZF + NT * 1024;           // D row means of the initial W, then mean(b)
  static constexpr int P_CTL = P_M0 + (D + 4) * 4;
  static constexpr int P_BYTES = P_CTL + 16;
  // at least 81 KiB, so that a CU never hosts two workgroups of this kernel: the two sides of a unit must not share
  // the matrix pipes they were split to double
  static constexpr int BYTES_RAW = C_BYTES > P_BYTES ? C_BYTES : P_BYTES;
  static constexpr int BYTES = BYTES_RAW > 81 * 1024 ? BYTES_RAW : 81 * 1024;
  static_assert(BYTES <= 160 * 1024, "exceeds the 160 KiB of LDS of a gfx950 CU");
  static_assert(P_M0 % 16 == 0 && C_FR % 16 == 0 && C_M0 % 16 == 0, "16-byte aligned areas");
};

template <int D, bool PK, bool FULL>
__global__ void __launch_bounds__(64 * (D / 16 + 1)) ttt_linear_bwd_pair_kernel(LinearBwdPairArgs pa) {
  using T = F32;
  using IO = Io<T>;
  using frag = f32x4;
  using L = LinBwdPair<D, PK>;
  constexpr int NT = L::NT, NW = L::NW, NQ = NT / 2;
  constexpr float inv_d = 1.0f / D;
  constexpr int R = kLinBwdPairSlots;
  const LinearBwdArgs& a = pa.a;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int lane = threadIdx.x & 63, c = lane & 15, g = lane >> 4;
  // NW compute waves and one control wave.  The control wave issues every global -> LDS copy (a copy costs the wave
  // that issues it about a hundred cycles of stalled issue, four dozen of them per mini-batch), polls the partner's
  // counter and raises this side's (a round trip to the L2 each): none of that then sits in the instruction stream
  // of a wave that feeds the matrix pipe.  It takes part in every barrier.
  const int w_raw = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const bool ctlw = w_raw == NW;
  const int w = ctlw ? 0 : w_raw;  // the control wave loads what wave 0 loads (valid addresses) and stores nothing
  const bool boss = ctlw && lane == 0;
  const size_t bh = (size_t)(blockIdx.x >> 4) * 8 + (blockIdx.x & 7);
  const int role = (blockIdx.x >> 3) & 1;  // 0 producer, 1 consumer
  if (bh >= (size_t)a.B * a.H) return;
  const int h = (int)(bh % a.H);
  const int K = a.K, N = a.n_stages;
  const bool tok_ok = FULL || c < K;

  unsigned* const fl = pa.flags + bh * (size_t)kLinBwdPairFlagWords;
  unsigned char* const hand = pa.hand + bh * (size_t)R * L::H_BYTES;
  const unsigned stg = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)smem;
  // control words in LDS, written by thread 0 only: [0] lost, [1] the partner sits behind the same L2
  int* const ctl = reinterpret_cast<int*>(smem + (role == 0 ? L::P_CTL : L::C_CTL));

  // rows of absent tokens (c >= K) are never fetched: they stay zero
  for (int i = threadIdx.x; i < L::BYTES / 16; i += 64 * (NW + 1)) reinterpret_cast<u32x4*>(smem)[i] = u32x4{0u, 0u, 0u, 0u};
  __syncthreads();
  unsigned my_xcc;
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(my_xcc));
  my_xcc &= 15u;
  if (boss) {
    ctl[0] = pa.spin_limit == 0 ? 1 : 0;
    ctl[1] = 0;
    __hip_atomic_store(fl + 2 + role, 0x100u | my_xcc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  // first lane of the control wave: polls the partner's counter until it has reached `want`.  The last value read is kept: the partner is
  // usually several mini-batches ahead, and a poll is a round trip to the L2 on the path of every mini-batch.
  unsigned known = 0;
  auto poll = [&](int which, int want) {
    if (want > 0 && boss && ctl[0] == 0 && known < (unsigned)want) {
      bool got = false;
      for (unsigned i = 0; i < pa.spin_limit; ++i) {
        const unsigned v = __hip_atomic_load(fl + which, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (v == kLinBwdPairPoison) break;
        if (v >= (unsigned)want) {
          known = v;
          got = true;
          break;
        }
        __builtin_amdgcn_s_sleep(2);
      }
      if (!got) ctl[0] = 1;
    }
  };
  // The word read from LDS is moved to a scalar register by hand: the compiler takes a value loaded from a uniform
  // LDS address for uniform, and has been seen to compare it on the vector unit and then select on the scalar
  // condition code, which that comparison does not set (the counter then read "poison" after a clean run).
  auto raise = [&](int which, int value) {
    if (boss) {
      const int lost_now = __builtin_amdgcn_readfirstlane(ctl[0]);
      __hip_atomic_store(fl + which, lost_now != 0 ? kLinBwdPairPoison : (unsigned)value, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    }
  };

  const float te_last = a.token_eta[K - 1];
  const frag ident = identity_frag<T>(c, g);
  const frag ones = splat_frag<T>(1.f);
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  const int fo = own_offset<1>(w, 0, g);
  const f32x4 gam = *reinterpret_cast<const f32x4*>(a.gamma + h * D + fo);
  const f32x4 bet = *reinterpret_cast<const f32x4*>(a.beta + h * D + fo);
  const f32x4 a2 = gam * gam;
  f32x4 dgam = zero4, dbet = zero4;
  float sum_a = 0.f;
  for (int f = 0; f < D; ++f) sum_a += a.gamma[h * D + f] * a.gamma[h * D + f];

  auto tokens_k = [&](frag x) {
    f32x4 t = {0.f, 0.f, 0.f, 0.f};
    IO::mma(t, x, ident);
    return t;
  };
  auto mma_all = [&](f32x4& acc, const frag (&A)[NT], const frag (&B)[NT]) {
#pragma unroll
    for (int qq = 0; qq < NQ; ++qq) IO::mma2(acc, A[2 * qq], A[2 * qq + 1], B[2 * qq], B[2 * qq + 1]);
  };
  auto xpub = [&](float* e, const float (&S)[8]) {
    const float v0 = xg_sum4_scatter(S[0], S[1], S[2], S[3]);
    const float v1 = xg_sum4_scatter(S[4], S[5], S[6], S[7]);
    e[(g * 16 + c) * NW + w] = v0;
    e[((g + 4) * 16 + c) * NW + w] = v1;
  };
  auto xcol = [&](const float* e, float (&S)[8]) {
    lds_barrier();
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float s = 0.f;
#pragma unroll
      for (int ww = 0; ww < NW; ++ww) s += e[(i * 16 + c) * NW + ww];
      S[i] = s;
    }
  };
  auto store_own = [&](void* base, size_t tokoff, f32x4 x) {
    *reinterpret_cast<f32x4*>(static_cast<float*>(base) + tokoff + fo) = x;
  };

  // the scan works on the centred state, as the one-workgroup kernel does: row means of the initial W (a packed
  // checkpoint holds the centred matrix already) and the mean of the initial bias
  float* const M0p = reinterpret_cast<float*>(smem + (role == 0 ? L::P_M0 : L::C_M0));
  {
    const size_t c0 = bh * (size_t)a.n_ckpt;
    if (!PK) {
      for (int i = threadIdx.x; i < D; i += 64 * (NW + 1)) {
        const f32x4* row = reinterpret_cast<const f32x4*>(a.W_ckpt + c0 * D * D + (size_t)i * D);
        float sum = 0.f;
        for (int j = 0; j < D / 4; ++j) {
          const f32x4 v = row[j];
          sum += (v[0] + v[1]) + (v[2] + v[3]);
        }
        M0p[i] = sum * inv_d;
      }
    }
    if (threadIdx.x == 0) {
      float sum = 0.f;
      for (int f = 0; f < D; ++f) sum += a.b_ckpt[c0 * D + f];
      M0p[D] = sum * inv_d;
    }
    __syncthreads();
  }
  const float mrowo = PK ? 0.f : M0p[feat(w, c)];  // mean of row feat(w, c): the wave's own row tile

  if (role == 0) {
    // =============================================================================================== producer
    float* const SUMp = reinterpret_cast<float*>(smem + L::P_SUM);
    f32x4* const PTp = reinterpret_cast<f32x4*>(smem + L::P_PT);
    enum { P_AT = 0, P_AT2, P_P, P_P2 };
    auto pt = [&](int kind, int ww) -> f32x4& { return PTp[(kind * NW + ww) * 64 + lane]; };
    auto ptsum = [&](int kind) {
      f32x4 s = pt(kind, 0);
#pragma unroll
      for (int ww = 1; ww < NW; ++ww) s += pt(kind, ww);
      return s;
    };
    const float te_c = (c < K) ? a.token_eta[c] : 0.f;
    f32x4 te_s;
#pragma unroll
    for (int r = 0; r < 4; ++r) te_s[r] = (4 * g + r < K) ? a.token_eta[4 * g + r] : 0.f;

    float mrow[NT];
#pragma unroll
    for (int I = 0; I < NT; ++I) mrow[I] = PK ? 0.f : M0p[feat(I, c)];
    const float bbar = M0p[D];

    // copies of one mini-batch into staging buffer (stage & 1): the control wave's
    auto copy_in = [&](int stage) {
      const unsigned dst = stg + (unsigned)(stage & 1) * L::P_BUF;
      const size_t ci = bh * (size_t)a.n_ckpt + stage;
      const float* Wg = a.W_ckpt + ci * D * D;
#pragma unroll
      for (int n = 0; n < NT * NT; ++n) {
        const int I = n / NT, J = n - I * NT;
        if (PK)
          lds_dma16(Wg, (unsigned)(n * 1024 + lane * 16), dst + L::P_W + n * 1024);
        else
          lds_dma16(Wg, (unsigned)(feat(I, c) * D + 32 * (J >> 1) + 8 * g + 4 * (J & 1)) * 4u, dst + L::P_W + n * 1024);
      }
      const size_t tok0 = (bh * (size_t)a.seq_stride + (size_t)stage * K) * D;
#pragma unroll
      for (int J = 0; J < NT; ++J) {
        const unsigned foJ = (unsigned)(32 * (J >> 1) + 8 * g + 4 * (J & 1));  // own_offset of wave J's tile
        lds_dma16(a.b_ckpt + ci * D, foJ * 4u, dst + L::P_B + J * 1024);
        if (FULL || c < K) {
          lds_dma16(static_cast<const float*>(a.xq) + tok0, ((unsigned)(c * D) + foJ) * 4u, dst + L::P_X + (0 * NT + J) * 1024);
          lds_dma16(static_cast<const float*>(a.xk) + tok0, ((unsigned)(c * D) + foJ) * 4u, dst + L::P_X + (1 * NT + J) * 1024);
          lds_dma16_nt(static_cast<const float*>(a.xv) + tok0, ((unsigned)(c * D) + foJ) * 4u, dst + L::P_X + (2 * NT + J) * 1024);
          lds_dma16_nt(static_cast<const float*>(a.d_out) + tok0, ((unsigned)(c * D) + foJ) * 4u, dst + L::P_X + (3 * NT + J) * 1024);
        }
      }
      if (lane < 16) {
        const float* lrp = static_cast<const float*>(a.lr) + bh * (size_t)a.seq_stride + (size_t)stage * K;
        lds_dma4(lrp, 4u * (unsigned)(c < K ? c : K - 1), dst + L::P_LR);
      }
    };
    if (ctlw) {
      // ---- the control wave: per mini-batch the four barriers of the compute waves
      copy_in(N - 1);
      for (int st = N - 1; st >= 0; --st) {
        // the copies of this mini-batch have landed; its slot, last read as the slot of mini-batch st + R, is free
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        poll(1, N - (st + R));
        if (boss && ctl[1] == 0 && pa.agent_release == 0) {
          const unsigned other = __hip_atomic_load(fl + 3, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          ctl[1] = other == (0x100u | my_xcc) ? 1 : 0;
        }
        lds_barrier();  // top
        if (st > 0) copy_in(st - 1);  // the other buffer: last read before the X1 barrier of mini-batch st + 1
        lds_barrier();  // X1: in front of it every compute wave has waited for its stores of mini-batch st + 1
        if (st + 1 < N) raise(0, N - (st + 1));
        lds_barrier();  // X2
        lds_barrier();  // X3
      }
      lds_barrier();
      raise(0, N);
      if (boss && ctl[0] != 0) atomicAdd(&g_mlp_fwd_lost_workgroups, 1u);
      return;
    }
    bool fast = false;  // the consumer is known to sit behind the same L2

    // The counted wait of the compute waves.  Memory operations of a wave retire in the order they were issued, stores
    // included, so "s_waitcnt vmcnt(n)" with n = the number of operations a wave is KNOWN to have issued behind the
    // ones it waits for leaves those younger operations in flight.  In front of X1 a compute wave stores nothing of
    // this mini-batch (the first store, xhat, follows the exchange), so everything it has in flight is waited for.
    constexpr int kStoresBeforeX1 = 0;
    auto open_slot = [&](int) { lds_barrier(); };
    // in front of the X1 barrier of mini-batch st: every store of the slot of mini-batch st + 1 has been acknowledged
    // (the stores of this mini-batch so far may stay in flight), or, while the partner is not known to share the L2,
    // written back
    auto close_slot_wait = [&]() {
      if (fast)
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kStoresBeforeX1) : "memory");
      else
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    };

    for (int st = N - 1; st >= 0; --st) {
      open_slot(st);
      unsigned char* const hs = hand + (size_t)(st % R) * L::H_BYTES + lane * 16;
      auto put = [&](int off, f32x4 v) { *reinterpret_cast<f32x4*>(hs + off) = v; };
      const unsigned char* sl = smem + (st & 1) * L::P_BUF + lane * 16;
      frag q[NT], k[NT];
#pragma unroll
      for (int s = 0; s < NT; ++s) {
        q[s] = *reinterpret_cast<const frag*>(sl + L::P_X + (0 * NT + s) * 1024);
        k[s] = *reinterpret_cast<const frag*>(sl + L::P_X + (1 * NT + s) * 1024);
      }
      const frag qo = *reinterpret_cast<const frag*>(sl + L::P_X + (0 * NT + w) * 1024);
      const frag ko = *reinterpret_cast<const frag*>(sl + L::P_X + (1 * NT + w) * 1024);
      const frag vo = *reinterpret_cast<const frag*>(sl + L::P_X + (2 * NT + w) * 1024);
      const frag oo = *reinterpret_cast<const frag*>(sl + L::P_X + (3 * NT + w) * 1024);
      float lr_c;
      f32x4 lr_s;
      {
        const float* lrw = reinterpret_cast<const float*>(smem + (st & 1) * L::P_BUF + L::P_LR);
        const f32x4 w4 = *reinterpret_cast<const f32x4*>(lrw + 4 * g);
        lr_c = (FULL || c < K) ? lrw[c] : 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) lr_s[r] = (FULL || 4 * g + r < K) ? w4[r] : 0.f;
      }
      const f32x4 bT = *reinterpret_cast<const f32x4*>(sl + L::P_B + w * 1024) - bbar;
      frag Wn[NT];
#pragma unroll
      for (int J = 0; J < NT; ++J) {
        if constexpr (PK)  // stored as (m = j, k = i): transposed on the matrix pipe
          Wn[J] = tokens_k(*reinterpret_cast<const frag*>(sl + L::P_W + (w * NT + J) * 1024));
        else
          Wn[J] = *reinterpret_cast<const f32x4*>(sl + L::P_W + (w * NT + J) * 1024) - mrowo;
      }
      const frag kdo = tokens_k(ko), qdo = tokens_k(qo);

      // ---- forward intermediates of the own features: Z1 = XK W + b, Zq = XQ W + b; partial attention blocks
      f32x4 z1 = bT, zb = bT;
#pragma unroll
      for (int qq = 0; qq < NQ; ++qq) {
        frag wa0, wa1;
        if constexpr (PK) {
          wa0 = *reinterpret_cast<const frag*>(sl + L::P_W + ((2 * qq) * NT + w) * 1024);
          wa1 = *reinterpret_cast<const frag*>(sl + L::P_W + ((2 * qq + 1) * NT + w) * 1024);
        } else {
          wa0 = tokens_k(*reinterpret_cast<const f32x4*>(sl + L::P_W + ((2 * qq) * NT + w) * 1024) - mrow[2 * qq]);
          wa1 = tokens_k(*reinterpret_cast<const f32x4*>(sl + L::P_W + ((2 * qq + 1) * NT + w) * 1024) - mrow[2 * qq + 1]);
        }
        IO::mma2(z1, wa0, wa1, k[2 * qq], k[2 * qq + 1]);
        IO::mma2(zb, wa0, wa1, q[2 * qq], q[2 * qq + 1]);
      }
      {
        f32x4 at = zero4, at2 = zero4;
        IO::mma(at, ko, qo);
        IO::mma(at2, qo, ko);
        pt(P_AT, w) = at;
        pt(P_AT2, w) = at2;
      }
      // ---- X1: raw moments of Z1
      const f32x4 tgt = bet - (vo - ko);
      const f32x4 bq = gam * tgt;
      float S1[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      {
        const f32x4 az = a2 * z1;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          S1[0] += z1[r];
          S1[1] += z1[r] * z1[r];
          S1[2] += az[r];
          S1[3] += az[r] * z1[r];
          S1[4] += bq[r];
          S1[5] += bq[r] * z1[r];
        }
      }
      xpub(SUMp, S1);
      close_slot_wait();
      xcol(SUMp, S1);
      fast = __builtin_amdgcn_readfirstlane(ctl[1]) != 0;

      const float mu1 = S1[0] * inv_d;
      const float rstd1 = __builtin_amdgcn_rsqf(fmaxf(S1[1] * inv_d - mu1 * mu1, 0.f) + a.eps);
      const float sa_xh = rstd1 * (S1[2] - mu1 * sum_a);
      const float sa_xh2 = rstd1 * rstd1 * (S1[3] - 2.f * mu1 * S1[2] + mu1 * mu1 * sum_a);
      const float s_gx = sa_xh + S1[4];
      const float s_gxxh = sa_xh2 + rstd1 * (S1[5] - mu1 * S1[4]);
      const float mgx = s_gx * inv_d, sgx = s_gxxh * inv_d;
      const f32x4 xh = (z1 - mu1) * rstd1;
      const f32x4 gx = a2 * xh + bq;
      const f32x4 G = (gx - mgx - xh * sgx) * rstd1;
      put(L::H_OWN + (L::XH * NT + w) * 1024, xh);
      put(L::H_OWN + (L::GX * NT + w) * 1024, gx);
      put(L::H_OWN + (L::GO * NT + w) * 1024, gam * xh + tgt);
      put(L::H_FRK + (L::GF * NT + w) * 1024, G);
      // ---- eta, tril(A), M = eta (1 + A) in both orientations
      f32x4 eta, onepA, eta2, onepA2, nM, M2;
      {
        const f32x4 At = ptsum(P_AT), At2 = ptsum(P_AT2);
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
      IO::mma(zb, tokens_k(G), nM);
      const f32x4 gx2 = oo * gam;
      float S2[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        S2[0] += zb[r];
        S2[1] += zb[r] * zb[r];
        S2[2] += gx2[r];
        S2[3] += gx2[r] * zb[r];
      }
      xpub(SUMp + 8 * 16 * NW, S2);
      xcol(SUMp + 8 * 16 * NW, S2);
      frag Zf, Zd;
      {
        const float mu2 = S2[0] * inv_d;
        const float rstd2 = __builtin_amdgcn_rsqf(fmaxf(S2[1] * inv_d - mu2 * mu2, 0.f) + a.eps);
        const float m1 = S2[2] * inv_d, m2 = rstd2 * (S2[3] - mu2 * S2[2]) * inv_d;
        const f32x4 x2 = (zb - mu2) * rstd2;
        dgam += oo * x2;
        dbet += oo;
        Zf = (gx2 - m1 - x2 * m2) * rstd2;
        Zd = tokens_k(Zf);
        *reinterpret_cast<frag*>(smem + L::P_ZF + w * 1024 + lane * 16) = Zf;
        put(L::H_FRK + (L::ZD * NT + w) * 1024, Zd);
        // ---- partial P = dZb G^T in both orientations
        f32x4 P = zero4, P2 = zero4;
        IO::mma(P, G, Zf);   // [s][t]
        IO::mma(P2, Zf, G);  // [t][s]
        pt(P_P, w) = P;
        pt(P_P2, w) = P2;
      }
      // ---- M^T dZb (own features)
      {
        f32x4 DGM = zero4;
        IO::mma(DGM, Zd, M2);
        put(L::H_OWN + (L::DGM * NT + w) * 1024, DGM);
      }
      lds_barrier();
      frag Zfa[NT];
#pragma unroll
      for (int J = 0; J < NT; ++J) Zfa[J] = *reinterpret_cast<const frag*>(smem + L::P_ZF + J * 1024 + lane * 16);
      const f32x4 P = ptsum(P_P), P2 = ptsum(P_P2);
      const f32x4 dA = -P * eta, dEta = -P * onepA, dA2 = -P2 * eta2, dEta2 = -P2 * onepA2;
      const size_t tokoff = (bh * (size_t)a.seq_stride + (size_t)st * K + c) * D;
      // ---- dXQ = dO + dZb W^T + dA XK   (own features)
      {
        f32x4 dQ = oo;
        mma_all(dQ, Wn, Zfa);
        IO::mma(dQ, kdo, dA);
        if (tok_ok) store_own(a.d_xq, tokoff, dQ);
      }
      // ---- dA^T XQ   (own features): where the consumer's dXK starts
      {
        f32x4 dKp = zero4;
        IO::mma(dKp, qdo, dA2);
        put(L::H_OWN + (L::DKP * NT + w) * 1024, dKp);
      }
      // ---- per-token scalars; the two sums over a row of d eta that d lr and d token_eta take
      {
        float e1 = 0.f, e2 = 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          e1 += dEta[r] * lr_s[r];
          e2 += dEta2[r] * te_s[r];
        }
        e1 = xg_sum(e1);
        e2 = xg_sum(e2);
        if (w == 0 && g == 0) {
          float* sc = reinterpret_cast<float*>(hand + (size_t)(st % R) * L::H_BYTES + L::H_SC) + c;
          sc[L::S_RSTD * 16] = rstd1;
          sc[L::S_AXH * 16] = sa_xh;
          sc[L::S_AXH2 * 16] = sa_xh2;
          sc[L::S_GX * 16] = s_gx;
          sc[L::S_GXXH * 16] = s_gxxh;
          sc[L::S_LR * 16] = lr_c;
          sc[L::S_E1 * 16] = e1;
          sc[L::S_E2 * 16] = e2;
        }
      }
    }
    if (fast)
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    lds_barrier();
    // the producer's share of the LayerNorm parameter gradients (output LayerNorm)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float sg = row16_sum_dpp(dgam[r]), sbt = row16_sum_dpp(dbet[r]);
      if (c == 0) {
        atomicAdd(a.d_gamma + h * D + fo + r, sg);
        atomicAdd(a.d_beta + h * D + fo + r, sbt);
      }
    }
    return;
  }

  // ================================================================================================= consumer
  float* const SUMp = reinterpret_cast<float*>(smem + L::C_SUM);
  auto fr2 = [&](int kind, int J) -> frag& { return *reinterpret_cast<frag*>(smem + L::C_FR + (kind * NT + J) * 1024 + lane * 16); };
  f32x4 dbT = a.d_b_out ? *reinterpret_cast<const f32x4*>(a.d_b_out + bh * D + fo) : zero4;
  // dWc[I]: rows i = feat(I, 4g+r), columns j = feat(w, c);  DT[J]: rows j = feat(J, 4g+r), columns i = feat(w, c)
  f32x4 dWc[NT], DT[NT];
#pragma unroll
  for (int I = 0; I < NT; ++I)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      dWc[I][r] = a.d_W_out ? a.d_W_out[bh * D * D + feat(I, 4 * g + r) * D + feat(w, c)] : 0.f;
      DT[I][r] = a.d_W_out ? a.d_W_out[bh * D * D + feat(w, c) * D + feat(I, 4 * g + r)] : 0.f;
    }
  // copies of one mini-batch into LDS buffer (stage & 1): the producer's slot, row by row, and the rows of XK.  The
  // slot is read with device-scope loads: the producer's stores were acknowledged by the L2 both sit behind.
  // In three portions, one per stretch between the barriers of a mini-batch and sized like the stretches: the compute
  // waves must not find the control wave still issuing copies when they reach a barrier.
  constexpr int kRowsA = L::H_ROWS / 4, kRowsB = L::H_ROWS / 2;
  auto copy_in = [&](int stage, int part) {
    const unsigned char* hs = hand + (size_t)(stage % R) * L::H_BYTES;
    const unsigned dst = stg + (unsigned)(stage & 1) * L::C_BUF;
    const int n0 = part == 0 ? 0 : part == 1 ? kRowsA : kRowsB, n1 = part == 0 ? kRowsA : part == 1 ? kRowsB : L::H_ROWS;
#pragma unroll 4
    for (int n = n0; n < n1; ++n) lds_dma16_dev(hs, (unsigned)(n * 1024 + lane * 16), dst + n * 1024);
    if (part == 0) {
      // the W tiles of the checkpoint, as the producer stages them
      const float* Wg = a.W_ckpt + (bh * (size_t)a.n_ckpt + stage) * D * D;
#pragma unroll 4
      for (int n = 0; n < NT * NT; ++n) {
        const int I = n / NT, J = n - I * NT;
        if (PK)
          lds_dma16_nt(Wg, (unsigned)(n * 1024 + lane * 16), dst + L::C_W + n * 1024);
        else
          lds_dma16_nt(Wg, (unsigned)(feat(I, c) * D + 32 * (J >> 1) + 8 * g + 4 * (J & 1)) * 4u, dst + L::C_W + n * 1024);
      }
    }
    if (part == 2) {
      const size_t tok0 = (bh * (size_t)a.seq_stride + (size_t)stage * K) * D;
      if (FULL || c < K) {
#pragma unroll
        for (int J = 0; J < NT; ++J) {
          const unsigned off = (unsigned)(c * D + 32 * (J >> 1) + 8 * g + 4 * (J & 1)) * 4u;
          lds_dma16_nt(static_cast<const float*>(a.xk) + tok0, off, dst + L::C_XK + J * 1024);
          lds_dma16_nt(static_cast<const float*>(a.xq) + tok0, off, dst + L::C_XQ + J * 1024);
        }
      }
    }
  };
  if (ctlw) {
    // ---- the control wave: per mini-batch the three barriers of the compute waves
    // whether the producer sits behind the same L2: until that is known, and for a producer behind another L2 (which
    // writes its L2 back), the copies follow a device-scope acquire
    auto acquire = [&]() {
      if (boss && ctl[1] == 0 && pa.agent_release == 0) {
        const unsigned other = __hip_atomic_load(fl + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ctl[1] = other == (0x100u | my_xcc) ? 1 : 0;
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      if (__builtin_amdgcn_readfirstlane(ctl[1]) == 0) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    };
    poll(0, N - (N - 1));
    __syncthreads();
    acquire();
    copy_in(N - 1, 0);
    copy_in(N - 1, 1);
    copy_in(N - 1, 2);
    for (int st = N - 1; st >= 0; --st) {
      // the copies of this mini-batch have landed; the producer has finished the next one
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      if (st > 0) poll(0, N - (st - 1));
      lds_barrier();  // top
      raise(1, N - st);
      if (st > 0) {
        acquire();
        copy_in(st - 1, 0);  // the other buffer: last read at the end of mini-batch st + 1
      }
      lds_barrier();  // X3
      if (st > 0) copy_in(st - 1, 1);
      lds_barrier();  // X4
      if (st > 0) copy_in(st - 1, 2);
    }
    if (boss && ctl[0] != 0) atomicAdd(&g_mlp_fwd_lost_workgroups, 1u);
    return;
  }
  __syncthreads();

  for (int st = N - 1; st >= 0; --st) {
    lds_barrier();  // top: the control wave has seen the copies of this mini-batch land
    const unsigned char* sl = smem + (st & 1) * L::C_BUF + lane * 16;
    auto own = [&](int kind) { return *reinterpret_cast<const f32x4*>(sl + L::H_OWN + (kind * NT + w) * 1024); };
    auto frk = [&](int kind, int J) { return *reinterpret_cast<const frag*>(sl + L::H_FRK + (kind * NT + J) * 1024); };
    const float* sc = reinterpret_cast<const float*>(smem + (st & 1) * L::C_BUF + L::H_SC) + c;
    const float rstd1 = sc[L::S_RSTD * 16], sa_xh = sc[L::S_AXH * 16], sa_xh2 = sc[L::S_AXH2 * 16];
    const float s_gx = sc[L::S_GX * 16], s_gxxh = sc[L::S_GXXH * 16], lr_c = sc[L::S_LR * 16];
    const float mgx = s_gx * inv_d, sgx = s_gxxh * inv_d;
    // ---- XK^T, XQ^T of the own features (tokens along k) for the state gradient: published for the other waves, read
    // behind the X4 barrier
    const frag kdo = tokens_k(*reinterpret_cast<const frag*>(sl + L::C_XK + w * 1024));
    const frag qdo = tokens_k(*reinterpret_cast<const frag*>(sl + L::C_XQ + w * 1024));
    fr2(2, w) = kdo;
    fr2(3, w) = qdo;
    // ---- S = XK dW + db, TMP = G dW^T (own features)
    f32x4 S = dbT, TMP = zero4;
    {
      frag k[NT], Gfa[NT];
#pragma unroll
      for (int J = 0; J < NT; ++J) {
        k[J] = *reinterpret_cast<const frag*>(sl + L::C_XK + J * 1024);
        Gfa[J] = frk(L::GF, J);
      }
#pragma unroll
      for (int qq = 0; qq < NQ; ++qq) {
        IO::mma2(S, dWc[2 * qq], dWc[2 * qq + 1], k[2 * qq], k[2 * qq + 1]);
        IO::mma2(TMP, DT[2 * qq], DT[2 * qq + 1], Gfa[2 * qq], Gfa[2 * qq + 1]);
      }
    }
    const f32x4 xh = own(L::XH), gx = own(L::GX), G = frk(L::GF, w);
    const float last = te_last * lr_c;
    const f32x4 u = (own(L::DGM) + last * S) * rstd1;  // u = -dG rstd1
    float S4[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    {
      const f32x4 au = a2 * u;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        S4[0] += u[r];
        S4[1] += u[r] * xh[r];
        S4[2] += au[r];
        S4[3] += au[r] * xh[r];
        S4[4] += u[r] * gx[r];
        S4[5] += G[r] * S[r];
      }
    }
    xpub(SUMp, S4);
    xcol(SUMp, S4);
    const size_t tokoff = (bh * (size_t)a.seq_stride + (size_t)st * K + c) * D;
    const float dl = -S4[5];
    f32x4 dK;
    frag Z1d;
    {
      const float s1 = S4[0] * inv_d, s2 = S4[1] * inv_d;
      const float q1 = (s1 * sum_a + s2 * sa_xh - S4[2] + s2 * s_gx + sgx * S4[0]) * inv_d;
      const float q2 = s1 * sa_xh + s2 * sa_xh2 - S4[3] + s2 * s_gxxh + sgx * S4[1];  // sum dxh xh
      const float s_uG = rstd1 * (S4[4] - mgx * S4[0] - sgx * S4[1]);                  // sum u G
      const float dsig = -(q2 * rstd1 - s_uG);
      const f32x4 dgx = s1 + xh * s2 - u;
      const f32x4 dy = gam * dgx;
      dgam += own(L::GO) * dgx + dy * xh;
      dbet += dy;
      const f32x4 dxh = dy * gam + gx * s2 + u * sgx;
      const frag Z1f = (dxh - q1) * rstd1 + xh * (dsig * inv_d);
      Z1d = tokens_k(Z1f);
      fr2(0, w) = Z1f;
      fr2(1, w) = Z1d;
      dK = own(L::DKP) + dy - last * TMP;
      if (tok_ok) store_own(a.d_xv, tokoff, -dy);
    }
    // ---- X4: dZ1 fragments
    lds_barrier();
    {
      frag Z1fa[NT], Wn[NT];
#pragma unroll
      for (int J = 0; J < NT; ++J) {
        Z1fa[J] = fr2(0, J);
        if constexpr (PK)  // stored as (m = j, k = i): transposed on the matrix pipe
          Wn[J] = tokens_k(*reinterpret_cast<const frag*>(sl + L::C_W + (w * NT + J) * 1024));
        else
          Wn[J] = *reinterpret_cast<const f32x4*>(sl + L::C_W + (w * NT + J) * 1024) - mrowo;
      }
      mma_all(dK, Wn, Z1fa);
      if (tok_ok) store_own(a.d_xk, tokoff, dK);
    }
    // ---- d lr (first wave), d token_eta (last wave)
    if (w == 0) {
      const float dlr = sc[L::S_E2 * 16] + te_last * dl;
      if (g == 0 && tok_ok) static_cast<float*>(a.d_lr)[bh * (size_t)a.seq_stride + (size_t)st * K + c] = dlr;
    }
    if (w == NW - 1) {
      float dte = sc[L::S_E1 * 16];
      const float tail = row16_sum_dpp(dl * lr_c);
      if (c == K - 1) dte += tail;
      if (g == 0 && tok_ok) atomicAdd(a.d_token_eta + (size_t)st * K + c, dte);
    }
    // ---- state gradient: dW += XQ^T dZb + XK^T dZ1 (column slice and transposed row slice), db
    {
      const frag Zd = frk(L::ZD, w);
#pragma unroll
      for (int I = 0; I < NT; ++I) {
        const frag qa = fr2(3, I), ka = fr2(2, I), za = frk(L::ZD, I), z1a = fr2(1, I);
        IO::mma2(dWc[I], qa, ka, Zd, Z1d);
        IO::mma2(DT[I], za, z1a, qdo, kdo);
      }
      IO::mma2(dbT, Zd, Z1d, ones, ones);
    }
  }

  const bool poison = ctl[0] != 0;
  // ---- results carried over the whole scan
#pragma unroll
  for (int I = 0; I < NT; ++I)
#pragma unroll
    for (int r = 0; r < 4; ++r) a.d_W0[bh * D * D + feat(I, 4 * g + r) * D + feat(w, c)] = dWc[I][r];
  if (c == 0) {
    const float nan = __builtin_nanf("");
    store4<F32>(a.d_b0 + bh * D + fo, poison ? f32x4{nan, nan, nan, nan} : dbT);
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const float sg = row16_sum_dpp(dgam[r]), sbt = row16_sum_dpp(dbet[r]);
    if (c == 0) {
      atomicAdd(a.d_gamma + h * D + fo + r, sg);
      atomicAdd(a.d_beta + h * D + fo + r, sbt);
    }
  }
}

}  // namespace ttt
