// TTT-MLP fused backward for gfx950: one workgroup (8 wavefronts) per (batch, head), or two (template flag PIPE: a
// producer that walks the state back and a consumer that carries the gradient, on two CUs).
//
// Arithmetic: the gradient of the TTT-MLP inner loop (reference rust/core/src/mlp.rs:127-208
// looped as rust/core/src/inner.rs:25-50).  The reference has no fused MLP kernel and
// differentiates these ops with Burn autodiff; this kernel applies the closed-form one-mini-batch
// backward in a reverse scan, the way the reference's TTT-Linear backward does
// (rust/fused/src/linear_fused_tile/backward/kernel.rs:253-429), including the second-order
// LayerNorm term (layer_norm.rs:428-709) and the second derivative of the tanh-GELU
// (rust/thundercube/src/unary_ops.rs:175-195).
//
// State without checkpoints.  The state (W1 [d,4d], W2 [4d,d], b1, b2) entering mini-batch t is
// not stored by the forward.  The forward sweep saves, per mini-batch, the two rank-16 factors of
// its state update, G1l = eta_last * G1 [16,4d] and G2l = eta_last * G2 [16,d] (30 KiB at d = 96
// against 590 KiB for the state), and hands over the FINAL state; the reverse scan un-applies the
// update of mini-batch t (W1 += XK^T G1l, W2 += X2^T G2l, ...) before it differentiates it.  The
// roll-back is exact up to one f32 rounding per element and mini-batch.
//
// Data placement: [16 x d] tiles, the [16 x 16] causal matrices, biases and their gradients live
// in LDS; the [16 x 4d] tiles, the rolling state and the gradient accumulators dW1, dW2 live in
// global memory (caller's workspace / output buffers, an L2-resident working set) and are read
// in place as MFMA operands.  Contractions are true-f32 MFMA, or (template flag BF) bf16-operand MFMA with f32
// accumulation; the state, the gradient accumulators and every tile stay f32 in memory either way.
#pragma once
#include "ttt_engine_fwd.hip.h"

namespace ttt {

struct MlpBwdArgs {
  const void* xq;
  const void* xk;
  const void* xv;
  const float* token_eta;
  const void* lr;
  const float* gamma;
  const float* beta;
  const void* d_out;
  const float* G1s;  // [B*H][N][16][4d]  eta_last * G1 per mini-batch (forward sweep)
  const float* G2s;  // [B*H][N][16][d]
  float* W1;         // [B*H][d][4d] final state on entry, initial state on exit
  float* W2;         // [B*H][4d][d]
  const float* b1f;  // [B*H][4d] final biases
  const float* b2f;  // [B*H][d]
  float* mt;         // [B*H][NMT][16][4d] scratch tiles
  void* d_xq;
  void* d_xk;
  void* d_xv;
  float* d_W1;  // [B*H][d][4d]; holds the upstream gradient (or zeros) on entry
  float* d_b1;
  float* d_W2;
  float* d_b2;
  void* d_lr;
  float* d_token_eta;
  float* d_gamma;
  float* d_beta;
  int B, H, seq, seq_stride, K, n_stages;
  float eps;
  // two workgroups per unit (template flag PIPE of the kernel)
  float* pipe;           // [B*H][MlpBwdPipe<d>::FLOATS]: second state buffer, second set of shared tiles, exchange blocks
  unsigned* pipe_flags;  // [B*H][kMlpBwdPipeFlagWords] progress words, zero on entry
  unsigned spin_limit;   // polls before a wait for the partner gives up; 0: give up at once (tests of that path)
  int agent_release;     // 1: the producer always publishes with a device-scope release
};

constexpr int kMlpBwdMTiles = 9;  // [16 x 4d] scratch tiles per (batch, head)
constexpr int kMlpBwdSharedTiles = 6;  // the first six are written by the recomputation and read by the gradient part
constexpr int kMlpBwdPipeFlagWords = 32;  // per unit: [0] producer's count, [1] consumer's count, [2], [3] XCD ids
constexpr unsigned kMlpBwdPipePoison = 0xffffffffu;

// What the two workgroups of a unit share besides the kernel's ordinary workspace (float offsets within a.pipe's
// slice of the unit): the second buffer of the rolling state, the second set of the shared [16 x 4d] tiles, and two
// exchange blocks for what the one-workgroup kernel hands from its first half to its second in LDS.
template <int D>
struct MlpBwdPipe {
  static constexpr int M = 4 * D;
  // exchange block
  static constexpr int XH = 0, G2 = XH + 16 * D, XH2 = G2 + 16 * D, A1 = XH2 + 16 * D, M1 = A1 + 256, M2 = M1 + 256,
                       A2P = M2 + 256, RSTD = A2P + 256, B2 = RSTD + 16, XB = (B2 + D + 3) / 4 * 4;
  // SHB: bf16 copies of the two state buffers (W1 then W2, D * M uint16_t each, for the buffer that held the final
  // state on entry and then for the second one), read as operands where the products take bf16 operands
  static constexpr int W1X = 0, W2X = W1X + D * M, TILES = W2X + M * D, XBLK = TILES + kMlpBwdSharedTiles * 16 * M,
                       SHB = XBLK + 2 * XB, FLOATS = SHB + 2 * D * M;
};

template <int D>
struct MlpBwdLds {
  static constexpr int M = 4 * D, LD = D + 4, LK = 17, KK = 16 * LK, TD = 16 * LD;
  // (XQ, XK) and (DZ2, G2, DZB2) are consecutive on purpose: see the fused accumulations of step 23
  static constexpr int XQ = 0, XK = XQ + TD, TG = XK + TD, DO = TG + TD, XH = DO + TD, DZ2 = XH + TD,
                       G2 = DZ2 + TD, DZB2 = G2 + TD, XH2 = DZB2 + TD, DG2 = XH2 + TD, DT = DG2 + TD,
                       DQ = DT + TD, DK = DQ + TD;
  static constexpr int ETA = DK + TD, A1 = ETA + KK, M1 = A1 + KK, M2 = M1 + KK, P = M2 + KK,
                       DA = P + KK, DETA = DA + KK, PART = DETA + KK;
  static constexpr int b1 = PART + 8 * 256, b2 = b1 + M, db1 = b2 + D, db2 = db1 + M, gam = db2 + D,
                       bet = gam + D, lr = bet + D, te = lr + 16, rstd1 = te + 16, dlast = rstd1 + 16,
                       PIPEW = dlast + 16, SKP = PIPEW + 16;
  // partial products of the split-k [16 x d] products, one tile per wave: where LDS has the room (d <= 96)
  static constexpr bool SPLITK = D <= 96;
  static constexpr int END = SKP + (SPLITK ? 8 * TD : 0);
  static constexpr size_t BYTES = sizeof(float) * END;
  static_assert(BYTES <= 160 * 1024, "exceeds the 160 KiB of LDS of a gfx950 CU");
};

// tanh-GELU with first and second derivative
__device__ __forceinline__ void gelu_tanh_all(float x, float& y, float& dy, float& ddy) {
  const float c = 0.7978845608f, a = 0.044715f;
  const float t = tanhf(c * (x + a * x * x * x));
  const float du = c * (1.f + 3.f * a * x * x), ddu = 6.f * a * c * x, s = 1.f - t * t;
  y = 0.5f * x * (1.f + t);
  dy = 0.5f * (1.f + t) + 0.5f * x * s * du;
  ddy = s * du + 0.5f * x * s * (ddu - 2.f * t * du * du);
}

// BF: every product takes its operands rounded to bf16 (bf16 I/O behind the register-resident forward sweep, whose
// own products and state updates took bf16 operands: the states the scan walks back through are the ones that
// sweep formed).  Otherwise all contractions are true-f32 MFMA.
//
// PIPE: two workgroups per unit on two CUs of one XCD.  A mini-batch's work falls into a part that needs only the
// state walked back (steps 1 - 10: the roll-back and the recomputation of the forward's intermediates) and a part
// that needs the gradient carried from the later mini-batches (steps 11 - 24).  The producer workgroup runs the
// first part one mini-batch ahead of the consumer, which runs the second; what crosses (the rolled-back state,
// six [16 x 4d] tiles, a block of LDS-sized tiles) lies in two sets of buffers used alternately, and two counters
// in global memory say how far each side has come.  Workgroup b is the producer and b + 8 the consumer of one
// unit: consecutive workgroup ids go to the XCDs in turn, so both run behind one L2; each reads its XCD id and the
// producer publishes with a device-scope release (write-back of its L2) until it has seen that the ids agree.
// Every wait is bounded: a side that waits in vain marks its counter, both run to the end without further waits, the
// consumer makes the unit's d_b1 NaN and the status word g_mlp_fwd_lost_workgroups counts the event.
template <class T, int D, bool BF = false, bool PIPE = false>
// One workgroup per CU (the LDS use decides that), two waves per SIMD: said explicitly, because the scheduler
// otherwise aims at a higher occupancy and, to save registers, issues independent loads one at a time.
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) ttt_mlp_bwd_kernel(MlpBwdArgs a) {
  using IO = Io<T>;
  using elem = typename IO::elem;
  using L = MlpBwdLds<D>;
  using E = Eng<BF>;
  constexpr int M = L::M, LD = L::LD, LK = L::LK;
  constexpr int NW = 8, GW = 32, NJD = D / GW, NJM = M / GW, NTD = D / 16, NTM = M / 16;
  constexpr int NBM = NTM / NW;  // [16 x 4d] products: one job of NBM tile columns per wave
  constexpr int NBD = NTD % 3 == 0 ? 3 : 2;
  constexpr float inv_d = 1.0f / D;
  // Two workgroups with bf16 operands: the producer also writes every rolled-back state matrix as bf16, and the eight
  // products that read W1 or W2 as an operand read that copy (half the bytes through the fabric; the same operand
  // bits, since the copy is rounded as the operand load would round).
  constexpr bool SHD = PIPE && BF;
  constexpr int RIDE = D <= 96 ? 2 : 1;  // products riding along on the W1 roll-back (head_dim 128 is at the register limit)
  extern __shared__ __attribute__((aligned(16))) float lds[];
  // The thread indices are re-derived from an opaque copy at the top of every mini-batch (below): the
  // address arithmetic of the ~30 tile products is cheap, but hoisted out of the scan as loop invariants
  // it would occupy several hundred registers and spill.
  int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int t = tid >> 5, cg = tid & 31;  // elementwise mapping: token t, columns cg + 32 j
  using PX = MlpBwdPipe<D>;
  size_t bh = blockIdx.x;
  int role = 2;  // 0 producer, 1 consumer, 2 both
  if constexpr (PIPE) {
    bh = (size_t)(blockIdx.x >> 4) * 8 + (blockIdx.x & 7);
    role = (blockIdx.x >> 3) & 1;
    if (bh >= (size_t)a.B * a.H) return;
  }
  const bool do_p = !PIPE || role == 0, do_c = !PIPE || role == 1;
  const int h = (int)(bh % a.H), K = a.K, N = a.n_stages;
  float *sb1 = lds + L::b1, *sb2 = lds + L::b2, *sdb1 = lds + L::db1, *sdb2 = lds + L::db2,
        *sgam = lds + L::gam, *sbet = lds + L::bet, *slr = lds + L::lr, *ste = lds + L::te;
  float* const W1h = a.W1 + bh * (size_t)D * M;
  float* const W2h = a.W2 + bh * (size_t)M * D;
  float* dW1 = a.d_W1 + bh * (size_t)D * M;
  float* dW2 = a.d_W2 + bh * (size_t)M * D;
  // [16 x 4d] scratch tiles
  float* mt = a.mt + bh * (size_t)kMlpBwdMTiles * 16 * M;
  float* const px = PIPE ? a.pipe + bh * (size_t)PX::FLOATS : nullptr;
  unsigned* const fl = PIPE ? a.pipe_flags + bh * (size_t)kMlpBwdPipeFlagWords : nullptr;
  int& lost = *reinterpret_cast<int*>(lds + L::PIPEW);  // written by thread 0 only
  unsigned my_xcc = 0;
  bool fast_release = false;  // producer: the consumer is known to sit behind the same L2
  if constexpr (PIPE) {
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(my_xcc));
    my_xcc &= 15u;
    if (tid == 0) {
      lost = a.spin_limit == 0 ? 1 : 0;
      __hip_atomic_store(fl + 2 + role, 0x100u | my_xcc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  // Waits until the partner's counter has reached `want` (thread 0 polls), then every wave drops what its CU's
  // vector cache holds, so that the loads that follow see what the partner stored before it raised the counter.
  auto wait_for = [&](int which, int want) {
    if (want > 0 && tid == 0 && lost == 0) {
      bool got = false;
      for (unsigned i = 0; i < a.spin_limit; ++i) {
        const unsigned v = __hip_atomic_load(fl + which, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (v == kMlpBwdPipePoison) break;
        if (v >= (unsigned)want) {
          got = true;
          break;
        }
        __builtin_amdgcn_s_sleep(2);
      }
      if (!got) lost = 1;
    }
    __syncthreads();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  };
  // Raises this side's counter once every store of every wave has reached the L2 (or, `wide`, device scope).  The
  // barrier inside also closes the mini-batch for the reuse of LDS.
  auto signal = [&](int which, int value, bool wide) {
    if (wide)
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    else
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0)
      __hip_atomic_store(fl + which, lost != 0 ? kMlpBwdPipePoison : (unsigned)value, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
  };

  for (int i = tid; i < M; i += 512) {
    sb1[i] = a.b1f[bh * M + i];
    sdb1[i] = a.d_b1[bh * M + i];
  }
  for (int i = tid; i < D; i += 512) {
    sb2[i] = a.b2f[bh * D + i];
    sdb2[i] = a.d_b2[bh * D + i];
    sgam[i] = a.gamma[h * D + i];
    sbet[i] = a.beta[h * D + i];
  }
  if (tid < 16) ste[tid] = (tid < K) ? a.token_eta[tid] : 0.f;
  float dgam_acc[NJD], dbet_acc[NJD];
#pragma unroll
  for (int j = 0; j < NJD; ++j) dgam_acc[j] = dbet_acc[j] = 0.f;
  __syncthreads();
  const float te_last = ste[K - 1];

  // the four activation tiles and the learning rates of the next mini-batch to be processed, in registers
  struct {
    float q[NJD], k[NJD], v[NJD], o[NJD], lr;
  } pre;
  auto fetch_inputs = [&](int stage) {
    const size_t r = (bh * (size_t)a.seq_stride + (size_t)stage * K + (t < K ? t : 0)) * D;
    const bool ok = t < K;
#pragma unroll
    for (int j = 0; j < NJD; ++j) {
      const float q = IO::load1(static_cast<const elem*>(a.xq) + r + cg + GW * j);
      const float k = IO::load1(static_cast<const elem*>(a.xk) + r + cg + GW * j);
      const float v = IO::load1(static_cast<const elem*>(a.xv) + r + cg + GW * j);
      const float o = IO::load1(static_cast<const elem*>(a.d_out) + r + cg + GW * j);
      pre.q[j] = ok ? q : 0.f, pre.k[j] = ok ? k : 0.f, pre.v[j] = ok ? v : 0.f, pre.o[j] = ok ? o : 0.f;
    }
    const int tl = (tid < K) ? tid : 0;
    const float l = IO::load1(static_cast<const elem*>(a.lr) + bh * (size_t)a.seq_stride + (size_t)stage * K + tl);
    pre.lr = (tid < K) ? l : 0.f;
  };
  // at head_dim 128 the kernel is at the register limit: there the tiles are fetched where they are needed
  constexpr bool PFIN = D <= 96;
  if constexpr (PFIN) fetch_inputs(N - 1);
  // C[16 x 16] (PART slices) = X Y^T over the 4d columns of two [16 x 4d] tiles, one k-slice per wave
  auto splitk_xyT = [&](const float* X, const float* Y) {
    const int c = lane & 15, g = lane >> 4;
    constexpr int KS = M / NW, NS = KS / 16;
    static_assert(KS % 16 == 0, "a wave's k-slice is a whole number of 16-deep steps");
    // both tiles are contiguous along k: loaded four lanes to a row, then exchanged into operand order
    f32x4 xa[NS], ya[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      xa[s] = load_rows_raw(X + wave * KS + 16 * s, M, lane);
      ya[s] = load_rows_raw(Y + wave * KS + 16 * s, M, lane);
    }
    __builtin_amdgcn_sched_barrier(0);
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      const f32x4 xo = rows_to_operand(xa[s], lane), yo = rows_to_operand(ya[s], lane);
      mma16<BF>(acc, xo, yo);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) lds[L::PART + wave * 256 + (4 * g + r) * 16 + c] = acc[r];
  };
  // this thread's NJM elements of a [16 x 4d] tile, all loads issued before any use (the tiles are
  // in global memory and may alias as far as the compiler knows, so a load-compute-store loop would
  // pay the full memory latency per element)
  // One address per tile and immediate offsets for its NJM elements: the element offset is made opaque per
  // call, or the compiler shares NJM 64-bit element indices between all tiles and spends a register pair and
  // a 64-bit add on every access.
  auto ldm = [&](const float* tile, float (&v)[NJM]) {
    int o = t * M + cg;
    asm volatile("" : "+v"(o));
    const float* p = tile + o;
#pragma unroll
    for (int j = 0; j < NJM; ++j) v[j] = p[GW * j];
  };
  auto stm = [&](float* tile, const float (&v)[NJM]) {
    int o = t * M + cg;
    asm volatile("" : "+v"(o));
    float* p = tile + o;
#pragma unroll
    for (int j = 0; j < NJM; ++j) p[GW * j] = v[j];
  };
  // C[16 x d] (LDS) op= A[16 x 4d] (global tile) * B[4d x d]: split over k across the waves where LDS has room
  // for the partial products, one job per tile column otherwise
  auto prod_k = [&](auto mode, float* C, const float* A, const float* B, int b_rs, int b_cs) {
    constexpr int MODE = decltype(mode)::value;
    if constexpr (L::SPLITK)
      E::template splitk<MODE, NW, NTD, M / (16 * NW)>(C, LD, lds + L::SKP, A, M, B, b_rs, b_cs, wave, lane, tid);
    else
      E::template lds<MODE, NW>(C, LD, A, M, 1, B, b_rs, b_cs, 1, NTD, M, wave, lane);
  };
  // the same with W1 or W2 as B: from the bf16 copy where there is one
  auto prod_w = [&](auto mode, float* C, const float* A, const float* B, int b_rs, int b_cs) {
    constexpr int MODE = decltype(mode)::value;
    if constexpr (L::SPLITK)
      E::template splitk<MODE, NW, NTD, M / (16 * NW), SHD>(C, LD, lds + L::SKP, A, M, B, b_rs, b_cs, wave, lane, tid);
    else
      E::template lds<MODE, NW>(C, LD, A, M, 1, B, b_rs, b_cs, 1, NTD, M, wave, lane);
  };
  static_assert(!SHD || L::SPLITK, "bf16 operands exist up to head_dim 96");
  using M0 = std::integral_constant<int, 0>;
  using M1 = std::integral_constant<int, 1>;
  using M2 = std::integral_constant<int, 2>;
  auto part_sum = [&](int tt, int s) {
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) v += lds[L::PART + w * 256 + tt * 16 + s];
    return v;
  };

  for (int st = N - 1; st >= 0; --st) {
    asm volatile("" : "+v"(tid));
    lane = tid & 63, wave = tid >> 6, t = tid >> 5, cg = tid & 31;
    const float* G1l = a.G1s + ((bh * N + st) * (size_t)16) * M;
    const float* G2l = a.G2s + ((bh * N + st) * (size_t)16) * D;
    const size_t row = bh * (size_t)a.seq_stride + (size_t)st * K + t;
    // The state entering mini-batch st is formed in W1 / W2 from the state in W1r / W2r (the same buffers, walked
    // back in place, unless two workgroups share the unit: then the buffer that held the final state on entry and
    // the second one take turns, so that the consumer still reads one while the producer forms the next).
    float *W1 = W1h, *W2 = W2h;
    const float *W1r = nullptr, *W2r = nullptr;
    // (X2, U, Xbar2) and (dZbar1, dZ1) are consecutive: each group is the k-side operand of one fused
    // rank-48 / rank-32 accumulation into dW2 / dW1
    float* sh = mt;
    float* xb = nullptr;
    uint16_t *W1b = nullptr, *W2b = nullptr;
    if constexpr (PIPE) {
      const bool home = ((st ^ N) & 1) == 0;
      W1 = home ? W1h : px + PX::W1X;
      W2 = home ? W2h : px + PX::W2X;
      W1r = home ? px + PX::W1X : W1h;
      W2r = home ? px + PX::W2X : W2h;
      if (st & 1) sh = px + PX::TILES;
      xb = px + PX::XBLK + (st & 1) * PX::XB;
      if constexpr (SHD) {
        W1b = reinterpret_cast<uint16_t*>(px + PX::SHB + (home ? 0 : D * M));
        W2b = W1b + D * M;
      }
    }
    // the state matrices as the products read them
    const float* W1o = SHD ? reinterpret_cast<const float*>(W1b) : W1;
    const float* W2o = SHD ? reinterpret_cast<const float*>(W2b) : W2;
    float *mZ1 = sh, *mX2 = sh + 16 * M, *mU = sh + 2 * 16 * M, *mXB2 = sh + 3 * 16 * M, *mG1 = sh + 4 * 16 * M,
          *mZB1 = sh + 5 * 16 * M, *mDXB = mt + 6 * 16 * M, *mDX2 = mt + 7 * 16 * M, *mS1 = mt + 8 * 16 * M;
    if constexpr (PIPE) {
      if (role == 0) {
        // the buffers of this parity were last read by the consumer in mini-batch st + 2
        wait_for(1, N - st - 2);
        if (!fast_release && a.agent_release == 0 && N - st - 2 > 0) {
          const unsigned other = __hip_atomic_load(fl + 3, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          fast_release = other == (0x100u | my_xcc);
        }
      } else {
        wait_for(0, N - st);
      }
    }

    // ---- 1. inputs of this mini-batch (fetched while the previous one was computed); target = XV - XK
    if constexpr (!PFIN) fetch_inputs(st);
#pragma unroll
    for (int j = 0; j < NJD; ++j) {
      const int o = t * LD + cg + GW * j;
      lds[L::XQ + o] = pre.q[j];
      lds[L::XK + o] = pre.k[j];
      lds[L::TG + o] = pre.v[j] - pre.k[j];
      lds[L::DO + o] = pre.o[j];
    }
    if (tid < 16) slr[tid] = pre.lr;
    if constexpr (PIPE) {
      if (role == 1) {
        // what the producer left for this mini-batch
#pragma unroll
        for (int j = 0; j < NJD; ++j) {
          const int o = t * LD + cg + GW * j, x = t * D + cg + GW * j;
          lds[L::XH + o] = xb[PX::XH + x];
          lds[L::G2 + o] = xb[PX::G2 + x];
          lds[L::XH2 + o] = xb[PX::XH2 + x];
        }
        if (tid < 256) {
          const int o = (tid >> 4) * LK + (tid & 15);
          lds[L::A1 + o] = xb[PX::A1 + tid];
          lds[L::M1 + o] = xb[PX::M1 + tid];
          lds[L::M2 + o] = xb[PX::M2 + tid];
          lds[L::DETA + o] = xb[PX::A2P + tid];  // 1 + A2: read and replaced by the same thread in step 13
        }
        if (tid < 16) lds[L::rstd1 + tid] = xb[PX::RSTD + tid];
        if (tid < D) sb2[tid] = xb[PX::B2 + tid];
      }
    }
    __syncthreads();
    if constexpr (PFIN) fetch_inputs(st > 0 ? st - 1 : 0);  // always: a load under a branch weakens every later wait
    const float last = te_last * slr[t];
    float rstd1 = 0.f;
    if (do_p) {
    // ---- 2. roll W1, b1 back to the state entering this mini-batch
    // Z1 = XK W1 (step 3) rides along on the rolled-back tiles, and where the registers allow so does XQ W1 (step 7)
    E::template rank<1, NW, NBM, 4, RIDE>(W1, M, lds + L::XK, 1, LD, G1l, M, 1, NTD, NTM, wave, lane, lds + L::XK, LD, mZ1, M, W1r,
                                          lds + L::XQ, mZB1, W1b);
    if (tid < M) sb1[tid] += col16_sum(G1l + tid, M);
    __syncthreads();
    // ---- 3. Z1 = XK W1 + b1 ; X2 = gelu(Z1)
    {
      float z[NJM], y[NJM];
      ldm(mZ1, z);
#pragma unroll
      for (int j = 0; j < NJM; ++j) {
        float dy;
        z[j] += sb1[cg + GW * j];
        gelu_tanh_pair(z[j], y[j], dy);
      }
      stm(mZ1, z);
      stm(mX2, y);
    }
    __syncthreads();
    // ---- 4. roll W2, b2 back
    E::template rank<1, NW, NBD, 4>(W2, D, mX2, 1, M, G2l, D, 1, NTM, NTD, wave, lane, nullptr, 0, nullptr, 0, W2r, nullptr,
                                    nullptr, W2b);
    if (tid < D) sb2[tid] += col16_sum(G2l + tid, D);
    __syncthreads();
    // ---- 5. Z2 = X2 W2 ; A1 = XQ XK^T ; eta
    prod_w(M0{}, lds + L::XH, mX2, W2o, D, 1);
    E::template lds<0, NW>(lds + L::A1, LK, lds + L::XQ, LD, 1, lds + L::XK, 1, LD, 1, 1, D, wave, lane, NTD % NW);
    if (tid < 256) {
      const int tt = tid >> 4, s = tid & 15;
      lds[L::ETA + tt * LK + s] = (s <= tt) ? ste[tt] * slr[s] : 0.f;
    }
    __syncthreads();
    // ---- 6. LayerNorm of Z2 + b2: x_hat, rstd, G2 ; M1 = eta (1 + A1)
    {
      float xh[NJD], gx[NJD], s1 = 0.f, s2 = 0.f;
      ln_stats<D, GW>(lds + L::XH + t * LD, sb2, cg, a.eps, xh, rstd1);
#pragma unroll
      for (int j = 0; j < NJD; ++j) {
        const int o = cg + GW * j;
        gx[j] = (sgam[o] * xh[j] + sbet[o] - lds[L::TG + t * LD + o]) * sgam[o];
        s1 += gx[j];
        s2 += gx[j] * xh[j];
      }
      s1 = rowgroup_sum<GW>(s1) * inv_d;
      s2 = rowgroup_sum<GW>(s2) * inv_d;
#pragma unroll
      for (int j = 0; j < NJD; ++j) {
        const int o = cg + GW * j;
        lds[L::XH + t * LD + o] = xh[j];
        lds[L::G2 + t * LD + o] = (gx[j] - s1 - xh[j] * s2) * rstd1;
      }
    }
    if (tid < 256) {
      const int tt = tid >> 4, s = tid & 15;
      lds[L::M1 + tt * LK + s] = lds[L::ETA + tt * LK + s] * (1.f + lds[L::A1 + tt * LK + s]);
    }
    __syncthreads();
    // ---- 7. U = G2 W2^T ; Zbar1 = XQ W1
    E::template lds<0, NW, NBM, 2, true, SHD>(mU, M, lds + L::G2, LD, 1, W2o, 1, D, 1, NTM, D, wave, lane);
    if constexpr (RIDE != 2) E::template lds<0, NW, NBM>(mZB1, M, lds + L::XQ, LD, 1, W1, M, 1, 1, NTM, D, wave, lane);
    __syncthreads();
    // ---- 8. G1 = U gelu'(Z1)
    {
      float z[NJM], u[NJM];
      ldm(mZ1, z);
      ldm(mU, u);
#pragma unroll
      for (int j = 0; j < NJM; ++j) {
        float y, dy;
        gelu_tanh_pair(z[j], y, dy);
        u[j] *= dy;
      }
      stm(mG1, u);
    }
    __syncthreads();
    // ---- 9. Zbar1 -= M1 G1 ; then + b1, Xbar2 = gelu
    E::template lds<2, NW, NBM, 4>(mZB1, M, lds + L::M1, LK, 1, mG1, M, 1, 1, NTM, 16, wave, lane);
    __syncthreads();
    {
      float z[NJM], y[NJM];
      ldm(mZB1, z);
#pragma unroll
      for (int j = 0; j < NJM; ++j) {
        float dy;
        z[j] += sb1[cg + GW * j];
        gelu_tanh_pair(z[j], y[j], dy);
      }
      stm(mZB1, z);
      stm(mXB2, y);
    }
    __syncthreads();
    // ---- 10. A2 = Xbar2 X2^T (split-k) ; Zbar2 = Xbar2 W2
    splitk_xyT(mXB2, mX2);
    prod_w(M0{}, lds + L::XH2, mXB2, W2o, D, 1);
    __syncthreads();
    if (tid < 256) {
      const int tt = tid >> 4, s = tid & 15;
      const float a2p = 1.f + part_sum(tt, s);
      lds[L::M2 + tt * LK + s] = lds[L::ETA + tt * LK + s] * a2p;
      if constexpr (PIPE) xb[PX::A2P + tid] = a2p;
    }
    __syncthreads();
    E::template lds<2, NW, 1, 4>(lds + L::XH2, LD, lds + L::M2, LK, 1, lds + L::G2, LD, 1, 1, NTD, 16, wave, lane);
    if constexpr (PIPE) {
      __syncthreads();
      // hand the LDS-resident results to the consumer
#pragma unroll
      for (int j = 0; j < NJD; ++j) {
        const int o = t * LD + cg + GW * j, x = t * D + cg + GW * j;
        xb[PX::XH + x] = lds[L::XH + o];
        xb[PX::G2 + x] = lds[L::G2 + o];
        xb[PX::XH2 + x] = lds[L::XH2 + o];
      }
      if (tid < 256) {
        const int o = (tid >> 4) * LK + (tid & 15);
        xb[PX::A1 + tid] = lds[L::A1 + o];
        xb[PX::M1 + tid] = lds[L::M1 + o];
        xb[PX::M2 + tid] = lds[L::M2 + o];
      }
      if (cg == 0) xb[PX::RSTD + t] = rstd1;
      if (tid < D) xb[PX::B2 + tid] = sb2[tid];
      signal(0, N - st, !fast_release);
    } else {
      __syncthreads();
    }
    }  // do_p
    if (do_c) {
    if constexpr (PIPE) {
      if (tid < 256) {
        const int tt = tid >> 4, s = tid & 15;
        lds[L::ETA + tt * LK + s] = (s <= tt) ? ste[tt] * slr[s] : 0.f;
      }
      rstd1 = lds[L::rstd1 + t];
    }
    // ---- 11. output LayerNorm backward: dZbar2
    {
      float xh[NJD], rstd2, gx2[NJD], s1 = 0.f, s2 = 0.f;
      ln_stats<D, GW>(lds + L::XH2 + t * LD, sb2, cg, a.eps, xh, rstd2);
#pragma unroll
      for (int j = 0; j < NJD; ++j) {
        const int o = cg + GW * j;
        const float dO = lds[L::DO + t * LD + o];
        dgam_acc[j] += dO * xh[j];
        dbet_acc[j] += dO;
        gx2[j] = dO * sgam[o];
        s1 += gx2[j];
        s2 += gx2[j] * xh[j];
      }
      s1 = rowgroup_sum<GW>(s1) * inv_d;
      s2 = rowgroup_sum<GW>(s2) * inv_d;
#pragma unroll
      for (int j = 0; j < NJD; ++j) lds[L::DZB2 + t * LD + cg + GW * j] = (gx2[j] - s1 - xh[j] * s2) * rstd2;
    }
    __syncthreads();
    // ---- 12. P2 = dZbar2 G2^T ; dXbar2 = dZbar2 W2^T ; S2 = X2 dW2
    E::template lds<0, NW>(lds + L::P, LK, lds + L::DZB2, LD, 1, lds + L::G2, 1, LD, 1, 1, D, wave, lane, NW - 1);
    E::template lds<0, NW, NBM, 2, true, SHD>(mDXB, M, lds + L::DZB2, LD, 1, W2o, 1, D, 1, NTM, D, wave, lane);
    prod_k(M0{}, lds + L::DG2, mX2, dW2, D, 1);
    // T2 = (last G2) dW2^T, the term step 15 used to subtract from dX2, right behind the other pass over dW2: a wave
    // meets the same 4d/8 rows of dW2 in both, and the second pass finds them in the L2.  From here to step 22 the
    // tile holds -dX2.
    E::template lds<0, NW, NBM, 2, true>(mDX2, M, G2l, D, 1, dW2, 1, D, 1, NTM, D, wave, lane);
    __syncthreads();
    // ---- 13. dA2, d eta ; dG2 = -last (S2 + db2) ; d last
    if (tid < 256) {
      const int tt = tid >> 4, s = tid & 15;
      const float p = (s <= tt) ? lds[L::P + tt * LK + s] : 0.f;
      const float et = lds[L::ETA + tt * LK + s];
      lds[L::DA + tt * LK + s] = -p * et;
      // 1 + A2 = M2 / eta is not safe for eta = 0: recompute from the split-k sums still in PART (two workgroups:
      // the producer left it in this very element)
      const float a2p = PIPE ? lds[L::DETA + tt * LK + s] : 1.f + part_sum(tt, s);
      lds[L::DETA + tt * LK + s] = -p * a2p;
    }
    {
      float q = 0.f;
#pragma unroll
      for (int j = 0; j < NJD; ++j) {
        const int o = cg + GW * j;
        const float s2v = lds[L::DG2 + t * LD + o] + sdb2[o];
        q += lds[L::G2 + t * LD + o] * s2v;
        lds[L::DG2 + t * LD + o] = -last * s2v;
      }
      q = rowgroup_sum<GW>(q);
      if (cg == 0) lds[L::dlast + t] = -q;
    }
    __syncthreads();
    // ---- 14. dXbar2 += dA2 X2 ; dG2 -= M2^T dZbar2 ; -dX2 = T2 - dA2^T Xbar2
    E::template lds<1, NW, NBM, 4>(mDXB, M, lds + L::DA, LK, 1, mX2, M, 1, 1, NTM, 16, wave, lane);
    E::template lds<2, NW, 1, 4>(lds + L::DG2, LD, lds + L::M2, 1, LK, lds + L::DZB2, LD, 1, 1, NTD, 16, wave, lane);
    E::template lds<2, NW, NBM, 4>(mDX2, M, lds + L::DA, 1, LK, mXB2, M, 1, 1, NTM, 16, wave, lane);
    __syncthreads();
    // ---- 15. dZbar1 = dXbar2 gelu'(Zbar1)
    {
      float z[NJM], v[NJM];
      ldm(mZB1, z);
      ldm(mDXB, v);
#pragma unroll
      for (int j = 0; j < NJM; ++j) {
        float y, dy;
        gelu_tanh_pair(z[j], y, dy);
        v[j] *= dy;
      }
      stm(mDXB, v);
    }
    __syncthreads();
    // ---- 16. P1 = dZbar1 G1^T (split-k) ; dQ = dZbar1 W1^T ; S1 = XK dW1
    splitk_xyT(mDXB, mG1);
    prod_w(M0{}, lds + L::DQ, mDXB, W1o, 1, M);
    E::template lds<0, NW, NBM>(mS1, M, lds + L::XK, LD, 1, dW1, M, 1, 1, NTM, D, wave, lane);
    // T1 = (last G1) dW1^T, the term step 19 used to subtract from dK, right behind the other pass over dW1 (a wave
    // meets the same 4d/8 columns in both).  The barrier separates the two split-k products' partial sums.  From here
    // on the DK tile holds -dK.
    __syncthreads();
    prod_k(M0{}, lds + L::DK, G1l, dW1, 1, M);
    __syncthreads();
    // ---- 17. dA1, d eta ; dG1 = -last (S1 + db1) ; d last
    if (tid < 256) {
      const int tt = tid >> 4, s = tid & 15;
      const float p = (s <= tt) ? part_sum(tt, s) : 0.f;
      lds[L::DA + tt * LK + s] = -p * lds[L::ETA + tt * LK + s];
      lds[L::DETA + tt * LK + s] += -p * (1.f + lds[L::A1 + tt * LK + s]);
    }
    {
      float q = 0.f, sv[NJM], gv[NJM];
      ldm(mS1, sv);
      ldm(mG1, gv);
#pragma unroll
      for (int j = 0; j < NJM; ++j) {
        const float s1v = sv[j] + sdb1[cg + GW * j];
        q += gv[j] * s1v;
        sv[j] = -last * s1v;
      }
      stm(mS1, sv);
      q = rowgroup_sum<GW>(q);
      if (cg == 0) lds[L::dlast + t] -= q;
    }
    __syncthreads();
    // ---- 18. dG1 -= M1^T dZbar1 ; dQ += dA1 XK ; -dK = T1 - dA1^T XQ
    E::template lds<2, NW, NBM, 4>(mS1, M, lds + L::M1, 1, LK, mDXB, M, 1, 1, NTM, 16, wave, lane);
    E::template lds<1, NW, 1, 4>(lds + L::DQ, LD, lds + L::DA, LK, 1, lds + L::XK, LD, 1, 1, NTD, 16, wave, lane);
    E::template lds<2, NW, 1, 4>(lds + L::DK, LD, lds + L::DA, 1, LK, lds + L::XQ, LD, 1, 1, NTD, 16, wave, lane, NTD % NW);
    __syncthreads();
    // ---- 19. dU = dG1 gelu'(Z1) (kept in mU's place after saving U * gelu'')
    {
      float z[NJM], dg1[NJM], u[NJM];
      ldm(mZ1, z);
      ldm(mS1, dg1);
      ldm(mU, u);
#pragma unroll
      for (int j = 0; j < NJM; ++j) {
        float y, dy, ddy;
        gelu_tanh_all(z[j], y, dy, ddy);
        z[j] = dg1[j] * u[j] * ddy;  // first term of dZ1
        u[j] = dg1[j] * dy;          // dU
      }
      stm(mS1, z);
      stm(mU, u);
    }
    __syncthreads();
    // ---- 20. dG2 += dU W2
    prod_w(M1{}, lds + L::DG2, mU, W2o, D, 1);
    __syncthreads();
    // ---- 21. second-order LayerNorm: dZ2, dT, d gamma, d beta
    {
      float xh[NJD], dG[NJD], u[NJD], gO[NJD], gx[NJD], s1 = 0.f, s2 = 0.f, sgx = 0.f;
#pragma unroll
      for (int j = 0; j < NJD; ++j) {
        const int o = cg + GW * j;
        xh[j] = lds[L::XH + t * LD + o];
        dG[j] = lds[L::DG2 + t * LD + o];
        u[j] = -dG[j] * rstd1;
        gO[j] = sgam[o] * xh[j] + sbet[o] - lds[L::TG + t * LD + o];
        gx[j] = gO[j] * sgam[o];
        s1 += u[j];
        s2 += u[j] * xh[j];
        sgx += gx[j] * xh[j];
      }
      s1 = rowgroup_sum<GW>(s1) * inv_d;
      s2 = rowgroup_sum<GW>(s2) * inv_d;
      sgx = rowgroup_sum<GW>(sgx) * inv_d;
      float dxh[NJD], dy[NJD], q1 = 0.f, q2 = 0.f;
#pragma unroll
      for (int j = 0; j < NJD; ++j) {
        const int o = cg + GW * j;
        const float dgx = -u[j] + s1 + xh[j] * s2;
        dy[j] = sgam[o] * dgx;
        dgam_acc[j] += gO[j] * dgx + dy[j] * xh[j];
        dbet_acc[j] += dy[j];
        dxh[j] = dy[j] * sgam[o] + gx[j] * s2 + u[j] * sgx;
        q1 += dxh[j];
        q2 += dxh[j] * xh[j] + dG[j] * lds[L::G2 + t * LD + o];
      }
      q1 = rowgroup_sum<GW>(q1) * inv_d;
      const float dsig = -rowgroup_sum<GW>(q2) * rstd1;
#pragma unroll
      for (int j = 0; j < NJD; ++j) {
        const int o = cg + GW * j;
        lds[L::DZ2 + t * LD + o] = (dxh[j] - q1) * rstd1 + xh[j] * dsig * inv_d;
        lds[L::DT + t * LD + o] = -dy[j];
      }
    }
    __syncthreads();
    // ---- 22. dX2 += dZ2 W2^T (the tile holds -dX2) ; then dZ1 = dG1 U gelu''(Z1) + dX2 gelu'(Z1)
    E::template lds<2, NW, NBM, 2, true, SHD>(mDX2, M, lds + L::DZ2, LD, 1, W2o, 1, D, 1, NTM, D, wave, lane);
    __syncthreads();
    {
      float z[NJM], f1[NJM], dx[NJM];
      ldm(mZ1, z);
      ldm(mS1, f1);
      ldm(mDX2, dx);
#pragma unroll
      for (int j = 0; j < NJM; ++j) {
        float y, dy;
        gelu_tanh_pair(z[j], y, dy);
        dx[j] = f1[j] - dx[j] * dy;  // dZ1 (dx holds -dX2)
      }
      stm(mDX2, dx);
    }
    __syncthreads();
    // ---- 23. gradient accumulation; dK += dZ1 W1^T (as -dK -= ...)
    // dW2 += X2^T dZ2 + dU^T G2 + Xbar2^T dZbar2 as ONE rank-48 pass over dW2 (operands consecutive)
    E::template rank<1, NW, NBD, 12>(dW2, D, mX2, 1, M, lds + L::DZ2, LD, 1, NTM, NTD, wave, lane);
    // dW1 += XQ^T dZbar1 + XK^T dZ1 as one rank-32 pass
    E::template rank<1, NW, NBM, 8>(dW1, M, lds + L::XQ, 1, LD, mDXB, M, 1, NTD, NTM, wave, lane);
    prod_w(M2{}, lds + L::DK, mDX2, W1o, 1, M);  // the tile holds -dK
    if (tid < M) sdb1[tid] += col16_sum2(mDXB + tid, mDX2 + tid, M);
    if (tid < D) {
      float s = 0.f;
      for (int r = 0; r < 16; ++r) s += lds[L::DZB2 + r * LD + tid] + lds[L::DZ2 + r * LD + tid];
      sdb2[tid] += s;
    }
    __syncthreads();
    // ---- 24. stores
    if (t < K) {
      elem* pq = static_cast<elem*>(a.d_xq) + row * D;
      elem* pk = static_cast<elem*>(a.d_xk) + row * D;
      elem* pv = static_cast<elem*>(a.d_xv) + row * D;
#pragma unroll
      for (int j = 0; j < NJD; ++j) {
        const int o = cg + GW * j;
        const float dT = lds[L::DT + t * LD + o];
        IO::store1(pq + o, lds[L::DQ + t * LD + o] + lds[L::DO + t * LD + o]);
        IO::store1(pk + o, -lds[L::DK + t * LD + o] - dT);
        IO::store1(pv + o, dT);
      }
    }
    if (tid < 16) {
      const int s = tid;
      float dl = te_last * lds[L::dlast + s];
      for (int r = 0; r < 16; ++r) dl += lds[L::DETA + r * LK + s] * ste[r];
      if (s < K)
        IO::store1(static_cast<elem*>(a.d_lr) + bh * (size_t)a.seq_stride + (size_t)st * K + s, dl);
    } else if (tid >= 64 && tid < 80) {
      const int tt = tid - 64;
      float s = 0.f;
      for (int r = 0; r < 16; ++r) s += lds[L::DETA + tt * LK + r] * slr[r];
      if (tt == K - 1)
        for (int r = 0; r < 16; ++r) s += lds[L::dlast + r] * slr[r];
      if (tt < K) atomicAdd(a.d_token_eta + (size_t)st * K + tt, s);
    }
    if constexpr (PIPE)
      signal(1, N - st, false);
    else
      __syncthreads();
    }  // do_c
  }
  if constexpr (PIPE) {
    if (tid == 0 && lost != 0) atomicAdd(&g_mlp_fwd_lost_workgroups, 1u);
    if (role == 0) return;
  }
  const bool poison = PIPE && lost != 0;

  // ---- results carried over the whole scan
  for (int i = tid; i < M; i += 512) a.d_b1[bh * M + i] = poison ? __builtin_nanf("") : sdb1[i];
  for (int i = tid; i < D; i += 512) a.d_b2[bh * D + i] = sdb2[i];
#pragma unroll
  for (int j = 0; j < NJD; ++j) {
    lds[L::XQ + t * LD + cg + GW * j] = dgam_acc[j];
    lds[L::XK + t * LD + cg + GW * j] = dbet_acc[j];
  }
  __syncthreads();
  if (tid < D) {
    float sg = 0.f, sbt = 0.f;
    for (int r = 0; r < 16; ++r) {
      sg += lds[L::XQ + r * LD + tid];
      sbt += lds[L::XK + r * LD + tid];
    }
    atomicAdd(a.d_gamma + h * D + tid, sg);
    atomicAdd(a.d_beta + h * D + tid, sbt);
  }
}

}  // namespace ttt
