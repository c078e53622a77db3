// Workgroup-level tile engine shared by the LDS-resident kernels (TTT-Linear backward, the
// generic TTT-Linear forward and the TTT-MLP forward).
//
// Operands are f32 arrays addressed through (row stride, column stride) pairs, in LDS or in
// global memory, so a transposed operand is just a swapped pair of strides.  All products are
// true-f32 MFMA (v_mfma_f32_16x16x4_f32): lane (c = lane%16, g = lane/16) supplies A(16tm+c, k+g)
// and B(k+g, 16tn+c) for k = 0, 4, 8, ... and owns C(16tm+4g+r, 16tn+c), r = 0..3.
#pragma once
#include <type_traits>
#include "ttt_frag.hip.h"

namespace ttt {

// Status word of the kernels that spread a (batch, head) unit over two workgroups (TTT-MLP forward at head_dim 128,
// TTT-MLP backward): workgroups whose wait for their partner ran out, counted since the library was loaded (one
// copy per GPU).  Read by ttt_mlp_fwd_lost_workgroups.
__device__ unsigned int g_mlp_fwd_lost_workgroups = 0u;

// 16 rows x 64 bytes of a row-major matrix in GLOBAL memory, delivered in matrix-operand order: lane (c = lane % 16,
// g = lane / 16) receives the 16 bytes at row c, byte offset 16 g.  Loaded directly in that order, each quarter
// wave (16 lanes with the same g) touches 16 cache lines and the load runs at 16 B per cycle and CU; here lane l
// loads row l / 4, chunk l % 4, so a quarter wave touches 4 lines (the rate of a coalesced load), and the values
// change lanes afterwards (ds_bpermute: lane 16 g + c takes from lane 4 c + g).  `load_rows_raw` issues the load,
// `rows_to_operand` does the exchange, so that the exchange can sit where the value is used.  All 64 lanes of the
// wave must be active in both.
__device__ __forceinline__ f32x4 load_rows_raw(const float* block, int row_stride, int lane) {
  return *reinterpret_cast<const f32x4*>(block + (lane >> 2) * row_stride + 4 * (lane & 3));
}
__device__ __forceinline__ f32x4 rows_to_operand(const f32x4& v, int lane) {
  const int src = 4 * (4 * (lane & 15) + (lane >> 4));
  f32x4 o;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const float x = v[r];  // through a scalar: a bit_cast applied to the vector element itself reads element 0
    o[r] = __int_as_float(__builtin_amdgcn_ds_bpermute(src, __float_as_int(x)));
  }
  return o;
}

// The same for a matrix kept as bf16 (a second copy of a state matrix, written for the operand reads): 16 rows x 32
// bytes, lane l loads row l / 4, 8-byte chunk l % 4, and the exchange delivers a ready bf16 operand fragment.
__device__ __forceinline__ u32x2 load_rows_raw_h(const uint16_t* block, int row_stride, int lane) {
  return *reinterpret_cast<const u32x2*>(block + (lane >> 2) * row_stride + 4 * (lane & 3));
}
__device__ __forceinline__ u32x2 rows_to_operand(const u32x2& v, int lane) {
  const int src = 4 * (4 * (lane & 15) + (lane >> 4));
  const uint32_t x0 = v[0], x1 = v[1];
  return u32x2{(uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)x0), (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)x1)};
}
// operand fragment of a 16-deep step from what was loaded: f32 values are rounded, bf16 bits are taken as they are
__device__ __forceinline__ Io<BF16>::frag bf_frag(const f32x4& v) { return Io<BF16>::to_frag(v); }
__device__ __forceinline__ Io<BF16>::frag bf_frag(const u32x2& v) { return __builtin_bit_cast(Io<BF16>::frag, v); }

// One 16-deep step of a product: lane (c, g) holds four k slots of A (row c) and of B (column c).  BF: the operands
// are rounded to bf16 and take one v_mfma_f32_16x16x16_bf16 (a quarter of the issue slots of the f32 form at an
// eighth of the matrix-pipe time); otherwise four true-f32 v_mfma_f32_16x16x4_f32.  The accumulator is f32 either way.
// A kernel uses ONE of the two forms throughout, so no matrix instruction ever follows one of another opcode.
template <bool BF>
__device__ __forceinline__ void mma16(f32x4& acc, const f32x4& a, const f32x4& b) {
  if constexpr (BF)
    Io<BF16>::mma(acc, Io<BF16>::to_frag(a), Io<BF16>::to_frag(b));
  else
    Io<F32>::mma(acc, a, b);
}

// C[16*Mt x 16*Nt] (row-major, stride ldc)  op=  A * B over k in [k0, k0+Kd), Kd a multiple of 4 (of 16 with BF).
// A(m,k) = A[m*a_rs + k*a_cs], B(k,n) = B[k*b_rs + n*b_cs].
// MODE 0: C = AB   1: C += AB   2: C -= AB   3: C *= AB (elementwise)
//
// Work split: the tile row tm and a block of NB consecutive tile columns form one job; jobs are
// dealt round-robin to the NW waves of the workgroup, starting at wave `first`.  Inside a job the
// A element of a k-step is loaded once and feeds NB MFMAs, and KU k-steps of operands are fetched
// before the first MFMA of the group issues, so the loads of a group overlap its MFMAs.
// BG: B is in global memory and contiguous along k (a transposed weight matrix): loaded four lanes to a row and
// exchanged between lanes before use (load_rows_raw / rows_to_operand).
// BF: bf16 operands (mma16); the k-steps outside the contiguous-A path are then taken four at a time.
// BH (with BF and BG, A contiguous along k): B points at a bf16 copy of the matrix (uint16_t elements, same strides),
// whose bits are the operands; half the bytes per pass, no conversion.
template <bool BF, int MODE, int NW, int NB, int KU0, bool BG, bool BH = false>
__device__ __forceinline__ void mm_lds_t(float* C, int ldc, const float* A, int a_rs, int a_cs,
                                         const float* B, int b_rs, int b_cs, int Mt, int Nt, int Kd,
                                         int wave, int lane, int first, int k0) {
  constexpr int KU = BF ? ((KU0 + 3) / 4) * 4 : KU0;
  static_assert(!BH || (BF && BG), "a bf16 copy is read as a k-contiguous global operand of a bf16 product");
  using bop = std::conditional_t<BH, u32x2, f32x4>;
  const int c = lane & 15, g = lane >> 4;
  const int nblk = (Nt + NB - 1) / NB;
  const int njobs = Mt * nblk;
#pragma nounroll
  for (int job = (wave - first + NW) % NW; job < njobs; job += NW) {
    const int tm = job / nblk, tn0 = (job - tm * nblk) * NB;
    // 32-bit element offsets from the (wave-uniform) base pointers keep the address math in
    // single registers: base in SGPRs, one VGPR offset per access
    f32x4 acc[NB];
    const int coff = (16 * tm + 4 * g) * ldc + 16 * tn0 + c;
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const bool live = Nt % NB == 0 || tn0 + j < Nt;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float v = 0.f;
        if (MODE == 1 || MODE == 2) v = C[coff + r * ldc + 16 * (live ? j : 0)];
        acc[j][r] = (MODE == 2) ? -v : v;
      }
    }
    const int aoff = (16 * tm + c) * a_rs + (k0 + g) * a_cs;
    const int boff = (k0 + g) * b_rs + (16 * tn0 + c) * b_cs;
    const int astep = 4 * a_cs, bstep = 4 * b_rs, bcol = 16 * b_cs;
    // two operand buffers in ping-pong: the loads of the next group of KU k-steps are in flight
    // while the MFMAs of the current group issue (fixed buffers, so no load is ever copied)
    float avA[KU], bvA[KU][NB], avB[KU], bvB[KU][NB];
    auto fetch = [&](float (&av)[KU], float (&bv)[KU][NB], int kk) {
      const int ak = aoff + kk * a_cs, bk = boff + kk * b_rs;
#pragma unroll
      for (int u = 0; u < KU; ++u) {
        av[u] = A[ak + u * astep];
#pragma unroll
        for (int j = 0; j < NB; ++j) {
          // a tile column past the edge re-reads column tn0 and is zeroed afterwards: a load under a
          // branch would make every wait that follows it count as if the load had not been issued
          const bool live = Nt % NB == 0 || tn0 + j < Nt;
          const float v = B[bk + u * bstep + (live ? j : 0) * bcol];
          bv[u][j] = live ? v : 0.f;
        }
      }
    };
    auto fma_group = [&](const float (&av)[KU], const float (&bv)[KU][NB]) {
      if constexpr (BF) {
#pragma unroll
        for (int u = 0; u < KU; u += 4) {
          const auto af = Io<BF16>::to_frag(f32x4{av[u], av[u + 1], av[u + 2], av[u + 3]});
#pragma unroll
          for (int j = 0; j < NB; ++j)
            Io<BF16>::mma(acc[j], af, Io<BF16>::to_frag(f32x4{bv[u][j], bv[u + 1][j], bv[u + 2][j], bv[u + 3][j]}));
        }
      } else {
#pragma unroll
        for (int u = 0; u < KU; ++u)
#pragma unroll
          for (int j = 0; j < NB; ++j)
            acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[u], bv[u][j], acc[j], 0, 0, 0);
      }
    };
    constexpr int KG = 4 * KU;
    // Operand A contiguous along k (rows 16-byte aligned): the k values of a 16-deep step are re-assigned so
    // that lane (c, g) supplies k = 4g .. 4g+3 to the four matrix instructions of the step (the pairing of
    // slot and k only has to agree between A and B).  A is then one 16-byte load per step instead of four
    // scalar ones, and so is B when it is contiguous along k too (a transposed weight matrix: its lanes
    // would otherwise touch a different cache line each).
    const bool fastA = a_cs == 1 && (a_rs & 3) == 0 && (Kd & 15) == 0 && (k0 & 3) == 0;
    if (fastA) {
      const bool vecB = b_rs == 1 && (b_cs & 3) == 0;
      const int ao = (16 * tm + c) * a_rs + k0 + 4 * g;
      const int bo = (k0 + 4 * g) * b_rs + (16 * tn0 + c) * b_cs;
      auto loadA = [&](int kk) { return *reinterpret_cast<const f32x4*>(A + ao + kk); };
      auto loadB = [&](int kk, int j) {
        // a tile column past the edge re-reads column tn0 and is zeroed afterwards (no load under a branch)
        const bool live = Nt % NB == 0 || tn0 + j < Nt;
        const float* pb = B + bo + kk * b_rs + (live ? j : 0) * bcol;
        bop v;
        if constexpr (BH) {
          v = load_rows_raw_h(reinterpret_cast<const uint16_t*>(B) + (k0 + kk) * b_rs + 16 * (tn0 + (live ? j : 0)) * b_cs,
                              b_cs, lane);
          if (!live) v = u32x2{0u, 0u};
        } else {
          if (BG) {
            v = load_rows_raw(B + (k0 + kk) * b_rs + 16 * (tn0 + (live ? j : 0)) * b_cs, b_cs, lane);
          } else if (vecB) {
            v = *reinterpret_cast<const f32x4*>(pb);
          } else {
#pragma unroll
            for (int r = 0; r < 4; ++r) v[r] = pb[r * b_rs];
          }
          if (!live) v = f32x4{0.f, 0.f, 0.f, 0.f};
        }
        return v;
      };
      auto step = [&](const f32x4& av, const bop (&bv)[NB]) {
        if constexpr (BF) {
          const auto af = Io<BF16>::to_frag(av);
#pragma unroll
          for (int j = 0; j < NB; ++j) Io<BF16>::mma(acc[j], af, bf_frag(bv[j]));
        } else if constexpr (!BH) {
#pragma unroll
          for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int j = 0; j < NB; ++j) acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[r], bv[j][r], acc[j], 0, 0, 0);
        }
      };
      // PF 16-deep steps of operands are in flight at any time (a ring of PF register buffers, refilled
      // right after use): the operands come from global memory, and with one step in flight a product
      // over 4d would pay 24 memory latencies in a row.  PF divides the step count, so no refill is
      // conditional; the scheduling barriers keep the refills where they are written.
      auto run = [&](auto pf_tag) {
        constexpr int PF = decltype(pf_tag)::value;
        f32x4 av[PF];
        bop bv[PF][NB];
#pragma unroll
        for (int u = 0; u < PF; ++u) {
          av[u] = loadA(16 * u);
#pragma unroll
          for (int j = 0; j < NB; ++j) bv[u][j] = loadB(16 * u, j);
        }
        __builtin_amdgcn_sched_barrier(0);
        int kk = 0;
#pragma nounroll
        for (; kk + 16 * PF < Kd; kk += 16 * PF) {
#pragma unroll
          for (int u = 0; u < PF; ++u) {
            if (BG) {
#pragma unroll
              for (int j = 0; j < NB; ++j) bv[u][j] = rows_to_operand(bv[u][j], lane);
            }
            step(av[u], bv[u]);
            av[u] = loadA(kk + 16 * (PF + u));
#pragma unroll
            for (int j = 0; j < NB; ++j) bv[u][j] = loadB(kk + 16 * (PF + u), j);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
#pragma unroll
        for (int u = 0; u < PF; ++u) {
          if (BG) {
#pragma unroll
            for (int j = 0; j < NB; ++j) bv[u][j] = rows_to_operand(bv[u][j], lane);
          }
          step(av[u], bv[u]);
        }
      };
      constexpr int PFMAX = NB >= 4 ? 4 : NB == 3 ? 6 : 8;
      const int nsteps = Kd >> 4;
      if (PFMAX >= 8 && nsteps % 8 == 0)
        run(std::integral_constant<int, 8>{});
      else if (PFMAX >= 6 && nsteps % 6 == 0)
        run(std::integral_constant<int, 6>{});
      else if (nsteps % 4 == 0)
        run(std::integral_constant<int, 4>{});
      else if (nsteps % 3 == 0)
        run(std::integral_constant<int, 3>{});
      else if (nsteps % 2 == 0)
        run(std::integral_constant<int, 2>{});
      else
        run(std::integral_constant<int, 1>{});
    }
    const int ngroups = fastA ? 0 : Kd / KG;
    int k = fastA ? Kd : 0;
    if (ngroups > 0) {
      fetch(avA, bvA, 0);
      // the loads of a group are issued together: left to itself the scheduler, short of registers, issues
      // them one at a time through a single register, and a product pays one memory latency per k-step
      __builtin_amdgcn_sched_barrier(0);
      int gi = 0;
#pragma nounroll
      for (; gi + 2 <= ngroups; gi += 2) {
        fetch(avB, bvB, (gi + 1) * KG);
        __builtin_amdgcn_sched_barrier(0);
        fma_group(avA, bvA);
        if (gi + 2 < ngroups) fetch(avA, bvA, (gi + 2) * KG);
        __builtin_amdgcn_sched_barrier(0);
        fma_group(avB, bvB);
      }
      if (gi < ngroups) fma_group(avA, bvA);
      k = ngroups * KG;
    }
    if constexpr (BF) {
#pragma nounroll
      for (; k < Kd; k += 16) {
        f32x4 av, bv[NB];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          av[u] = A[aoff + (k + 4 * u) * a_cs];
#pragma unroll
          for (int j = 0; j < NB; ++j) {
            const bool live = Nt % NB == 0 || tn0 + j < Nt;
            const float v = B[boff + (k + 4 * u) * b_rs + (live ? j : 0) * bcol];
            bv[j][u] = live ? v : 0.f;
          }
        }
        const auto af = Io<BF16>::to_frag(av);
#pragma unroll
        for (int j = 0; j < NB; ++j) Io<BF16>::mma(acc[j], af, Io<BF16>::to_frag(bv[j]));
      }
    } else {
#pragma nounroll
      for (; k < Kd; k += 4) {
        const float av = A[aoff + k * a_cs];
#pragma unroll
        for (int j = 0; j < NB; ++j) {
          const float bv = (tn0 + j < Nt) ? B[boff + k * b_rs + j * bcol] : 0.f;
          acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, bv, acc[j], 0, 0, 0);
        }
      }
    }
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      if (tn0 + j >= Nt) continue;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float* p = C + coff + r * ldc + 16 * j;
        if (MODE == 3)
          *p *= acc[j][r];
        else
          *p = (MODE == 2) ? -acc[j][r] : acc[j][r];
      }
    }
  }
}

template <int MODE, int NW = 4, int NB = 1, int KU = (NB >= 3 ? 2 : NB == 2 ? 4 : 8), bool BG = false>
__device__ __forceinline__ void mm_lds(float* C, int ldc, const float* A, int a_rs, int a_cs,
                                       const float* B, int b_rs, int b_cs, int Mt, int Nt, int Kd,
                                       int wave, int lane, int first = 0, int k0 = 0) {
  mm_lds_t<false, MODE, NW, NB, KU, BG>(C, ldc, A, a_rs, a_cs, B, b_rs, b_cs, Mt, Nt, Kd, wave, lane, first, k0);
}

// Rank-K update of a matrix in global memory, K = 4 * KS small (16, 32, 48):
//   C[16*Mt x 16*Nt] (+/-)= A * B   with A(m,k) = A[m*a_rs + k*a_cs], B(k,n) = B[k*b_rs + n*b_cs],
// MODE 1: C += AB, 2: C -= AB; Nt a multiple of NB.  Jobs (tile row, NB tile columns) are dealt round-robin to the
// waves as in mm_lds.  A job is a read-modify-write of its C tiles with only 4*KS*NB matrix instructions
// in between, so a wave that handled its jobs one after the other would sit through a load latency and a
// store latency per job.  Here the C tiles and operands of a wave's NEXT job are requested before the matrix
// instructions of the current one (two register sets in ping-pong).  Every load is unconditional: past a
// wave's last job the last job is re-read (and dropped), because a load under a branch makes the waits that
// follow count as if it had not been issued.
//
// FZ (needs one column block per wave, Nt / NB == NW): the product Z[16 x 16*Nt] = X[16 x 16*Mt] * C_new rides
// along.  A wave meets every tile row of its column block, and an updated tile, still in accumulator layout (lane
// (c, g), register r = C(16 tm + 4g + r, c)), is the B operand of a matrix instruction whose k slots are assigned
// as k = 4g + r; with X (LDS, contiguous along k, row stride x_rs) read 16 bytes per lane as the matching A operand,
// four more instructions per tile give the wave its complete columns of Z: the separate pass over C that the
// product would need is saved.  Z (row stride ldz) is written once at the end.
//
// Ordering, as written (two named register sets s0 / s1 in ping-pong):
//   * every job is one C tile row x NB tile columns and belongs to exactly one wave (job % NW), so no two waves
//     ever touch the same element of C, and a lane reads and writes only its own elements of a tile;
//   * a wave requests job n+1 into the idle set, then finishes job n (products, stores); the two jobs are different
//     tiles, so the loads of n+1 and the stores of n never alias;
//   * past its last job a wave requests that last job once more into the idle set, only so that the loop body is
//     the same on every trip; that load may be overtaken by the last job's own stores, and nothing reads it.
// So the result does not depend on how loads and stores of one wave interleave.  A variant that kept the sets in
// an array indexed by the trip parity (`Set s[2]`) gave wrong head_dim-128 gradients that differed from run to run,
// while the same array with three sets and this two-named-sets form never did.  Reading finds no ordering problem
// in that source either; what differs is that the indexed array is not promoted to registers at 256 VGPRs (the
// sets then live in per-lane scratch memory and are addressed with the loop-carried parity), i.e. the failure was
// in code generated for that form, which is why it is not used.  The head_dim-128 instance (256 VGPRs, a handful of
// registers spilled outside the loops) is held by a test that runs it three times and asks for identical bits.
// BF: bf16 operands, four k-steps per matrix instruction (mma16).
// FZ == 2: a second product of the same kind, Z2 = X2 * C_new (same strides as X and Z), rides along as well.
template <bool BF, int MODE, int NW, int NB, int KS, int FZ>
__device__ __forceinline__ void mm_rank_t(float* C, int ldc, const float* A, int a_rs, int a_cs, const float* B,
                                          int b_rs, int b_cs, int Mt, int Nt, int wave, int lane,
                                          const float* X, int x_rs, float* Z, int ldz, const float* Csrc = nullptr,
                                          const float* X2 = nullptr, float* Z2 = nullptr, uint16_t* Cb = nullptr) {
  static_assert(MODE == 1 || MODE == 2, "read-modify-write modes only");
  // Csrc: where the tiles of C are read from when the updated matrix goes to another buffer (same layout); the
  // ordering argument below only gets easier, since no load ever meets a store
  const float* Cin = Csrc != nullptr ? Csrc : C;
  static_assert(!BF || KS % 4 == 0, "bf16 operands: whole 16-deep steps");
  const int c = lane & 15, g = lane >> 4;
  const int nblk = Nt / NB, njobs = Mt * nblk;
  f32x4 zacc[NB], zacc2[FZ == 2 ? NB : 1];
#pragma unroll
  for (int j = 0; j < NB; ++j) zacc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < (FZ == 2 ? NB : 1); ++j) zacc2[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  // When the number of column blocks divides the number of waves, all jobs of a wave lie in one column block
  // and share their B operand: it is loaded once and kept in registers.
  const bool bfix = NW % nblk == 0;
  float bf[KS][NB];
  if (bfix) {
    const int boff = g * b_rs + (16 * (wave % nblk) * NB + c) * b_cs;
#pragma unroll
    for (int u = 0; u < KS; ++u)
#pragma unroll
      for (int j = 0; j < NB; ++j) bf[u][j] = B[boff + 4 * u * b_rs + 16 * j * b_cs];
  }
  struct Set {
    f32x4 acc[NB];
    float av[KS], bv[KS][NB];
  };
  auto request = [&](int job, Set& s) {
    const int tm = job / nblk, tn0 = (job - tm * nblk) * NB;
    const int coff = (16 * tm + 4 * g) * ldc + 16 * tn0 + c;
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) s.acc[j][r] = Cin[coff + r * ldc + 16 * j];
    const int aoff = (16 * tm + c) * a_rs + g * a_cs, boff = g * b_rs + (16 * tn0 + c) * b_cs;
#pragma unroll
    for (int u = 0; u < KS; ++u) {
      s.av[u] = A[aoff + 4 * u * a_cs];
      if (!bfix) {
#pragma unroll
        for (int j = 0; j < NB; ++j) s.bv[u][j] = B[boff + 4 * u * b_rs + 16 * j * b_cs];
      }
    }
  };
  auto finish = [&](int job, Set& s) {
    const int tm = job / nblk, tn0 = (job - tm * nblk) * NB;
    const int coff = (16 * tm + 4 * g) * ldc + 16 * tn0 + c;
    if (MODE == 2) {
#pragma unroll
      for (int u = 0; u < KS; ++u) s.av[u] = -s.av[u];
    }
    if constexpr (BF) {
#pragma unroll
      for (int u = 0; u < KS; u += 4) {
        const auto af = Io<BF16>::to_frag(f32x4{s.av[u], s.av[u + 1], s.av[u + 2], s.av[u + 3]});
#pragma unroll
        for (int j = 0; j < NB; ++j) {
          const f32x4 b4 = bfix ? f32x4{bf[u][j], bf[u + 1][j], bf[u + 2][j], bf[u + 3][j]}
                                : f32x4{s.bv[u][j], s.bv[u + 1][j], s.bv[u + 2][j], s.bv[u + 3][j]};
          Io<BF16>::mma(s.acc[j], af, Io<BF16>::to_frag(b4));
        }
      }
    } else {
#pragma unroll
      for (int u = 0; u < KS; ++u)
#pragma unroll
        for (int j = 0; j < NB; ++j)
          s.acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(s.av[u], bfix ? bf[u][j] : s.bv[u][j], s.acc[j], 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) C[coff + r * ldc + 16 * j] = s.acc[j][r];
    // Cb: a bf16 copy of the updated matrix (same layout), rounded as an operand load of the f32 matrix would be
    if (Cb != nullptr) {
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const u32x2 h = __builtin_bit_cast(u32x2, Io<BF16>::to_frag(s.acc[j]));
        Cb[coff + 16 * j] = (uint16_t)(h[0] & 0xffffu);
        Cb[coff + ldc + 16 * j] = (uint16_t)(h[0] >> 16);
        Cb[coff + 2 * ldc + 16 * j] = (uint16_t)(h[1] & 0xffffu);
        Cb[coff + 3 * ldc + 16 * j] = (uint16_t)(h[1] >> 16);
      }
    }
    if (FZ) {
      const f32x4 xv = *reinterpret_cast<const f32x4*>(X + c * x_rs + 16 * tm + 4 * g);
      if constexpr (BF) {
        const auto xf = Io<BF16>::to_frag(xv);
#pragma unroll
        for (int j = 0; j < NB; ++j) Io<BF16>::mma(zacc[j], xf, Io<BF16>::to_frag(s.acc[j]));
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
          for (int j = 0; j < NB; ++j) zacc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[r], s.acc[j][r], zacc[j], 0, 0, 0);
      }
      if constexpr (FZ == 2) {
        const f32x4 xw = *reinterpret_cast<const f32x4*>(X2 + c * x_rs + 16 * tm + 4 * g);
        if constexpr (BF) {
          const auto xf = Io<BF16>::to_frag(xw);
#pragma unroll
          for (int j = 0; j < NB; ++j) Io<BF16>::mma(zacc2[j], xf, Io<BF16>::to_frag(s.acc[j]));
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int j = 0; j < NB; ++j)
              zacc2[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(xw[r], s.acc[j][r], zacc2[j], 0, 0, 0);
        }
      }
    }
  };
  int job = wave;
  if (job >= njobs) return;
  const int last = job + ((njobs - 1 - job) / NW) * NW;  // this wave's last job
  if constexpr (BF) {
    // With bf16 operands the matrix instructions of a job no longer cover a memory round trip: two jobs are kept in
    // flight while a third is finished (three named sets; the ordering argument above holds unchanged: every request
    // of a job not yet finished reads tiles that no store in flight touches, and what is re-requested past the end is
    // never used).
    Set s0, s1, s2;
    auto at = [&](int j) { return j <= last ? j : last; };
    request(job, s0);
    request(at(job + NW), s1);
#pragma nounroll
    for (;;) {
      request(at(job + 2 * NW), s2);
      __builtin_amdgcn_sched_barrier(0);
      finish(job, s0);
      if (job + NW > last) break;
      request(at(job + 3 * NW), s0);
      __builtin_amdgcn_sched_barrier(0);
      finish(job + NW, s1);
      if (job + 2 * NW > last) break;
      request(at(job + 4 * NW), s1);
      __builtin_amdgcn_sched_barrier(0);
      finish(job + 2 * NW, s2);
      if (job + 3 * NW > last) break;
      job += 3 * NW;
    }
  } else {
    Set s0, s1;
    request(job, s0);
#pragma nounroll
    for (;;) {
      const int j1 = job + NW, j2 = job + 2 * NW;
      request(j1 <= last ? j1 : last, s1);
      __builtin_amdgcn_sched_barrier(0);
      finish(job, s0);
      if (j1 > last) break;
      request(j2 <= last ? j2 : last, s0);
      __builtin_amdgcn_sched_barrier(0);
      finish(j1, s1);
      if (j2 > last) break;
      job = j2;
    }
  }
  if (FZ) {
    const int zoff = 4 * g * ldz + 16 * (wave % nblk) * NB + c;
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) Z[zoff + r * ldz + 16 * j] = zacc[j][r];
    if constexpr (FZ == 2) {
#pragma unroll
      for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) Z2[zoff + r * ldz + 16 * j] = zacc2[j][r];
    }
  }
}

template <int MODE, int NW, int NB, int KS, int FZ = 0>
__device__ __forceinline__ void mm_rank(float* C, int ldc, const float* A, int a_rs, int a_cs, const float* B,
                                        int b_rs, int b_cs, int Mt, int Nt, int wave, int lane,
                                        const float* X = nullptr, int x_rs = 0, float* Z = nullptr, int ldz = 0) {
  mm_rank_t<false, MODE, NW, NB, KS, FZ>(C, ldc, A, a_rs, a_cs, B, b_rs, b_cs, Mt, Nt, wave, lane, X, x_rs, Z, ldz);
}

// C[16 x 16*NT] (LDS, row stride ldc) op= A[16 x Kd] * B[Kd x 16*NT] with Kd = NW * 16 * KSTEPS split over the waves:
// wave w takes k in [w*16*KSTEPS, (w+1)*16*KSTEPS) for ALL NT tile columns, leaves its partial product in
// part[w] (LDS, NW tiles of 16 rows, stride ldc), and after a barrier the partials are summed in wave order
// (deterministic).  MODE 0: C = AB, 1: C += AB, 2: C -= AB.  A is in global memory, contiguous along k (rows 16-byte
// aligned), and so is B where b_rs == 1: both are then loaded four lanes to a row (load_rows_raw).  Against one job per tile column (mm_lds) every
// element of A is fetched once instead of NT times, all NW waves work, and every operand of a wave is requested
// before its first matrix instruction.  Contains a barrier: call from all threads; the caller's next barrier
// publishes C.
// BH (with BF): B points at a bf16 copy of the matrix (uint16_t elements, same strides).
template <bool BF, int MODE, int NW, int NT, int KSTEPS, bool BH = false>
__device__ __forceinline__ void mm_splitk_t(float* C, int ldc, float* part, const float* A, int a_rs, const float* B,
                                            int b_rs, int b_cs, int wave, int lane, int tid) {
  static_assert(!BH || BF, "a bf16 copy feeds a bf16 product");
  using bop = std::conditional_t<BH, u32x2, f32x4>;
  const int c = lane & 15, g = lane >> 4;
  const int kw = wave * 16 * KSTEPS, k0 = kw + 4 * g;
  const bool vecB = b_rs == 1 && (b_cs & 3) == 0;
  f32x4 av[KSTEPS];
  bop bv[KSTEPS][NT];
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) {
    av[s] = load_rows_raw(A + kw + 16 * s, a_rs, lane);
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      if constexpr (BH) {
        const uint16_t* Bh = reinterpret_cast<const uint16_t*>(B);
        if (vecB) {
          bv[s][j] = load_rows_raw_h(Bh + (kw + 16 * s) * b_rs + 16 * j * b_cs, b_cs, lane);
        } else {
          const uint16_t* pb = Bh + (k0 + 16 * s) * b_rs + (16 * j + c) * b_cs;
          const uint32_t h0 = pb[0], h1 = pb[b_rs], h2 = pb[2 * b_rs], h3 = pb[3 * b_rs];
          bv[s][j] = u32x2{h0 | (h1 << 16), h2 | (h3 << 16)};
        }
      } else {
        const float* pb = B + (k0 + 16 * s) * b_rs + (16 * j + c) * b_cs;
        if (vecB) {
          bv[s][j] = load_rows_raw(B + (kw + 16 * s) * b_rs + 16 * j * b_cs, b_cs, lane);
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r) bv[s][j][r] = pb[r * b_rs];
        }
      }
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  // A (and B where it is contiguous along k) arrived four lanes to a row: into operand order
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) {
    av[s] = rows_to_operand(av[s], lane);
    if (vecB) {
#pragma unroll
      for (int j = 0; j < NT; ++j) bv[s][j] = rows_to_operand(bv[s][j], lane);
    }
  }
  f32x4 acc[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  if constexpr (BF) {
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      const auto af = Io<BF16>::to_frag(av[s]);
#pragma unroll
      for (int j = 0; j < NT; ++j) Io<BF16>::mma(acc[j], af, bf_frag(bv[s][j]));
    }
  } else if constexpr (!BH) {
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s)
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[s][r], bv[s][j][r], acc[j], 0, 0, 0);
  }
  float* mine = part + wave * 16 * ldc;
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int r = 0; r < 4; ++r) mine[(4 * g + r) * ldc + 16 * j + c] = acc[j][r];
  __syncthreads();
  for (int i = tid; i < 16 * 16 * NT; i += NW * 64) {
    const int row = i / (16 * NT), col = i - row * (16 * NT);
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) v += part[(w * 16 + row) * ldc + col];
    float* pc = C + row * ldc + col;
    *pc = MODE == 0 ? v : MODE == 1 ? *pc + v : *pc - v;
  }
}

template <int MODE, int NW, int NT, int KSTEPS>
__device__ __forceinline__ void mm_splitk(float* C, int ldc, float* part, const float* A, int a_rs, const float* B,
                                          int b_rs, int b_cs, int wave, int lane, int tid) {
  mm_splitk_t<false, MODE, NW, NT, KSTEPS>(C, ldc, part, A, a_rs, B, b_rs, b_cs, wave, lane, tid);
}

// The tile engine's products with the operand type fixed for a whole kernel instantiation: BF = operands rounded to
// bf16 (one v_mfma_f32_16x16x16_bf16 per 16-deep step), otherwise true f32.  Accumulation is f32 in both.
template <bool BF>
struct Eng {
  template <int MODE, int NW = 4, int NB = 1, int KU = (NB >= 3 ? 2 : NB == 2 ? 4 : 8), bool BG = false, bool BH = false>
  static __device__ __forceinline__ void lds(float* C, int ldc, const float* A, int a_rs, int a_cs, const float* B,
                                             int b_rs, int b_cs, int Mt, int Nt, int Kd, int wave, int lane,
                                             int first = 0, int k0 = 0) {
    mm_lds_t<BF, MODE, NW, NB, KU, BG, BH>(C, ldc, A, a_rs, a_cs, B, b_rs, b_cs, Mt, Nt, Kd, wave, lane, first, k0);
  }
  template <int MODE, int NW, int NB, int KS, int FZ = 0>
  static __device__ __forceinline__ void rank(float* C, int ldc, const float* A, int a_rs, int a_cs, const float* B,
                                              int b_rs, int b_cs, int Mt, int Nt, int wave, int lane,
                                              const float* X = nullptr, int x_rs = 0, float* Z = nullptr, int ldz = 0,
                                              const float* Csrc = nullptr, const float* X2 = nullptr,
                                              float* Z2 = nullptr, uint16_t* Cb = nullptr) {
    mm_rank_t<BF, MODE, NW, NB, KS, FZ>(C, ldc, A, a_rs, a_cs, B, b_rs, b_cs, Mt, Nt, wave, lane, X, x_rs, Z, ldz, Csrc, X2,
                                        Z2, Cb);
  }
  template <int MODE, int NW, int NT, int KSTEPS, bool BH = false>
  static __device__ __forceinline__ void splitk(float* C, int ldc, float* part, const float* A, int a_rs,
                                                const float* B, int b_rs, int b_cs, int wave, int lane, int tid) {
    mm_splitk_t<BF, MODE, NW, NT, KSTEPS, BH>(C, ldc, part, A, a_rs, B, b_rs, b_cs, wave, lane, tid);
  }
};

// Sum over r of p[r * stride] (+ q[r * stride]), r = 0..15, with all loads issued before the first add: written as
// a plain loop the loads are issued one at a time, each waiting for the one before.
__device__ __forceinline__ float col16_sum(const float* p, int stride) {
  float v[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) v[r] = p[r * stride];
  __builtin_amdgcn_sched_barrier(0);
  float s = 0.f;
#pragma unroll
  for (int r = 0; r < 16; ++r) s += v[r];
  return s;
}
__device__ __forceinline__ float col16_sum2(const float* p, const float* q, int stride) {
  float v[16], w[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) v[r] = p[r * stride], w[r] = q[r * stride];
  __builtin_amdgcn_sched_barrier(0);
  float s = 0.f;
#pragma unroll
  for (int r = 0; r < 16; ++r) s += v[r] + w[r];
  return s;
}

// sum over an aligned group of W lanes (W = 16 or 32) that share a token
template <int W>
__device__ __forceinline__ float rowgroup_sum(float v) {
  if (W == 32) {
    // rows 2k and 2k+1 exchanged: the two results add up to the sum of the pair in both rows
    const uint32_t u = __float_as_uint(v);
    const auto q = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    const uint32_t q0 = q[0], q1 = q[1];
    v = __uint_as_float(q0) + __uint_as_float(q1);
  }
  return row16_sum_dpp(v);
}
__device__ __forceinline__ float row16_sum(float v) { return rowgroup_sum<16>(v); }

__global__ void ttt_fill_zero_kernel(float* p, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0.f;
}
// three small buffers in one launch (the accumulated outputs of a backward: every launch costs a few microseconds
// on the stream whatever it does)
__global__ void ttt_fill_zero3_kernel(float* p0, size_t n0, float* p1, size_t n1, float* p2, size_t n2) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n0) p0[i] = 0.f;
  if (i < n1) p1[i] = 0.f;
  if (i < n2) p2[i] = 0.f;
}

// tanh-approximated GELU and its derivative (reference rust/thundercube/src/unary_ops.rs:136-173)
__device__ __forceinline__ void gelu_tanh_pair(float x, float& y, float& dy) {
  const float c = 0.7978845608f, a = 0.044715f;
  const float t = tanhf(c * (x + a * x * x * x));
  y = 0.5f * x * (1.f + t);
  dy = 0.5f * (1.f + t) + 0.5f * x * (1.f - t * t) * c * (1.f + 3.f * a * x * x);
}

// The same through the hardware exp2 / rcp (absolute error about 1e-7): for the kernels whose VALU issue
// is the bottleneck.
// y = gelu_tanh(x), dy = its derivative.  With r = 1 / (1 + exp(2u)), u = c (x + a x^3):
// (1 + tanh u) / 2 = 1 - r and 1 - tanh^2 u = 4 r (1 - r).
__device__ __forceinline__ void gelu_fast_pair(float x, float& y, float& dy) {
  const float c2 = 2.f * 0.7978845608f;
  const float x2 = x * x;
  const float u = x * __builtin_fmaf(0.044715f, x2, 1.f);
  const float e = __builtin_amdgcn_exp2f(u * (c2 * 1.4426950409f));
  const float r = __builtin_amdgcn_rcpf(1.f + e);
  const float hp = 1.f - r;
  y = x * hp;
  dy = hp * __builtin_fmaf(c2 * __builtin_fmaf(3.f * 0.044715f, x2, 1.f), x * r, 1.f);
}
__device__ __forceinline__ float gelu_fast(float x) {
  const float u = x * __builtin_fmaf(0.044715f, x * x, 1.f);
  const float e = __builtin_amdgcn_exp2f(u * (2.f * 0.7978845608f * 1.4426950409f));
  return x - x * __builtin_amdgcn_rcpf(1.f + e);
}

}  // namespace ttt
