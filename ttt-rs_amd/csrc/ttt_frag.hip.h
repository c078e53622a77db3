// Wave-level building blocks for the gfx950 TTT kernels.
//
// One wavefront (64 lanes) is viewed as c = lane & 15 (a column / token index) and
// g = lane >> 4 (a group of four rows).  All contractions are 16-row MFMAs:
//
//   D[m = 4g+r, n = c]  +=  sum_k  A[m = c, k] * B[k, n = c]
//
// and a "fragment" is the per-lane slice of one operand for sixteen values of k:
// lane (c, g) holds slots r = 0..3 standing for k = (g, r).  The pairing of slot and k is
// the same for A and B, so the k order never has to be the natural one.  This is what lets
// an accumulator tile D (rows in registers, columns across lanes) be fed back as an operand
// without moving data:
//
//   acc used as B:  B[k = 4g+r, n = c] = D[4g+r, c]      (D itself)
//   acc used as A:  A[m = c, k = 4g+r] = D[4g+r, c]      (D transposed)
//
// Feature axis permutation.  A head_dim index f is split as
//   f = 32*q + 8*gf + 4*h + r     (q = f/32, gf in 0..3, h in 0..1, r in 0..3)
// and lives in tile J = 2q+h at in-tile position p = 4*gf + r.  With this choice the eight
// features a lane needs for tiles 2q and 2q+1 are contiguous in memory
// (f = 32q + 8g .. 32q + 8g + 7), so a [16 tokens x d] activation tile is fetched with one
// 16-byte (bf16) or two 16-byte (f32) loads per lane and 32 features.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ttt {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

struct F32 {};
struct BF16 {};

// feature index of in-tile position p of tile J
__device__ __forceinline__ int feat(int J, int p) {
  return 32 * (J >> 1) + 8 * (p >> 2) + 4 * (J & 1) + (p & 3);
}

// Sum over the four lane groups g (lanes c, c+16, c+32, c+48); result in every lane.
__device__ __forceinline__ float xg_sum(float v) {
  // permlane32_swap(a, b) exchanges a's upper 32 lanes with b's lower 32 lanes; with a == b == v
  // that leaves {lo,lo} in a and {hi,hi} in b, so a + b is lo + hi in every lane.
  // permlane16_swap does the same for odd/even rows of 16 lanes.  The two results are copied
  // into scalars before the float reinterpretation: bit-casting the vector elements in place
  // makes the front end read element 0 twice.
  const uint32_t u = __float_as_uint(v);
  const auto p = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const uint32_t p0 = p[0], p1 = p[1];
  v = __uint_as_float(p0) + __uint_as_float(p1);
  const uint32_t w = __float_as_uint(v);
  const auto q = __builtin_amdgcn_permlane16_swap(w, w, false, false);
  const uint32_t q0 = q[0], q1 = q[1];
  v = __uint_as_float(q0) + __uint_as_float(q1);
  return v;
}

// Reduce four values over the four lane groups at once: returns, in lane group g, the sum over
// all groups of the g-th argument.  One 32-lane swap per pair sends each half the partner's copy of
// the value it keeps; one 16-lane swap finishes both pairs: 3 swaps + 3 adds for four sums.
__device__ __forceinline__ float xg_sum4_scatter(float a, float b, float c, float d) {
  const auto p = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(c), false, false);
  const uint32_t p0 = p[0], p1 = p[1];
  const float ac = __uint_as_float(p0) + __uint_as_float(p1);  // lower half: a, upper half: c (2 rows each)
  const auto q = __builtin_amdgcn_permlane32_swap(__float_as_uint(b), __float_as_uint(d), false, false);
  const uint32_t q0 = q[0], q1 = q[1];
  const float bd = __uint_as_float(q0) + __uint_as_float(q1);  // lower half: b, upper half: d
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(ac), __float_as_uint(bd), false, false);
  const uint32_t r0 = r[0], r1 = r[1];
  return __uint_as_float(r0) + __uint_as_float(r1);            // rows: a, b, c, d
}

// Sum over the 16 lanes of a row, in every lane: four rotations inside the row on the DPP path
// (a shuffle goes through the LDS crossbar and costs an LDS round trip per step).
__device__ __forceinline__ float row16_sum_dpp(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, false));  // row_ror:8
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xf, 0xf, false));  // row_ror:4
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x122, 0xf, 0xf, false));  // row_ror:2
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x121, 0xf, 0xf, false));  // row_ror:1
  return v;
}
// The value of the first lane (c = 0) of each row of 16 lanes, in every lane of that row.  A rotation sum leaves
// every lane with the same terms added in a different order, i.e. possibly different last bits; where all lanes
// of a row must hold the SAME number (a pivot subtracted from a whole matrix row), one lane's result is shared.
__device__ __forceinline__ float row16_first(float v) { return __shfl(v, (int)(threadIdx.x & 48u), 64); }

// Workgroup barrier for LDS exchanges only: waits for this wave's LDS traffic, not for the
// global prefetches in flight (a full __syncthreads() would drain those every mini-batch).
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// 16 bytes per lane, global -> LDS at lds_base + 16 * lane, not passing registers.  Written as assembly
// because the compiler makes every later LDS read wait for all copies it knows to be in flight (it cannot
// tell the two stage buffers apart), which would turn the prefetch into a synchronous load; the waits
// are placed by hand instead.  M0 (the LDS base of the copy) is restored.
__device__ __forceinline__ void lds_dma16(const void* src, unsigned lds_base) {
  unsigned saved;
  asm volatile(
      "s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\ts_nop 0\n\ts_mov_b32 m0, %0"
      : "=&s"(saved)
      : "v"(src), "s"(lds_base)
      : "memory");
}

// A wave-uniform pointer the compiler cannot prove uniform, moved to scalar registers.
__device__ __forceinline__ const void* uniform_ptr(const void* p) {
  const uint64_t v = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return reinterpret_cast<const void*>(((uint64_t)hi << 32) | lo);
}
// The same with the global address as wave-uniform base + 32-bit lane offset (one VGPR instead of two).
__device__ __forceinline__ void lds_dma16(const void* base, unsigned lane_off, unsigned lds_base) {
  unsigned saved;
  asm volatile(
      "s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_nop 0\n\ts_mov_b32 m0, %0"
      : "=&s"(saved)
      : "v"(lane_off), "s"(uniform_ptr(base)), "s"(lds_base)
      : "memory");
}
// One 2-byte element per lane, zero-extended to a dword at lds_base + 4 * lane.
__device__ __forceinline__ void lds_dma2(const void* src, unsigned lds_base) {
  unsigned saved;
  asm volatile(
      "s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_ushort %1, off\n\ts_nop 0\n\ts_mov_b32 m0, %0"
      : "=&s"(saved)
      : "v"(src), "s"(lds_base)
      : "memory");
}

__device__ __forceinline__ void lds_dma2(const void* base, unsigned lane_off, unsigned lds_base) {
  unsigned saved;
  asm volatile(
      "s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_ushort %1, %2\n\ts_nop 0\n\ts_mov_b32 m0, %0"
      : "=&s"(saved)
      : "v"(lane_off), "s"(uniform_ptr(base)), "s"(lds_base)
      : "memory");
}

// One dword per lane at lds_base + 4 * lane.
__device__ __forceinline__ void lds_dma4(const void* base, unsigned lane_off, unsigned lds_base) {
  unsigned saved;
  asm volatile(
      "s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2\n\ts_nop 0\n\ts_mov_b32 m0, %0"
      : "=&s"(saved)
      : "v"(lane_off), "s"(uniform_ptr(base)), "s"(lds_base)
      : "memory");
}

template <class T>
struct Io;

// ---- f32 storage, true-f32 MFMA (v_mfma_f32_16x16x4_f32: one k per lane group and step)
template <>
struct Io<F32> {
  using elem = float;
  using frag = f32x4;
  static constexpr int kBytes = 4;
  __device__ static __forceinline__ frag to_frag(f32x4 v) { return v; }
  __device__ static __forceinline__ f32x4 to_f32(frag f) { return f; }
  __device__ static __forceinline__ frag zero() { return frag{0.f, 0.f, 0.f, 0.f}; }
  __device__ static __forceinline__ void mma(f32x4& acc, frag a, frag b) {
#pragma unroll
    for (int r = 0; r < 4; ++r) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[r], b[r], acc, 0, 0, 0);
  }
  __device__ static __forceinline__ void mma2(f32x4& acc, frag a0, frag a1, frag b0, frag b1) {
    mma(acc, a0, b0);
    mma(acc, a1, b1);
  }
  // eight consecutive elements -> fragments of tiles 2q (lo) and 2q+1 (hi)
  __device__ static __forceinline__ void load8(const elem* p, bool ok, frag& lo, frag& hi) {
    if (ok) {
      lo = *reinterpret_cast<const f32x4*>(p);
      hi = *reinterpret_cast<const f32x4*>(p + 4);
    } else {
      lo = zero();
      hi = zero();
    }
  }
  __device__ static __forceinline__ void store8(elem* p, f32x4 lo, f32x4 hi) {
    *reinterpret_cast<f32x4*>(p) = lo;
    *reinterpret_cast<f32x4*>(p + 4) = hi;
  }
  __device__ static __forceinline__ float load1(const elem* p) { return *p; }
  __device__ static __forceinline__ void store1(elem* p, float v) { *p = v; }
  // what load1 reads back after store1(v)
  __device__ static __forceinline__ float rounded(float v) { return v; }
};

// ---- bf16 storage, bf16 MFMA with f32 accumulation
template <>
struct Io<BF16> {
  using elem = uint16_t;
  using frag = bf16x4;
  static constexpr int kBytes = 2;
  // two packed conversions (v_cvt_pk_bf16_f32); converting the 4-vector in one go makes the
  // compiler convert element by element and re-pack with v_perm
  __device__ static __forceinline__ frag to_frag(f32x4 v) {
    const bf16x2 lo = __builtin_convertvector(f32x2{v[0], v[1]}, bf16x2);
    const bf16x2 hi = __builtin_convertvector(f32x2{v[2], v[3]}, bf16x2);
    return __builtin_bit_cast(frag, u32x2{__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi)});
  }
  __device__ static __forceinline__ f32x4 to_f32(frag f) { return __builtin_convertvector(f, f32x4); }
  __device__ static __forceinline__ frag zero() {
    return __builtin_bit_cast(frag, u32x2{0u, 0u});
  }
  __device__ static __forceinline__ void mma(f32x4& acc, frag a, frag b) {
    acc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a),
                                                    __builtin_bit_cast(s16x4, b), acc, 0, 0, 0);
  }
  __device__ static __forceinline__ void mma2(f32x4& acc, frag a0, frag a1, frag b0, frag b1) {
    bf16x8 a = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
    bf16x8 b = __builtin_shufflevector(b0, b1, 0, 1, 2, 3, 4, 5, 6, 7);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
  }
  __device__ static __forceinline__ void load8(const elem* p, bool ok, frag& lo, frag& hi) {
    // activation tiles are read once per pass: loaded non-temporal (the `nt` bit), so that they do not displace the
    // state and the checkpoints in L2.  (The stores stay plain: a token's row is written by several waves, 64 bytes
    // each, and streaming stores are not always merged into one line on their way out: 20 % more bytes written for
    // no measurable gain.)
    u32x4 v = ok ? __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p)) : u32x4{0u, 0u, 0u, 0u};
    lo = __builtin_bit_cast(frag, u32x2{v[0], v[1]});
    hi = __builtin_bit_cast(frag, u32x2{v[2], v[3]});
  }
  __device__ static __forceinline__ void store8(elem* p, f32x4 lo, f32x4 hi) {
    u32x2 a = __builtin_bit_cast(u32x2, to_frag(lo));
    u32x2 b = __builtin_bit_cast(u32x2, to_frag(hi));
    *reinterpret_cast<u32x4*>(p) = u32x4{a[0], a[1], b[0], b[1]};
  }
  __device__ static __forceinline__ float load1(const elem* p) {
    return __builtin_bit_cast(float, static_cast<uint32_t>(*p) << 16);
  }
  __device__ static __forceinline__ void store1(elem* p, float v) {
    *p = __builtin_bit_cast(uint16_t, static_cast<__bf16>(v));
  }
  __device__ static __forceinline__ float rounded(float v) {
    return __builtin_bit_cast(float, static_cast<uint32_t>(__builtin_bit_cast(uint16_t, static_cast<__bf16>(v))) << 16);
  }
};

// Identity fragment: as B operand, B[k = 4g+r, n = c] = (c == 4g+r).  acc = mma(0, X, I) turns
// an A-side fragment X[m = c, k = (g,r)] into the accumulator tile D[4g+r, c] = X^T.
template <class T>
__device__ __forceinline__ typename Io<T>::frag identity_frag(int c, int g, float scale = 1.f) {
  f32x4 v;
#pragma unroll
  for (int r = 0; r < 4; ++r) v[r] = (c == 4 * g + r) ? scale : 0.f;
  return Io<T>::to_frag(v);
}

template <class T>
__device__ __forceinline__ typename Io<T>::frag splat_frag(float x) {
  return Io<T>::to_frag(f32x4{x, x, x, x});
}

// Rotary embedding of four consecutive features: the adjacent pairs (x0, x1) and (x2, x3) are rotated by the angles
// whose cosines and sines are cs, sn.  One routine with explicit fused multiply-adds for every kernel that rotates:
// the pass that prepares the inner loop's inputs and the forward that forms them itself must give the same bits.
__device__ __forceinline__ f32x4 rope_rotate4(f32x4 x, f32x2 cs, f32x2 sn) {
  return f32x4{__builtin_fmaf(x[0], cs[0], -(x[1] * sn[0])), __builtin_fmaf(x[1], cs[0], x[0] * sn[0]),
               __builtin_fmaf(x[2], cs[1], -(x[3] * sn[1])), __builtin_fmaf(x[3], cs[1], x[2] * sn[1])};
}
// ttt_lr_eta of a token: scale * sigmoid(z), scale = base_lr / head_dim (reference rust/layer/src/ttt.rs:205-227)
__device__ __forceinline__ float lr_gate(float z, float scale) { return scale / (1.f + __expf(-z)); }

// A launch may carry several independent problems of one shape, gridDim.y of them (windows of different layers of
// a stack that are ready at the same time: one layer's 64 units alone leave three quarters of the CUs idle).  The
// argument blocks of all of them travel as kernel arguments and workgroup (x, y) works on block y: the index is
// uniform over the workgroup, so the fields are scalar loads from the kernel-argument segment exactly as for a
// single block.
constexpr int kMaxProblems = 8;
template <class A>
struct Problems {
  A p[kMaxProblems];
};

}  // namespace ttt
