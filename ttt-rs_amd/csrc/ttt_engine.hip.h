// Workgroup-level tile engine shared by the LDS-resident kernels (TTT-Linear backward, the
// generic TTT-Linear forward and the TTT-MLP forward).
//
// Operands are f32 arrays addressed through (row stride, column stride) pairs, in LDS or in
// global memory, so a transposed operand is just a swapped pair of strides.  All products are
// true-f32 MFMA (v_mfma_f32_16x16x4_f32): lane (c = lane%16, g = lane/16) supplies A(16tm+c, k+g)
// and B(k+g, 16tn+c) for k = 0, 4, 8, ... and owns C(16tm+4g+r, 16tn+c), r = 0..3.
#pragma once
#include "ttt_frag.hip.h"

namespace ttt {

// C[16*Mt x 16*Nt] (row-major, stride ldc)  op=  A * B over k in [k0, k0+Kd), Kd a multiple of 4.
// A(m,k) = A[m*a_rs + k*a_cs], B(k,n) = B[k*b_rs + n*b_cs].  Output tiles are dealt round-robin
// to the NW waves of the workgroup, starting at wave `first`.
// MODE 0: C = AB   1: C += AB   2: C -= AB   3: C *= AB (elementwise)
template <int MODE, int NW = 4>
__device__ __forceinline__ void mm_lds(float* C, int ldc, const float* A, int a_rs, int a_cs,
                                       const float* B, int b_rs, int b_cs, int Mt, int Nt, int Kd,
                                       int wave, int lane, int first = 0, int k0 = 0) {
  const int c = lane & 15, g = lane >> 4;
  const int ntiles = Mt * Nt;
  for (int tile = (wave - first + NW) % NW; tile < ntiles; tile += NW) {
    const int tm = tile / Nt, tn = tile - tm * Nt;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    float* Ct = C + (size_t)(16 * tm + 4 * g) * ldc + 16 * tn + c;
    if (MODE == 1 || MODE == 2) {
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[r] = (MODE == 1) ? Ct[(size_t)r * ldc] : -Ct[(size_t)r * ldc];
    }
    const float* Ap = A + (size_t)(16 * tm + c) * a_rs + (size_t)(k0 + g) * a_cs;
    const float* Bp = B + (size_t)(k0 + g) * b_rs + (size_t)(16 * tn + c) * b_cs;
#pragma unroll 4
    for (int k = 0; k < Kd; k += 4)
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(Ap[(size_t)k * a_cs], Bp[(size_t)k * b_rs], acc, 0, 0, 0);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      if (MODE == 3)
        Ct[(size_t)r * ldc] *= acc[r];
      else
        Ct[(size_t)r * ldc] = (MODE == 2) ? -acc[r] : acc[r];
    }
  }
}

// sum over an aligned group of W lanes (W = 16 or 32) that share a token
template <int W>
__device__ __forceinline__ float rowgroup_sum(float v) {
  if (W == 32) v += __shfl_xor(v, 16, 32);
  v += __shfl_xor(v, 8, W);
  v += __shfl_xor(v, 4, W);
  v += __shfl_xor(v, 2, W);
  v += __shfl_xor(v, 1, W);
  return v;
}
__device__ __forceinline__ float row16_sum(float v) { return rowgroup_sum<16>(v); }

__global__ void ttt_fill_zero_kernel(float* p, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

// tanh-approximated GELU and its derivative (reference rust/thundercube/src/unary_ops.rs:136-173)
__device__ __forceinline__ void gelu_tanh_pair(float x, float& y, float& dy) {
  const float c = 0.7978845608f, a = 0.044715f;
  const float t = tanhf(c * (x + a * x * x * x));
  y = 0.5f * x * (1.f + t);
  dy = 0.5f * (1.f + t) + 0.5f * x * (1.f - t * t) * c * (1.f + 3.f * a * x * x);
}

}  // namespace ttt
