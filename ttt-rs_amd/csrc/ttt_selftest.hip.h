// Self-test of one hardware/toolchain fact the bf16 kernels depend on (see isa_check.py): a matrix instruction that
// takes the result of a matrix instruction of another shape as its accumulator input needs five wait states after
// it.  One wave computes D = A1 B1 (first shape) and D2 = A2 B2 + D (second shape) on small-integer operands derived
// from the lane index, so the expected result is exact and the host can form it itself.
//   order 0: 16x16x32 then 16x16x16, in place (D2 is D);  order 1: 16x16x16 then 16x16x32, in place;
//   order 2, 3: the same two with D2 in other registers than D
//   gap: inline assembly with exactly `gap` wait states between the two (0, 4 or 5).
// The pair written with the compiler's builtins is not part of this test: the compiler puts no wait state between
// them, which is what the build's assembly scan exists to refuse.
#pragma once
#include "ttt_frag.hip.h"

namespace ttt {

// operand element for row/column i (0..15) and reduction index k of product p (0 first, 1 second): integers in [-3, 3]
__device__ __forceinline__ float selftest_a(int p, int i, int k) { return (float)((i * 7 + k * 3 + p * 5) % 7 - 3); }
__device__ __forceinline__ float selftest_b(int p, int k, int j) { return (float)((j * 5 + k * 11 + p * 3) % 7 - 3); }

template <int ORDER, int GAP, bool INPLACE>
__device__ __forceinline__ f32x4 selftest_chain(bf16x8 A8, bf16x8 B8, bf16x4 A4, bf16x4 B4) {
  f32x4 acc, acc2;
#define TTT_ST_TAIL "s_nop 15\n\ts_nop 15\n\t"
#define TTT_ST_GAP(n) "s_nop " #n "\n\t"
#define TTT_ST_32F "v_mfma_f32_16x16x32_bf16 %0, %2, %3, 0\n\t"
#define TTT_ST_16F "v_mfma_f32_16x16x16_bf16 %0, %4, %5, 0\n\t"
#define TTT_ST_32S "v_mfma_f32_16x16x32_bf16 %0, %2, %3, %0\n\t"
#define TTT_ST_16S "v_mfma_f32_16x16x16_bf16 %0, %4, %5, %0\n\t"
#define TTT_ST_32O "v_mfma_f32_16x16x32_bf16 %1, %2, %3, %0\n\t"
#define TTT_ST_16O "v_mfma_f32_16x16x16_bf16 %1, %4, %5, %0\n\t"
#define TTT_ST_RUN(first, gap, second) \
  asm volatile(first gap second TTT_ST_TAIL : "=&v"(acc), "=&v"(acc2) : "v"(A8), "v"(B8), "v"(A4), "v"(B4))
#define TTT_ST_GAPS(first, second)                                   \
  if constexpr (GAP == 0) TTT_ST_RUN(first, "", second);             \
  else if constexpr (GAP == 4) TTT_ST_RUN(first, TTT_ST_GAP(3), second); \
  else TTT_ST_RUN(first, TTT_ST_GAP(4), second)
  if constexpr (ORDER == 0 && INPLACE) {
    TTT_ST_GAPS(TTT_ST_32F, TTT_ST_16S);
  } else if constexpr (ORDER == 1 && INPLACE) {
    TTT_ST_GAPS(TTT_ST_16F, TTT_ST_32S);
  } else if constexpr (ORDER == 0) {
    TTT_ST_GAPS(TTT_ST_32F, TTT_ST_16O);
  } else {
    TTT_ST_GAPS(TTT_ST_16F, TTT_ST_32O);
  }
#undef TTT_ST_GAPS
#undef TTT_ST_RUN
#undef TTT_ST_16O
#undef TTT_ST_32O
#undef TTT_ST_16S
#undef TTT_ST_32S
#undef TTT_ST_16F
#undef TTT_ST_32F
#undef TTT_ST_GAP
#undef TTT_ST_TAIL
  return INPLACE ? acc : acc2;
}

// out[(4g + r) * 16 + c] = D[4g + r][c]
__global__ void __launch_bounds__(64) ttt_selftest_mfma_mixed_kernel(int order, int gap, float* out) {
  const int lane = threadIdx.x & 63, c = lane & 15, g = lane >> 4;
  const int p32 = (order & 1) == 0 ? 0 : 1, p16 = 1 - p32;  // which product each shape computes
  bf16x8 A8, B8;
  bf16x4 A4, B4;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    A8[j] = (__bf16)selftest_a(p32, c, 8 * g + j);
    B8[j] = (__bf16)selftest_b(p32, 8 * g + j, c);
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    A4[j] = (__bf16)selftest_a(p16, c, 4 * g + j);
    B4[j] = (__bf16)selftest_b(p16, 4 * g + j, c);
  }
  f32x4 acc;
  const bool inplace = order < 2;
  order &= 1;
#define TTT_ST_PICK(O, I)                                                                            \
  (gap == 0 ? selftest_chain<O, 0, I>(A8, B8, A4, B4) : gap == 4 ? selftest_chain<O, 4, I>(A8, B8, A4, B4) \
                                                                 : selftest_chain<O, 5, I>(A8, B8, A4, B4))
  if (inplace) acc = order == 0 ? TTT_ST_PICK(0, true) : TTT_ST_PICK(1, true);
  else acc = order == 0 ? TTT_ST_PICK(0, false) : TTT_ST_PICK(1, false);
#undef TTT_ST_PICK
#pragma unroll
  for (int r = 0; r < 4; ++r) out[(4 * g + r) * 16 + c] = acc[r];
}

}  // namespace ttt
