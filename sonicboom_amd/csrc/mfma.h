// Matrix-core (MFMA) building blocks for gfx950, wave of 64 lanes.
//
// v_mfma_f32_16x16x32_bf16: D[16x16] += A[16x32] * B[32x16].  Lane l holds
//   A[row = l % 16][k = 8 * (l / 16) + 0..7]   (8 bf16 = 16 bytes)
//   B[k = 8 * (l / 16) + 0..7][col = l % 16]
//   D[row = 4 * (l / 16) + i][col = l % 16], i = 0..3
// A and B take their k elements by the same rule, so a kernel that feeds both
// operands from memory with one address formula computes the full dot product
// whatever that rule is; only the D layout shapes the epilogues.
#pragma once

#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));
typedef float floatx16_t __attribute__((ext_vector_type(16)));

__device__ __forceinline__ bf16x8_t as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8_t, v); }

__device__ __forceinline__ floatx4_t mfma16(bf16x8_t a, bf16x8_t b, floatx4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ floatx16_t mfma32(bf16x8_t a, bf16x8_t b, floatx16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// 16 bytes from global memory, or zeros when the guard fails.
__device__ __forceinline__ uint4 ld16(const void *p, bool ok) {
  return ok ? *reinterpret_cast<const uint4 *>(p) : make_uint4(0u, 0u, 0u, 0u);
}

// Two floats to two bf16 packed in 32 bits (low half first), round to nearest even: one
// v_cvt_pk_bf16_f32.
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  const bf16x2_t v = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(uint32_t, v);
}

// The maximum over the four lanes l % 16, l % 16 + 16, + 32, + 48 (the four lane groups that hold
// one column of an MFMA result), in every one of them.  Two lane swaps inside the vector unit
// (v_permlane32_swap, v_permlane16_swap: halves of the wave, then odd against even rows of 16)
// where a shuffle would go through LDS and make the wave wait for everything it has asked of it.
// Both operands of a swap are the same value, and the halves it returns are taken apart into
// variables first: written as max(p[0], p[1]) the compiler drops the maximum.
__device__ __forceinline__ float max_over_lane_groups(float v) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const auto p = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const uint32_t p0 = p[0], p1 = p[1];
  const float a = fmaxf(__builtin_bit_cast(float, p0), __builtin_bit_cast(float, p1));
  const uint32_t ua = __builtin_bit_cast(uint32_t, a);
  const auto q = __builtin_amdgcn_permlane16_swap(ua, ua, false, false);
  const uint32_t q0 = q[0], q1 = q[1];
  return fmaxf(__builtin_bit_cast(float, q0), __builtin_bit_cast(float, q1));
}
