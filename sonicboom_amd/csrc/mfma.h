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
