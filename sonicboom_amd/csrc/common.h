// Shared device helpers and the host-side error slot of the kernel library.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "sb_hip.h"

typedef uint16_t bf16_t;

// ---- bfloat16 <-> float ----------------------------------------------------
__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
  return __uint_as_float(uint32_t(v) << 16);
}
// Round to nearest even; a NaN stays a (quiet) NaN.
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return bf16_t((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return bf16_t(u >> 16);
}

__device__ __forceinline__ float ld_f(const float *p, size_t i) { return p[i]; }
__device__ __forceinline__ float ld_f(const bf16_t *p, size_t i) { return bf16_to_f32(p[i]); }
__device__ __forceinline__ void st_f(float *p, size_t i, float v) { p[i] = v; }
__device__ __forceinline__ void st_f(bf16_t *p, size_t i, float v) { p[i] = f32_to_bf16(v); }

// The gate's activation of a gated feed-forward, by the value of the products' `gated` argument:
// SB_GATE_SILU g / (1 + exp(-g)) with the full-precision expf
// (/root/reference/core/src/nn/activation.cpp:41-50); SB_GATE_GELU_TANH the tanh form of GELU,
// 0.5 g (1 + tanh(sqrt(2/pi) g (1 + 0.044715 g^2))), constants and order of :27-36.
__device__ __forceinline__ float gate_act(float g, int kind) {
  if (kind == SB_GATE_GELU_TANH)
    return 0.5f * g * (1.0f + tanhf(0.79788456080286535587989211986876f * g * (1.0f + 0.044715f * g * g)));
  return g / (1.0f + expf(-g));
}

// The rotation of one pair (x0, x1) by the angle whose cosine and sine are c and s: every product
// and sum rounded on its own (no fused multiply-add), so that every kernel that rotates a pair
// gives the same bits (/root/reference/core/src/nn/rope.cpp:46-55).
__device__ __forceinline__ void rotate_pair(float x0, float x1, float c, float s, float &y0, float &y1) {
#pragma clang fp contract(off)
  y0 = x0 * c - x1 * s;
  y1 = x0 * s + x1 * c;
}

// Value of element i of a buffer whose type is only known at run time.
__device__ __forceinline__ float ld_dyn(const void *p, int dtype, size_t i) {
  return dtype == SB_F32 ? ((const float *)p)[i] : bf16_to_f32(((const bf16_t *)p)[i]);
}

// ---- wave (64 lanes) reductions with a fixed butterfly order -----------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// ---- host side ---------------------------------------------------------------
namespace sb {

char *error_slot();  // thread-local buffer of SB_ERROR_LEN bytes
constexpr int kErrorLen = 512;

template <typename... A>
inline int fail(int code, const char *fmt, A... a) {
  snprintf(error_slot(), kErrorLen, fmt, a...);
  return code;
}
inline int fail(int code, const char *msg) {
  snprintf(error_slot(), kErrorLen, "%s", msg);
  return code;
}

inline int check_launch(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(SB_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return SB_OK;
}

// Compute units of the current device (256 on an MI355X; fewer when the GPU is partitioned), asked
// of the runtime once per device: what the launchers spread their blocks over.
inline int cu_count() {
  static int counts[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (counts[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    counts[dev] = n;
  }
  return counts[dev];
}

inline bool valid_dtype(int d) { return d == SB_F32 || d == SB_BF16; }
inline size_t dtype_size(int d) { return d == SB_F32 ? 4 : 2; }

}  // namespace sb

#define SB_REQUIRE(cond, ...)                                  \
  do {                                                         \
    if (!(cond)) return sb::fail(SB_ERR_ARGUMENT, __VA_ARGS__); \
  } while (0)
#define SB_SUPPORT(cond, ...)                                     \
  do {                                                            \
    if (!(cond)) return sb::fail(SB_ERR_UNSUPPORTED, __VA_ARGS__); \
  } while (0)
