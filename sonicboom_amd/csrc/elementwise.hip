// Gated product, residual add, type conversion.
//
// act(g) * u with the gate's activation (SiLU with the full-precision expf, or the tanh form
// of GELU: gate_act in common.h), u the up projection
// (/root/reference/core/src/nn/activation.cpp:27-50, /root/reference/core/src/model/emit.cpp:364-374).
#include "common.h"

namespace {

template <typename TO, typename TI>
__global__ void gate_mul_kernel(TO *__restrict__ out, const TI *__restrict__ gu, int width,
                                size_t total, int gate) {
  const size_t idx = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t row = idx / width;
  const int col = int(idx - row * width);
  const TI *g_row = gu + row * size_t(2 * width);
  const float g = ld_f(g_row, col);
  const float u = ld_f(g_row, size_t(width) + col);
  st_f(out, idx, gate_act(g, gate) * u);
}

template <typename TI>
__global__ void add_into_kernel(float *__restrict__ resid, const TI *__restrict__ y, size_t n) {
  const size_t idx = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx < n) resid[idx] = ld_f(y, idx) + resid[idx];
}

template <typename TO, typename TI>
__global__ void cast_kernel(TO *__restrict__ dst, const TI *__restrict__ src, size_t n) {
  const size_t idx = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx < n) st_f(dst, idx, ld_f(src, idx));
}

inline unsigned blocks_for(size_t n, int threads) { return unsigned((n + threads - 1) / threads); }

}  // namespace

extern "C" int sb_gate_mul(void *out, int out_dtype, const void *gu, int gu_dtype, int n_rows,
                           int width, int gate, void *stream) {
  SB_REQUIRE(out && gu, "sb_gate_mul: null pointer");
  SB_REQUIRE(n_rows >= 0 && width > 0, "sb_gate_mul: bad sizes rows=%d width=%d", n_rows, width);
  SB_REQUIRE(sb::valid_dtype(out_dtype) && sb::valid_dtype(gu_dtype), "sb_gate_mul: unknown dtype");
  SB_SUPPORT(gate == SB_GATE_SILU || gate == SB_GATE_GELU_TANH, "sb_gate_mul: unknown gate activation %d", gate);
  const size_t total = size_t(n_rows) * width;
  if (total == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  const unsigned nb = blocks_for(total, 256);
#define SB_GO(TO, TI) gate_mul_kernel<TO, TI><<<nb, 256, 0, s>>>((TO *)out, (const TI *)gu, width, total, gate)
  if (out_dtype == SB_F32 && gu_dtype == SB_F32) SB_GO(float, float);
  else if (out_dtype == SB_BF16 && gu_dtype == SB_F32) SB_GO(bf16_t, float);
  else if (out_dtype == SB_BF16 && gu_dtype == SB_BF16) SB_GO(bf16_t, bf16_t);
  else SB_GO(float, bf16_t);
#undef SB_GO
  return sb::check_launch("sb_gate_mul");
}

extern "C" int sb_silu_mul(void *out, int out_dtype, const void *gu, int gu_dtype, int n_rows,
                           int width, void *stream) {
  return sb_gate_mul(out, out_dtype, gu, gu_dtype, n_rows, width, SB_GATE_SILU, stream);
}

extern "C" int sb_add_into(float *resid, const void *y, int y_dtype, size_t n, void *stream) {
  SB_REQUIRE(resid && y, "sb_add_into: null pointer");
  SB_REQUIRE(sb::valid_dtype(y_dtype), "sb_add_into: unknown dtype");
  if (n == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  const unsigned nb = blocks_for(n, 256);
  if (y_dtype == SB_F32) add_into_kernel<float><<<nb, 256, 0, s>>>(resid, (const float *)y, n);
  else add_into_kernel<bf16_t><<<nb, 256, 0, s>>>(resid, (const bf16_t *)y, n);
  return sb::check_launch("sb_add_into");
}

extern "C" int sb_cast(void *dst, int dst_dtype, const void *src, int src_dtype, size_t n,
                       void *stream) {
  SB_REQUIRE(dst && src, "sb_cast: null pointer");
  SB_REQUIRE(sb::valid_dtype(dst_dtype) && sb::valid_dtype(src_dtype), "sb_cast: unknown dtype");
  if (n == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  const unsigned nb = blocks_for(n, 256);
#define SB_GO(TO, TI) cast_kernel<TO, TI><<<nb, 256, 0, s>>>((TO *)dst, (const TI *)src, n)
  if (dst_dtype == SB_F32 && src_dtype == SB_F32) SB_GO(float, float);
  else if (dst_dtype == SB_BF16 && src_dtype == SB_F32) SB_GO(bf16_t, float);
  else if (dst_dtype == SB_BF16 && src_dtype == SB_BF16) SB_GO(bf16_t, bf16_t);
  else SB_GO(float, bf16_t);
#undef SB_GO
  return sb::check_launch("sb_cast");
}

// ---- measurement: how fast can this GPU stream memory? ---------------------------------------
namespace {
__global__ void __launch_bounds__(256)
read_probe_kernel(uint32_t *__restrict__ sink, const uint4 *__restrict__ src, size_t n_vec) {
  const size_t stride = size_t(gridDim.x) * blockDim.x;
  size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
  uint32_t acc = 0;
  for (; i + 3 * stride < n_vec; i += 4 * stride) {
    const uint4 a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
    acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
  }
  for (; i < n_vec; i += stride) {
    const uint4 a = src[i];
    acc ^= a.x ^ a.y ^ a.z ^ a.w;
  }
  if (acc == 0x9e3779b9u) sink[0] = acc;   // keeps the loads alive; practically never taken
}
}  // namespace

// Reads `bytes` (a multiple of 16) from src once with `blocks` blocks of 256 threads, 16 bytes
// per load, four loads in flight per thread.  For timing the memory system; writes nothing
// worth reading.
extern "C" int sb_read_probe(void *sink, const void *src, size_t bytes, int blocks, void *stream) {
  SB_REQUIRE(sink && src && blocks > 0, "sb_read_probe: bad arguments");
  read_probe_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>((uint32_t *)sink, (const uint4 *)src, bytes / 16);
  return sb::check_launch("sb_read_probe");
}
