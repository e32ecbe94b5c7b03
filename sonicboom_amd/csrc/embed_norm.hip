// Token embedding lookup and RMS norm.
//
// Formulas: /root/reference/core/src/model/emit.cpp:237-248 (row lookup, no
// scale), /root/reference/core/src/nn/norm.cpp:25-42 (eps inside the root,
// product order (x*inv)*w).  The mean of squares is accumulated in double, as
// the reference's default reduction does (/root/reference/core/src/nn/cpu_reduce.h:55-57).
#include "common.cuh"

namespace {

template <typename TT>
__global__ void embed_kernel(float *__restrict__ out, const TT *__restrict__ table,
                             const int32_t *__restrict__ ids, int width, int vocab) {
  const int row = blockIdx.x;
  const int id = ids[row];
  float *o = out + size_t(row) * width;
  if (id < 0 || id >= vocab) {
    for (int i = threadIdx.x; i < width; i += blockDim.x) o[i] = __uint_as_float(0x7fc00000u);
    return;
  }
  const TT *src = table + size_t(id) * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) o[i] = ld_f(src, i);
}

constexpr int kNormThreads = 256;
constexpr int kNormKeep = 8;   // float4 groups of a row that a thread keeps in registers

// One block per row.  A thread takes float4 groups tid, tid + 256, ...; all of a thread's loads
// are issued before the first is used, and the first kNormKeep groups stay in registers for the
// second pass.  The squares are summed in double: per thread in ascending order, then by a
// fixed butterfly over the wave, then wave by wave.
template <typename TO>
__global__ void __launch_bounds__(kNormThreads)
rmsnorm_kernel(TO *__restrict__ y, const float *__restrict__ x, const void *__restrict__ w,
               int w_dtype, const int32_t *__restrict__ rows, int width, float eps) {
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  const float *xr = x + size_t(src) * width;
  TO *yr = y + size_t(r) * width;
  const int tid = threadIdx.x;
  const bool vec = (width % 4 == 0) && (reinterpret_cast<uintptr_t>(xr) % 16 == 0);
  const int n_groups = vec ? width / 4 : 0;

  float4 keep[kNormKeep];
  double part = 0.0;
#pragma unroll
  for (int i = 0; i < kNormKeep; ++i) {
    const int g = tid + i * kNormThreads;
    keep[i] = g < n_groups ? reinterpret_cast<const float4 *>(xr)[g] : make_float4(0.f, 0.f, 0.f, 0.f);
  }
#pragma unroll
  for (int i = 0; i < kNormKeep; ++i)
    part += double(keep[i].x * keep[i].x) + double(keep[i].y * keep[i].y) + double(keep[i].z * keep[i].z) +
            double(keep[i].w * keep[i].w);
  // what does not fit the registers, or a row that cannot be read in groups of four
  const int tail0 = vec ? min(n_groups, kNormKeep * kNormThreads) * 4 : 0;
  for (int i = tail0 + tid; i < width; i += kNormThreads) {
    const float v = xr[i];
    part += double(v * v);
  }
  part = wave_sum(part);
  __shared__ double wave_part[kNormThreads / 64];
  if ((tid & 63) == 0) wave_part[tid >> 6] = part;
  __syncthreads();
  double total = 0.0;
#pragma unroll
  for (int k = 0; k < kNormThreads / 64; ++k) total += wave_part[k];
  const float mean = float(total / double(width));
  const float inv = 1.0f / sqrtf(mean + eps);

#pragma unroll
  for (int i = 0; i < kNormKeep; ++i) {
    const int g = tid + i * kNormThreads;
    if (g < n_groups) {
      const float v[4] = {keep[i].x, keep[i].y, keep[i].z, keep[i].w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float o = v[e] * inv;
        if (w) o = o * ld_dyn(w, w_dtype, g * 4 + e);
        st_f(yr, g * 4 + e, o);
      }
    }
  }
  for (int i = tail0 + tid; i < width; i += kNormThreads) {
    float o = xr[i] * inv;
    if (w) o = o * ld_dyn(w, w_dtype, i);
    st_f(yr, i, o);
  }
}

}  // namespace

extern "C" int sb_embed(float *out, const void *table, int table_dtype, const int32_t *ids,
                        int n_rows, int width, int vocab, void *stream) {
  SB_REQUIRE(out && table && ids, "sb_embed: null pointer");
  SB_REQUIRE(n_rows >= 0 && width > 0 && vocab > 0, "sb_embed: bad sizes rows=%d width=%d vocab=%d",
             n_rows, width, vocab);
  SB_REQUIRE(sb::valid_dtype(table_dtype), "sb_embed: unknown table dtype %d", table_dtype);
  if (n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  if (table_dtype == SB_F32)
    embed_kernel<float><<<n_rows, 256, 0, s>>>(out, (const float *)table, ids, width, vocab);
  else
    embed_kernel<bf16_t><<<n_rows, 256, 0, s>>>(out, (const bf16_t *)table, ids, width, vocab);
  return sb::check_launch("sb_embed");
}

extern "C" int sb_rmsnorm(void *y, int out_dtype, const float *x, const void *w, int w_dtype,
                          const int32_t *rows, int n_rows, int width, float eps, void *stream) {
  SB_REQUIRE(y && x, "sb_rmsnorm: null pointer");
  SB_REQUIRE(n_rows >= 0 && width > 0, "sb_rmsnorm: bad sizes rows=%d width=%d", n_rows, width);
  SB_REQUIRE(sb::valid_dtype(out_dtype) && (!w || sb::valid_dtype(w_dtype)),
             "sb_rmsnorm: unknown dtype");
  SB_REQUIRE(eps >= 0.0f, "sb_rmsnorm: eps must not be negative");
  if (n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  if (out_dtype == SB_F32)
    rmsnorm_kernel<float><<<n_rows, kNormThreads, 0, s>>>((float *)y, x, w, w_dtype, rows, width, eps);
  else
    rmsnorm_kernel<bf16_t><<<n_rows, kNormThreads, 0, s>>>((bf16_t *)y, x, w, w_dtype, rows, width, eps);
  return sb::check_launch("sb_rmsnorm");
}
