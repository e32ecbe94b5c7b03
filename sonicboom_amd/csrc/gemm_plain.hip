// Plain tiled matrix product  Y[t,n] = sum_k X[t,k] W[n,k] (+bias) (+resid).
//
// The true 32-bit path of every projection, and the fallback of the bf16 path
// for sizes the MFMA kernels refuse.  Every output element is accumulated by
// one thread with fmaf in ascending k starting from zero, so its value does
// not depend on how many rows share the launch or where its tile lies: the
// same (row, column) gives the same bits in a whole prompt, in a single-token
// step and in any batch.  W is [out, in] row-major, the memory of a
// projection weight (/root/reference/core/include/sonicboom/quant/quantized_matmul.h:74-77);
// the bias is added after the product and the residual after the bias
// (/root/reference/core/src/model/emit.cpp:260-261, :447).
#include "common.h"

namespace {

constexpr int kTile = 64;   // rows and columns of a block's tile
constexpr int kStep = 16;   // k per stage
constexpr int kThreads = 256;

template <typename TX, typename TW, typename TO>
__global__ void __launch_bounds__(kThreads)
gemm_plain_kernel(TO *y, const TX *__restrict__ x, const TW *__restrict__ w,
                  const void *__restrict__ bias, int bias_dtype, const float *resid, int n_rows,
                  int n_out, int n_in) {
  __shared__ float xs[kStep][kTile + 4];
  __shared__ float ws[kStep][kTile + 4];
  const int t0 = blockIdx.y * kTile;
  const int n0 = blockIdx.x * kTile;
  const int tid = threadIdx.x;
  const int ty = tid / 16, tx = tid % 16;

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.0f;

  for (int k0 = 0; k0 < n_in; k0 += kStep) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = tid + i * kThreads;
      const int r = e / kStep, k = e % kStep;
      const int gk = k0 + k;
      const int gt = t0 + r, gn = n0 + r;
      xs[k][r] = (gt < n_rows && gk < n_in) ? ld_f(x, size_t(gt) * n_in + gk) : 0.0f;
      ws[k][r] = (gn < n_out && gk < n_in) ? ld_f(w, size_t(gn) * n_in + gk) : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kStep; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gt = t0 + ty * 4 + i;
    if (gt >= n_rows) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + tx * 4 + j;
      if (gn >= n_out) continue;
      float v = acc[i][j];
      if (bias) v = v + ld_dyn(bias, bias_dtype, gn);
      if (resid) v = v + resid[size_t(gt) * n_out + gn];
      st_f(y, size_t(gt) * n_out + gn, v);
    }
  }
}

template <typename TX, typename TW>
int launch_y(void *y, int y_dtype, const TX *x, const TW *w, const void *bias, int bias_dtype,
             const float *resid, int n_rows, int n_out, int n_in, hipStream_t s) {
  dim3 grid((n_out + kTile - 1) / kTile, (n_rows + kTile - 1) / kTile);
  if (y_dtype == SB_F32)
    gemm_plain_kernel<TX, TW, float><<<grid, kThreads, 0, s>>>((float *)y, x, w, bias, bias_dtype,
                                                              resid, n_rows, n_out, n_in);
  else
    gemm_plain_kernel<TX, TW, bf16_t><<<grid, kThreads, 0, s>>>((bf16_t *)y, x, w, bias, bias_dtype,
                                                               resid, n_rows, n_out, n_in);
  return sb::check_launch("sb_gemm");
}

}  // namespace

extern "C" int sb_gemm(void *y, int y_dtype, const void *x, int x_dtype, const void *w, int w_dtype,
                       const void *bias, int bias_dtype, const float *resid, int n_rows, int n_out,
                       int n_in, void *stream) {
  SB_REQUIRE(y && x && w, "sb_gemm: null pointer");
  SB_REQUIRE(n_rows >= 0 && n_out > 0 && n_in > 0, "sb_gemm: bad sizes rows=%d out=%d in=%d", n_rows,
             n_out, n_in);
  SB_REQUIRE(sb::valid_dtype(y_dtype) && sb::valid_dtype(x_dtype) && sb::valid_dtype(w_dtype) &&
                 (!bias || sb::valid_dtype(bias_dtype)),
             "sb_gemm: unknown dtype");
  SB_REQUIRE(!(resid && y_dtype != SB_F32 && (const void *)resid == y),
             "sb_gemm: a residual that aliases the output must be f32");
  SB_SUPPORT((n_rows + kTile - 1) / kTile <= 65535, "sb_gemm: more than %d rows in one call",
             65535 * kTile);
  if (n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  if (x_dtype == SB_F32 && w_dtype == SB_F32)
    return launch_y(y, y_dtype, (const float *)x, (const float *)w, bias, bias_dtype, resid, n_rows,
                    n_out, n_in, s);
  if (x_dtype == SB_BF16 && w_dtype == SB_BF16)
    return launch_y(y, y_dtype, (const bf16_t *)x, (const bf16_t *)w, bias, bias_dtype, resid, n_rows,
                    n_out, n_in, s);
  if (x_dtype == SB_F32 && w_dtype == SB_BF16)
    return launch_y(y, y_dtype, (const float *)x, (const bf16_t *)w, bias, bias_dtype, resid, n_rows,
                    n_out, n_in, s);
  return launch_y(y, y_dtype, (const bf16_t *)x, (const float *)w, bias, bias_dtype, resid, n_rows,
                  n_out, n_in, s);
}
