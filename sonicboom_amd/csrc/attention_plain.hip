// Attention over the paged cache, one wave per (row, query head): the true
// 32-bit path, and the path of the bf16 engine for sizes its MFMA kernels
// refuse.
//
// Formula: /root/reference/core/src/nn/attention.cpp:26-105 and :121-181 —
// query head h reads kv head h / group; s_j = dot(q, k_j) * scale; a key is
// visible when j <= p and (window == 0 or p - j < window); softmax with the
// maximum subtracted; a row without visible keys is zero.
//
// The cache holds keys as [page][kv head][position][d] and values transposed,
// [page][kv head][d][position].
//
// Keys are taken 64 at a time in chunks at absolute positions [64c, 64c+64),
// lane l owning key 64c+l.  The running maximum, the running sum and the
// output accumulate chunk after chunk in ascending c, and inside a chunk in
// ascending key, so the arithmetic of a row is a function of its position and
// window alone: it does not change with the batch, with the cut of the prompt
// into steps or with the physical pages.
#include "common.h"

namespace {

constexpr int kMaxHeadDim = 256;

template <typename TA, typename TC>
__global__ void __launch_bounds__(64)
attention_plain_kernel(TA *__restrict__ out, const TA *__restrict__ q, int q_stride,
                       const TC *__restrict__ k_cache, const TC *__restrict__ v_cache,
                       const int32_t *__restrict__ page_table, int max_pages, int n_pages_total,
                       const int32_t *__restrict__ row_pos, const int32_t *__restrict__ row_seq,
                       int heads_q, int heads_kv, int head_dim, float scale, int window) {
  __shared__ float qs[kMaxHeadDim];
  __shared__ float ps[64];
  const int row = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int pos = row_pos[row], seq = row_seq[row];
  const int kvh = h / (heads_q / heads_kv);
  for (int d = lane; d < head_dim; d += 64) qs[d] = ld_f(q, size_t(row) * q_stride + size_t(h) * head_dim + d);
  __syncthreads();

  const int lo = (window > 0 && pos >= window) ? pos - window + 1 : 0;
  const float neg_inf = -__builtin_inff();
  float m = neg_inf, l = 0.0f;
  float o[kMaxHeadDim / 64] = {0.0f, 0.0f, 0.0f, 0.0f};

  for (int c = lo / SB_PAGE; c <= pos / SB_PAGE; ++c) {
    const int page = c < max_pages ? page_table[size_t(seq) * max_pages + c] : -1;
    if (page < 0 || page >= n_pages_total) continue;  // uniform over the wave
    const size_t base = (size_t(page) * heads_kv + kvh) * SB_PAGE * head_dim;
    const TC *kp = k_cache + base;
    const TC *vp = v_cache + base;
    const int j = c * SB_PAGE + lane;
    const bool visible = j >= lo && j <= pos;
    float s = neg_inf;
    if (visible) {
      float dot = 0.0f;
      for (int d = 0; d < head_dim; ++d) dot = fmaf(qs[d], ld_f(kp, sb_key_index(lane, d, head_dim)), dot);
      s = dot * scale;
    }
    const float cm = wave_max(s);
    const float m_new = fmaxf(m, cm);
    const float p = visible ? expf(s - m_new) : 0.0f;
    const float alpha = expf(m - m_new);  // 0 for the first chunk
    l = l * alpha + wave_sum(p);
    ps[lane] = p;
    __syncthreads();
    const int j0 = max(lo - c * SB_PAGE, 0), j1 = min(pos - c * SB_PAGE, SB_PAGE - 1);
#pragma unroll
    for (int i = 0; i < kMaxHeadDim / 64; ++i) {
      const int d = lane + 64 * i;
      if (d < head_dim) {
        float acc = o[i] * alpha;
        for (int jj = j0; jj <= j1; ++jj) acc = fmaf(ps[jj], ld_f(vp, sb_value_index(d, jj)), acc);
        o[i] = acc;
      }
    }
    __syncthreads();
    m = m_new;
  }
  const float inv = l > 0.0f ? 1.0f / l : 0.0f;
#pragma unroll
  for (int i = 0; i < kMaxHeadDim / 64; ++i) {
    const int d = lane + 64 * i;
    if (d < head_dim) st_f(out, size_t(row) * heads_q * head_dim + size_t(h) * head_dim + d, o[i] * inv);
  }
}

}  // namespace

extern "C" int sb_attention(void *out, const void *q, int act_dtype, int q_stride, const void *k_cache,
                            const void *v_cache, int cache_dtype, const int32_t *page_table,
                            int max_pages, int n_pages_total, const int32_t *row_pos,
                            const int32_t *row_seq, int n_rows, int heads_q, int heads_kv,
                            int head_dim, float scale, int window, void *stream) {
  SB_REQUIRE(out && q && k_cache && v_cache && page_table && row_pos && row_seq,
             "sb_attention: null pointer");
  SB_REQUIRE(n_rows >= 0 && heads_q > 0 && heads_kv > 0 && head_dim > 0 && max_pages > 0 &&
                 n_pages_total > 0 && window >= 0,
             "sb_attention: bad sizes rows=%d heads_q=%d heads_kv=%d head_dim=%d", n_rows, heads_q,
             heads_kv, head_dim);
  SB_REQUIRE(heads_q % heads_kv == 0, "sb_attention: %d query heads are not a multiple of %d kv heads",
             heads_q, heads_kv);
  SB_REQUIRE(q_stride >= heads_q * head_dim, "sb_attention: query stride %d shorter than %d", q_stride,
             heads_q * head_dim);
  SB_REQUIRE(sb::valid_dtype(act_dtype) && sb::valid_dtype(cache_dtype), "sb_attention: unknown dtype");
  SB_SUPPORT(head_dim <= kMaxHeadDim, "sb_attention: head size %d is above the limit of %d", head_dim,
             kMaxHeadDim);
  SB_SUPPORT(heads_q <= 65535, "sb_attention: more than 65535 query heads");
  if (n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  dim3 grid(n_rows, heads_q);
#define SB_GO(TA, TC)                                                                           \
  attention_plain_kernel<TA, TC><<<grid, 64, 0, s>>>(                                            \
      (TA *)out, (const TA *)q, q_stride, (const TC *)k_cache, (const TC *)v_cache, page_table,  \
      max_pages, n_pages_total, row_pos, row_seq, heads_q, heads_kv, head_dim, scale, window)
  if (act_dtype == SB_F32 && cache_dtype == SB_F32) SB_GO(float, float);
  else if (act_dtype == SB_BF16 && cache_dtype == SB_BF16) SB_GO(bf16_t, bf16_t);
  else if (act_dtype == SB_F32 && cache_dtype == SB_BF16) SB_GO(float, bf16_t);
  else SB_GO(bf16_t, float);
#undef SB_GO
  return sb::check_launch("sb_attention");
}
