// Rotary position encoding of queries and keys, and the store of keys and
// values into the paged cache, in one pass over a step's qkv rows.
//
// Rotation: /root/reference/core/src/nn/rope.cpp:26-56 — pair i of a head is
// (i, i + half), theta = float(pos) * base^(-2i/n) (the table inv_freq holds
// the second factor, computed by the caller as expf(-2i/n * logf(base))),
// divided by freq_factors[i] when a scaling table exists; cosf/sinf and the
// rotation in float.  The bias has been added before
// (/root/reference/core/src/model/emit.cpp:252-254); values are not rotated;
// the key is cached after its rotation (emit.cpp:291-293).
#include "common.cuh"

namespace {

constexpr int kMaxPairs = 256;   // rotated pairs of a head at most (head sizes up to 512)

template <typename TI, typename TQ, typename TC>
__global__ void __launch_bounds__(256)
rope_kv_kernel(TQ *__restrict__ q_out, const TI *__restrict__ qkv, int row_stride,
               const float *__restrict__ inv_freq, const float *__restrict__ freq_factors,
               int rot_dims, const int32_t *__restrict__ row_pos,
               const int32_t *__restrict__ row_seq, TC *__restrict__ k_cache,
               TC *__restrict__ v_cache, const int32_t *__restrict__ page_table, int max_pages,
               int n_pages_total, int heads_q, int heads_kv, int head_dim) {
  const int row = blockIdx.x;
  const int pos = row_pos[row];
  const TI *r = qkv + size_t(row) * row_stride;
  const int half = rot_dims / 2;
  const int q_width = heads_q * head_dim;
  const int kv_width = heads_kv * head_dim;
  TQ *qo = q_out + size_t(row) * q_width;

  // Where this row's key and value go.
  size_t slot_base = 0;
  int page_of_row = 0;
  bool store = heads_kv > 0;
  if (store) {
    const int seq = row_seq[row];
    const int lp = pos / SB_PAGE;
    const int page = (lp >= 0 && lp < max_pages) ? page_table[size_t(seq) * max_pages + lp] : -1;
    if (page < 0 || page >= n_pages_total) store = false;  // refused on the host; never write astray
    page_of_row = page < 0 ? 0 : page;
    slot_base = (size_t(page < 0 ? 0 : page) * heads_kv * SB_PAGE + size_t(pos % SB_PAGE)) * head_dim;
  }
  const size_t head_step = size_t(SB_PAGE) * head_dim;  // from one kv head to the next within a page

  // Rotated pairs of the query heads and of the key heads.  The angle of pair i is the same
  // for every head of the row: its cosine and sine are computed once and shared.
  __shared__ float cs[kMaxPairs], sn[kMaxPairs];
  if (inv_freq != nullptr) {
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
      float theta = float(pos) * inv_freq[i];
      if (freq_factors) theta = theta / freq_factors[i];
      cs[i] = cosf(theta);
      sn[i] = sinf(theta);
    }
    __syncthreads();
    const int n_pairs = (heads_q + heads_kv) * half;
#pragma unroll 4
    for (int it = threadIdx.x; it < n_pairs; it += blockDim.x) {
      const int head = it / half, i = it - head * half;
      const float c = cs[i], s = sn[i];
      const size_t e0 = size_t(head) * head_dim + i, e1 = e0 + half;
      const float x0 = ld_f(r, e0), x1 = ld_f(r, e1);
      const float y0 = x0 * c - x1 * s;
      const float y1 = x0 * s + x1 * c;
      if (head < heads_q) {
        st_f(qo, e0, y0);
        st_f(qo, e1, y1);
      } else if (store) {
        const int kh = head - heads_q;
        st_f(k_cache, slot_base + kh * head_step + i, y0);
        st_f(k_cache, slot_base + kh * head_step + i + half, y1);
      }
    }
  }
  // Elements that do not rotate (all of them without a table).
  const int first_plain = inv_freq ? rot_dims : 0;
  const int plain = head_dim - first_plain;
  for (int it = threadIdx.x; it < heads_q * plain; it += blockDim.x) {
    const int h = it / plain, d = first_plain + (it - h * plain);
    st_f(qo, size_t(h) * head_dim + d, ld_f(r, size_t(h) * head_dim + d));
  }
  if (!store) return;
  for (int it = threadIdx.x; it < heads_kv * plain; it += blockDim.x) {
    const int kh = it / plain, d = first_plain + (it - kh * plain);
    st_f(k_cache, slot_base + kh * head_step + d, ld_f(r, size_t(q_width) + kh * head_dim + d));
  }
  // Values: the cache keeps them transposed, [d][position in page], so that the matrix-core
  // kernels read eight consecutive keys of one d with one 16-byte load.
  const size_t v_base = size_t(page_of_row) * heads_kv * head_step + size_t(pos % SB_PAGE);
  for (int it = threadIdx.x; it < kv_width; it += blockDim.x) {
    const int kh = it / head_dim, d = it - kh * head_dim;
    st_f(v_cache, v_base + kh * head_step + size_t(d) * SB_PAGE, ld_f(r, size_t(q_width) + kv_width + it));
  }
}

}  // namespace

extern "C" int sb_rope_kv_store(void *q_out, int q_dtype, const void *qkv, int qkv_dtype,
                                int row_stride, const float *inv_freq, const float *freq_factors,
                                int rot_dims, const int32_t *row_pos, const int32_t *row_seq,
                                void *k_cache, void *v_cache, int cache_dtype,
                                const int32_t *page_table, int max_pages, int n_pages_total,
                                int n_rows, int heads_q, int heads_kv, int head_dim, void *stream) {
  SB_REQUIRE(qkv && row_pos, "sb_rope_kv_store: null pointer");
  SB_REQUIRE(n_rows >= 0 && heads_q >= 0 && heads_kv >= 0 && head_dim > 0 && heads_q + heads_kv > 0,
             "sb_rope_kv_store: bad sizes rows=%d heads_q=%d heads_kv=%d head_dim=%d", n_rows, heads_q,
             heads_kv, head_dim);
  SB_REQUIRE(heads_q == 0 || q_out, "sb_rope_kv_store: no buffer for the rotated queries");
  SB_REQUIRE(row_stride >= (heads_q + 2 * heads_kv) * head_dim,
             "sb_rope_kv_store: row stride %d is shorter than a qkv row of %d", row_stride,
             (heads_q + 2 * heads_kv) * head_dim);
  SB_REQUIRE(sb::valid_dtype(q_dtype) && sb::valid_dtype(qkv_dtype) && sb::valid_dtype(cache_dtype),
             "sb_rope_kv_store: unknown dtype");
  if (inv_freq) {
    SB_REQUIRE(rot_dims > 0 && rot_dims % 2 == 0 && rot_dims <= head_dim,
               "sb_rope_kv_store: rotary width %d must be even and at most head_dim %d", rot_dims,
               head_dim);
    SB_SUPPORT(rot_dims / 2 <= kMaxPairs, "sb_rope_kv_store: more than %d rotated pairs per head", kMaxPairs);
  }
  if (heads_kv > 0)
    SB_REQUIRE(k_cache && v_cache && page_table && row_seq && max_pages > 0 && n_pages_total > 0,
               "sb_rope_kv_store: a layer that stores keys needs a cache and a page table");
  if (n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
#define SB_GO(TI, TQ, TC)                                                                        \
  rope_kv_kernel<TI, TQ, TC><<<n_rows, 256, 0, s>>>(                                              \
      (TQ *)q_out, (const TI *)qkv, row_stride, inv_freq, freq_factors, rot_dims, row_pos, row_seq, \
      (TC *)k_cache, (TC *)v_cache, page_table, max_pages, n_pages_total, heads_q, heads_kv, head_dim)
  const int key = qkv_dtype * 4 + q_dtype * 2 + cache_dtype;
  switch (key) {
    case 0: SB_GO(float, float, float); break;
    case 1: SB_GO(float, float, bf16_t); break;
    case 2: SB_GO(float, bf16_t, float); break;
    case 3: SB_GO(float, bf16_t, bf16_t); break;
    case 4: SB_GO(bf16_t, float, float); break;
    case 5: SB_GO(bf16_t, float, bf16_t); break;
    case 6: SB_GO(bf16_t, bf16_t, float); break;
    default: SB_GO(bf16_t, bf16_t, bf16_t); break;
  }
#undef SB_GO
  return sb::check_launch("sb_rope_kv_store");
}
