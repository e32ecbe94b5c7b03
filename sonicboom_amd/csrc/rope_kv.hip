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
#include "common.h"

namespace {

constexpr int kMaxPairs = 256;   // rotated pairs of a head at most (head sizes up to 512)
constexpr int kMaxSlices = 8;    // K slices of the projection that are added on load

// Element e of a qkv row: the sum of the product's K slices in ascending order, then the bias.
// SLICES: length of the unrolled loop (1, 4 or 8: at least n_slices).
template <int SLICES, typename TI>
__device__ __forceinline__ float qkv_at(const TI *r, size_t e, int n_slices, size_t slice_stride,
                                        const float *bias) {
  float p[SLICES];
#pragma unroll
  for (int s = 0; s < SLICES; ++s) p[s] = s < n_slices ? ld_f(r + s * slice_stride, e) : 0.f;
  float v = p[0];
#pragma unroll
  for (int s = 1; s < SLICES; ++s)
    if (s < n_slices) v += p[s];
  if (bias) v = v + bias[e];
  return v;
}

// Block (row, head group): heads [hpb y, hpb (y + 1)) of the row's heads_q query heads, heads_kv
// key heads and heads_kv value heads, in that order.  Few rows (decode): groups of four heads,
// to have enough blocks; many rows (prefill): all heads of a row in one block, so that the
// row's cosines and sines and its page look-up are worked out once and every thread has
// several pairs to move.
template <typename TI, typename TQ, typename TC, int SLICES>
__global__ void __launch_bounds__(256)
rope_kv_kernel(TQ *__restrict__ q_out, const TI *__restrict__ qkv, int row_stride, int n_slices,
               size_t slice_stride, const float *__restrict__ bias,
               const float *__restrict__ inv_freq, const float *__restrict__ freq_factors,
               int rot_dims, const int32_t *__restrict__ row_pos,
               const int32_t *__restrict__ row_seq, TC *__restrict__ k_cache,
               TC *__restrict__ v_cache, const int32_t *__restrict__ page_table, int max_pages,
               int n_pages_total, int heads_q, int heads_kv, int head_dim, int heads_per_block) {
  const int row = blockIdx.x;
  const int pos = row_pos[row];
  const TI *r = qkv + size_t(row) * row_stride;
  const int half = rot_dims / 2;
  const int q_width = heads_q * head_dim;
  TQ *qo = q_out + size_t(row) * q_width;
  const int n_heads = heads_q + 2 * heads_kv;
  const int h_begin = blockIdx.y * heads_per_block, h_end = min(h_begin + heads_per_block, n_heads);

  const bool rotate = inv_freq != nullptr;
  const int first_plain = rotate ? rot_dims : 0;
  const int plain = head_dim - first_plain;
  // work items of a head: `half` rotated pairs, then `plain` elements that are copied
  const int per_head = (rotate ? half : 0) + plain;
  const int n_items = (h_end - h_begin) * per_head;

  // The operands of a thread's first rotated pair do not depend on the position: their loads go
  // out before the cosines are worked out, not after.
  float pre0 = 0.f, pre1 = 0.f;
  bool preloaded = false;
  if (rotate && int(threadIdx.x) < n_items) {
    const int head = h_begin + int(threadIdx.x) / per_head, w = int(threadIdx.x) % per_head;
    if (head < heads_q + heads_kv && w < half) {
      const size_t hoff = size_t(head) * head_dim;
      pre0 = qkv_at<SLICES>(r, hoff + w, n_slices, slice_stride, bias);
      pre1 = qkv_at<SLICES>(r, hoff + w + half, n_slices, slice_stride, bias);
      preloaded = true;
    }
  }

  // Where this row's key and value go.
  int page_of_row = 0;
  bool store = heads_kv > 0;
  if (store) {
    const int seq = row_seq[row];
    const int lp = pos / SB_PAGE;
    const int page = (lp >= 0 && lp < max_pages) ? page_table[size_t(seq) * max_pages + lp] : -1;
    if (page < 0 || page >= n_pages_total) store = false;  // refused on the host; never write astray
    page_of_row = page < 0 ? 0 : page;
  }
  const size_t head_step = size_t(SB_PAGE) * head_dim;  // from one kv head to the next within a page
  const size_t page_base = size_t(page_of_row) * heads_kv * head_step;
  const int slot = pos % SB_PAGE;      // keys [slot][d], values [d][slot], in the cache's order of groups

  // The angle of pair i is the same for every head of the row: cosine and sine once per block,
  // the cosines by one half of the threads that take part, the sines by the other.
  __shared__ float cs[kMaxPairs], sn[kMaxPairs];
  if (rotate && h_begin < heads_q + heads_kv) {
    for (int j = threadIdx.x; j < 2 * half; j += blockDim.x) {
      const int i = j < half ? j : j - half;
      float theta = float(pos) * inv_freq[i];
      if (freq_factors) theta = theta / freq_factors[i];
      if (j < half) cs[i] = cosf(theta);
      else sn[i] = sinf(theta);
    }
  }
  __syncthreads();
#pragma unroll 2
  for (int it = threadIdx.x; it < n_items; it += blockDim.x) {
    const int head = h_begin + it / per_head, w = it % per_head;
    const size_t hoff = size_t(head) * head_dim;      // heads lie back to back in the qkv row
    if (head >= heads_q + heads_kv) {
      // a value head: every element is copied, transposed into the page
      if (!store) continue;
      const int kh = head - heads_q - heads_kv;
#pragma unroll 1
      for (int d = w; d < head_dim; d += per_head)
        st_f(v_cache, page_base + kh * head_step + sb_value_index(d, slot),
             qkv_at<SLICES>(r, hoff + d, n_slices, slice_stride, bias));
      continue;
    }
    const bool is_q = head < heads_q;
    if (!is_q && !store) continue;
    const int kh = head - heads_q;
    if (rotate && w < half) {
      const int i = w;
      const float c = cs[i], sv = sn[i];
      const bool have = preloaded && it == int(threadIdx.x);
      const float x0 = have ? pre0 : qkv_at<SLICES>(r, hoff + i, n_slices, slice_stride, bias);
      const float x1 = have ? pre1 : qkv_at<SLICES>(r, hoff + i + half, n_slices, slice_stride, bias);
      float y0, y1;
      rotate_pair(x0, x1, c, sv, y0, y1);
      if (is_q) {
        st_f(qo, hoff + i, y0);
        st_f(qo, hoff + i + half, y1);
      } else {
        st_f(k_cache, page_base + kh * head_step + sb_key_index(slot, i, head_dim), y0);
        st_f(k_cache, page_base + kh * head_step + sb_key_index(slot, i + half, head_dim), y1);
      }
    } else {
      const int d = first_plain + (w - (rotate ? half : 0));
      const float v = qkv_at<SLICES>(r, hoff + d, n_slices, slice_stride, bias);
      if (is_q) st_f(qo, hoff + d, v);
      else st_f(k_cache, page_base + kh * head_step + sb_key_index(slot, d, head_dim), v);
    }
  }
}

// Many rows (a prompt step's qkv rows as the tiled product leaves them, whole or in K slices,
// with or without a bias still to add), bfloat16 queries and cache, head size and rotary width in
// 16s: a thread moves eight pairs at a time, 16 bytes per load and store instead of two or four.
// One block per row.  The arithmetic is rope_kv_kernel's (slices added in ascending order, then
// the bias, every element through float, the same rotate_pair), so the bits are the same.
__device__ __forceinline__ void load_eight(float (&f)[8], const float *p) {
  const float4 a = *reinterpret_cast<const float4 *>(p), b = *reinterpret_cast<const float4 *>(p + 4);
  f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
}
__device__ __forceinline__ void load_eight(float (&f)[8], const bf16_t *p) {
  const uint4 u = *reinterpret_cast<const uint4 *>(p);
  const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    f[2 * e] = bf16_to_f32(bf16_t(w[e] & 0xffffu));
    f[2 * e + 1] = bf16_to_f32(bf16_t(w[e] >> 16));
  }
}
// Eight elements from e on of a qkv row, as qkv_at gives them one by one.
template <int SLICES, typename TI>
__device__ __forceinline__ void qkv_eight(float (&f)[8], const TI *r, size_t e, int n_slices, size_t slice_stride,
                                          const float *bias) {
  float part[SLICES][8];
#pragma unroll
  for (int s = 0; s < SLICES; ++s)
    if (s == 0 || s < n_slices) load_eight(part[s], r + s * slice_stride + e);
#pragma unroll
  for (int i = 0; i < 8; ++i) f[i] = part[0][i];
#pragma unroll
  for (int s = 1; s < SLICES; ++s)
    if (s < n_slices) {
#pragma unroll
      for (int i = 0; i < 8; ++i) f[i] += part[s][i];
    }
  if (bias) {
    float b[8];
    load_eight(b, bias + e);
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = f[i] + b[i];
  }
}
template <typename TI, int SLICES>
__global__ void __launch_bounds__(256)
rope_kv_rows_kernel(bf16_t *__restrict__ q_out, const TI *__restrict__ qkv, int row_stride, int n_slices,
                    size_t slice_stride, const float *__restrict__ bias,
                    const float *__restrict__ inv_freq, const float *__restrict__ freq_factors, int rot_dims,
                    const int32_t *__restrict__ row_pos, const int32_t *__restrict__ row_seq,
                    bf16_t *__restrict__ k_cache, bf16_t *__restrict__ v_cache,
                    const int32_t *__restrict__ page_table, int max_pages, int n_pages_total, int heads_q,
                    int heads_kv, int head_dim) {
  const int row = blockIdx.x;
  const int pos = row_pos[row];
  const TI *r = qkv + size_t(row) * row_stride;
  bf16_t *qo = q_out + size_t(row) * heads_q * head_dim;
  const bool rotate = inv_freq != nullptr;
  const int half = rotate ? rot_dims / 2 : 0;
  int page_of_row = 0;
  bool store = heads_kv > 0;
  if (store) {
    const int seq = row_seq[row];
    const int lp = pos / SB_PAGE;
    const int page = (lp >= 0 && lp < max_pages) ? page_table[size_t(seq) * max_pages + lp] : -1;
    if (page < 0 || page >= n_pages_total) store = false;  // refused on the host; never write astray
    page_of_row = page < 0 ? 0 : page;
  }
  const size_t head_step = size_t(SB_PAGE) * head_dim;
  const size_t page_base = size_t(page_of_row) * heads_kv * head_step;
  const int slot = pos % SB_PAGE;
  __shared__ float cs[kMaxPairs], sn[kMaxPairs];
  for (int j = threadIdx.x; j < 2 * half; j += blockDim.x) {
    const int i = j < half ? j : j - half;
    float theta = float(pos) * inv_freq[i];
    if (freq_factors) theta = theta / freq_factors[i];
    if (j < half) cs[i] = cosf(theta);
    else sn[i] = sinf(theta);
  }
  __syncthreads();
  auto pack = [](const float (&f)[8]) {
    return make_uint4(uint32_t(f32_to_bf16(f[0])) | uint32_t(f32_to_bf16(f[1])) << 16,
                      uint32_t(f32_to_bf16(f[2])) | uint32_t(f32_to_bf16(f[3])) << 16,
                      uint32_t(f32_to_bf16(f[4])) | uint32_t(f32_to_bf16(f[5])) << 16,
                      uint32_t(f32_to_bf16(f[6])) | uint32_t(f32_to_bf16(f[7])) << 16);
  };
  // queries and keys: per head half / 8 groups of eight pairs, then (head_dim - rot_dims) / 8 groups copied
  const int pair_groups = half / 8, per_head = pair_groups + (head_dim - 2 * half) / 8;
  const int n_qk = (heads_q + (store ? heads_kv : 0)) * per_head;
  for (int it = threadIdx.x; it < n_qk; it += blockDim.x) {
    const int head = it / per_head, w = it % per_head;
    const size_t src = size_t(head) * head_dim;           // where the head starts in the row
    // a group of eight (d0 a multiple of 8) goes to the query row as it is, into the cache at the
    // group's place in the cache's order
    const bool is_q = head < heads_q;
    bf16_t *dst = is_q ? qo + size_t(head) * head_dim : k_cache + page_base + size_t(head - heads_q) * head_step;
    auto at = [&](int d0) { return is_q ? size_t(d0) : sb_key_index(slot, d0, head_dim); };
    if (w < pair_groups) {
      const int i0 = w * 8;
      float lo[8], hi[8], y0[8], y1[8];
      qkv_eight<SLICES>(lo, r, src + i0, n_slices, slice_stride, bias);
      qkv_eight<SLICES>(hi, r, src + i0 + half, n_slices, slice_stride, bias);
#pragma unroll
      for (int e = 0; e < 8; ++e) rotate_pair(lo[e], hi[e], cs[i0 + e], sn[i0 + e], y0[e], y1[e]);
      *reinterpret_cast<uint4 *>(dst + at(i0)) = pack(y0);
      *reinterpret_cast<uint4 *>(dst + at(i0 + half)) = pack(y1);
    } else {
      const int d0 = 2 * half + (w - pair_groups) * 8;
      float v[8];
      qkv_eight<SLICES>(v, r, src + d0, n_slices, slice_stride, bias);
      *reinterpret_cast<uint4 *>(dst + at(d0)) = pack(v);
    }
  }
  // values: eight elements a time, each to its own row of the transposed page
  if (!store) return;
  const int groups = head_dim / 8;
  for (int it = threadIdx.x; it < heads_kv * groups; it += blockDim.x) {
    const int kh = it / groups, d0 = (it % groups) * 8;
    float v[8];
    qkv_eight<SLICES>(v, r, size_t(heads_q + heads_kv + kh) * head_dim + d0, n_slices, slice_stride, bias);
#pragma unroll
    for (int e = 0; e < 8; ++e) v_cache[page_base + kh * head_step + sb_value_index(d0 + e, slot)] = f32_to_bf16(v[e]);
  }
}

}  // namespace

extern "C" int sb_rope_kv_store(void *q_out, int q_dtype, const void *qkv, int qkv_dtype,
                                int row_stride, int n_slices, const float *bias, const float *inv_freq, const float *freq_factors,
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
  SB_REQUIRE(n_slices >= 1, "sb_rope_kv_store: at least one slice");
  SB_SUPPORT(n_slices <= kMaxSlices, "sb_rope_kv_store: %d slices, at most %d", n_slices, kMaxSlices);
  const size_t slice_stride = size_t(n_rows) * row_stride;
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
  const int n_heads = heads_q + 2 * heads_kv;
  const uintptr_t addresses = reinterpret_cast<uintptr_t>(qkv) | reinterpret_cast<uintptr_t>(q_out) |
                              reinterpret_cast<uintptr_t>(k_cache);
  const uintptr_t bias_address = reinterpret_cast<uintptr_t>(bias);
  if (n_rows >= 512 && q_dtype == SB_BF16 && cache_dtype == SB_BF16 && head_dim % 8 == 0 && row_stride % 8 == 0 &&
      (!inv_freq || rot_dims % 16 == 0) && (addresses | bias_address) % 16 == 0) {
#define SB_ROWS(TI, SLICES)                                                                              \
  rope_kv_rows_kernel<TI, SLICES><<<n_rows, 256, 0, s>>>(                                                \
      (bf16_t *)q_out, (const TI *)qkv, row_stride, n_slices, slice_stride, bias, inv_freq, freq_factors, \
      rot_dims, row_pos, row_seq, (bf16_t *)k_cache, (bf16_t *)v_cache, page_table, max_pages,           \
      n_pages_total, heads_q, heads_kv, head_dim)
    if (qkv_dtype == SB_BF16) {
      if (n_slices == 1) SB_ROWS(bf16_t, 1);
      else if (n_slices <= 4) SB_ROWS(bf16_t, 4);
      else SB_ROWS(bf16_t, kMaxSlices);
    } else {
      if (n_slices == 1) SB_ROWS(float, 1);
      else if (n_slices <= 4) SB_ROWS(float, 4);
      else SB_ROWS(float, kMaxSlices);
    }
#undef SB_ROWS
    return sb::check_launch("sb_rope_kv_store");
  }
  const int heads_per_block = n_rows >= 512 ? n_heads : 4;
  const dim3 grid(n_rows, (n_heads + heads_per_block - 1) / heads_per_block);
  SB_SUPPORT(grid.y <= 65535, "sb_rope_kv_store: too many heads");
#define SB_GO(TI, TQ, TC)                                                                        \
  if (n_slices == 1) SB_GO2(TI, TQ, TC, 1);                                                        \
  else if (n_slices <= 4) SB_GO2(TI, TQ, TC, 4);                                                   \
  else SB_GO2(TI, TQ, TC, kMaxSlices)
#define SB_GO2(TI, TQ, TC, SLICES)                                                               \
  rope_kv_kernel<TI, TQ, TC, SLICES><<<grid, 256, 0, s>>>(                                      \
      (TQ *)q_out, (const TI *)qkv, row_stride, n_slices, slice_stride, bias, inv_freq, freq_factors,   \
      rot_dims, row_pos, row_seq,                                                                    \
      (TC *)k_cache, (TC *)v_cache, page_table, max_pages, n_pages_total, heads_q, heads_kv, head_dim,  \
      heads_per_block)
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
#undef SB_GO2
  return sb::check_launch("sb_rope_kv_store");
}
