/* C ABI of the sonicboom_amd HIP kernel library (gfx950).
 *
 * Conventions, in the manner of the reference's capi.h
 * (/root/reference/capi/include/sonicboom/capi.h:136-161): every entry point
 * returns a status, 0 on success; on failure the message of the calling
 * thread's last error is read with sb_last_error().  No exception crosses
 * this boundary.  All pointers are device pointers unless said otherwise;
 * `stream` is a hipStream_t.  Shapes are checked on the host before any
 * launch; a size that a kernel cannot take is refused with SB_ERR_UNSUPPORTED,
 * never computed wrongly.
 *
 * Element types are named by sb_dtype.  Tensors are row-major and dense unless
 * a stride is given.  The KV cache is paged: a layer's keys are
 * [pages][kv_heads][SB_PAGE][head_dim], its values transposed,
 * [pages][kv_heads][head_dim][SB_PAGE]; `page_table` is int32 [batch][max_pages]
 * and maps the logical page (position / SB_PAGE) of a sequence to a physical
 * page, -1 for none.  Within a row of keys (one slot of a page) and within a row
 * of values (one dimension over the page's slots) the groups of eight elements
 * are kept in a permuted order: sb_key_index and sb_value_index below say where
 * an element lies.  It is the order in which the matrix-core attention reads a
 * page from LDS without bank conflicts, so a page goes from the cache into LDS
 * as it lies.
 */
#ifndef SONICBOOM_AMD_SB_HIP_H
#define SONICBOOM_AMD_SB_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SB_PAGE 64

#if defined(__HIPCC__)
#define SB_INLINE static inline __host__ __device__
#else
#define SB_INLINE static inline
#endif

/* Offset (in elements) of element d of the key at slot `slot` (0..SB_PAGE-1)
 * within a page's [SB_PAGE][head_dim] block of one head: group d / 8 of the row
 * lies at group (d / 8) ^ s, s made of bits 0, 1, 3 and 4 of the slot, cut to the
 * largest power of two (up to 16) that divides the row's number of groups.
 * Head sizes that are no multiple of 16 keep the plain order. */
SB_INLINE int sb_key_swizzle(int slot, int head_dim) {
  if (head_dim % 16) return 0;
  const int groups = head_dim / 8;
  const int mask = groups % 16 == 0 ? 15 : (groups % 8 == 0 ? 7 : (groups % 4 == 0 ? 3 : 1));
  return ((slot & 3) | (((slot >> 3) & 3) << 2)) & mask;
}
SB_INLINE size_t sb_key_index(int slot, int d, int head_dim) {
  return (size_t)slot * (size_t)head_dim + (size_t)((((d >> 3) ^ sb_key_swizzle(slot, head_dim)) << 3) | (d & 7));
}
/* Offset of the value of dimension d at slot `slot` within a page's
 * [head_dim][SB_PAGE] block of one head: group slot / 8 of the row lies at group
 * (slot / 8) ^ ((d / 2) % 8). */
SB_INLINE size_t sb_value_index(int d, int slot) {
  return (size_t)d * SB_PAGE + (size_t)((((slot >> 3) ^ ((d >> 1) & 7)) << 3) | (slot & 7));
}

typedef enum sb_status {
  SB_OK = 0,
  SB_ERR_ARGUMENT = 1,    /* null pointer, negative size, inconsistent shapes */
  SB_ERR_UNSUPPORTED = 2, /* a size or type this kernel does not take */
  SB_ERR_LAUNCH = 3       /* the HIP runtime refused the launch */
} sb_status;

typedef enum sb_dtype { SB_F32 = 0, SB_BF16 = 1 } sb_dtype;

/* The `gated` argument of the products and of sb_gate_mul: not gated, or the activation of the
 * gate in Y = act(X Wg^T) * (X Wu^T). */
typedef enum sb_gate { SB_GATE_NONE = 0, SB_GATE_SILU = 1, SB_GATE_GELU_TANH = 2 } sb_gate;

/* Message of this thread's last failed call ("" if none). Never NULL. */
const char *sb_last_error(void);
/* A JSON object naming the target architecture, the page size and the build flags. */
const char *sb_build_info(void);

/* out[t,:] = table[ids[t],:]  as f32.  An id outside [0,vocab) yields a NaN row. */
int sb_embed(float *out, const void *table, int table_dtype, const int32_t *ids,
             int n_rows, int width, int vocab, void *stream);

/* y[r,:] = (x[src,:] * inv) * w,  inv = 1/sqrt(mean(x[src,:]^2) + eps), src = rows ? rows[r] : r.
 * x is f32; y is out_dtype; w is w_dtype (NULL = no weight). */
int sb_rmsnorm(void *y, int out_dtype, const float *x, const void *w, int w_dtype,
               const int32_t *rows, int n_rows, int width, float eps, void *stream);

/* x[t,:] += sum_s partial[s][t][:] (+ bias), slices in ascending order; with do_norm
 * also y[t,:] = rmsnorm(x[t,:]) * w.  partial is f32 [n_slices][n_rows][width]. */
int sb_reduce_resid_norm(void *y, int y_dtype, float *x, const float *partial, int n_slices,
                         const void *bias, int bias_dtype, const void *w, int w_dtype, int n_rows,
                         int width, float eps, int do_norm, void *stream);

/* Y[t,n] = sum_k X[t,k] W[n,k] (+ bias[n]) (+ resid[t,n]).   Plain tiled kernel,
 * float accumulation in ascending k for every element whatever the batch.
 * resid is f32 [t,n] and may be the same buffer as Y (when Y is f32). */
int sb_gemm(void *y, int y_dtype, const void *x, int x_dtype, const void *w, int w_dtype,
            const void *bias, int bias_dtype, const float *resid,
            int n_rows, int n_out, int n_in, void *stream);

/* out[t,i] = act(gu[t,i]) * gu[t,width+i];  gu is [t, 2*width]; gate: SB_GATE_SILU or
 * SB_GATE_GELU_TANH. */
int sb_gate_mul(void *out, int out_dtype, const void *gu, int gu_dtype, int n_rows, int width, int gate,
                void *stream);
/* The same with the SiLU gate. */
int sb_silu_mul(void *out, int out_dtype, const void *gu, int gu_dtype,
                int n_rows, int width, void *stream);

/* resid[i] += y[i]  (resid f32, y of y_dtype). */
int sb_add_into(float *resid, const void *y, int y_dtype, size_t n, void *stream);

/* dst[i] = src[i] converted. */
int sb_cast(void *dst, int dst_dtype, const void *src, int src_dtype, size_t n, void *stream);

/* Rotate the query heads and key heads of a step's qkv rows, write the queries
 * to q_out and store keys and values into the paged cache.
 *   qkv        [n_slices][n_rows, row_stride] of qkv_dtype, read only; a row is
 *              [heads_q*hd queries | heads_kv*hd keys | heads_kv*hd values];
 *              the slices (partial sums of the projection over K) are added
 *              in ascending order, then `bias` (f32 [row], may be NULL)
 *   q_out      [n_rows, heads_q*hd] of q_dtype
 *   inv_freq   f32 [rot_dims/2]: angle of pair i at position p is
 *              float(p)*inv_freq[i], divided by freq_factors[i] when given.
 *              NULL = no rotation.  Pair i is (i, i + rot_dims/2) of a head.
 *   row_pos    int32 [n_rows] absolute position;  row_seq int32 [n_rows] index
 *              of the row's sequence in page_table.
 *   k_cache/v_cache of cache_dtype; NULL (with heads_kv = 0) for a layer that
 *              stores nothing.
 */
int sb_rope_kv_store(void *q_out, int q_dtype, const void *qkv, int qkv_dtype, int row_stride,
                     int n_slices, const float *bias, const float *inv_freq, const float *freq_factors, int rot_dims,
                     const int32_t *row_pos, const int32_t *row_seq, void *k_cache, void *v_cache,
                     int cache_dtype, const int32_t *page_table, int max_pages, int n_pages_total,
                     int n_rows, int heads_q, int heads_kv, int head_dim, void *stream);

/* Attention of every row over its sequence's cached keys, position by position:
 * row r at position p of sequence s sees keys j with j <= p and (window == 0 or
 * p - j < window).  One wave per (row, query head), 64 keys at a time, online
 * softmax in f32 whose reduction order depends on key positions only.
 *   q   [n_rows, q_stride] of act_dtype (heads back to back at the row's start)
 *   out [n_rows, heads_q*hd] of act_dtype
 */
int sb_attention(void *out, const void *q, int act_dtype, int q_stride, const void *k_cache,
                 const void *v_cache, int cache_dtype, const int32_t *page_table, int max_pages,
                 int n_pages_total, const int32_t *row_pos, const int32_t *row_seq, int n_rows,
                 int heads_q, int heads_kv, int head_dim, float scale, int window, void *stream);

/* ids[r] = index of the first maximum of logits[r,:].  Two stages over
 * sb_argmax_parts(vocab) parts of a row; part_val / part_idx hold n_rows * parts
 * partial results (NULL allowed when parts == 1). */
int sb_argmax_parts(int vocab);
int sb_argmax(int32_t *ids, const float *logits, int n_rows, int vocab, float *part_val,
              int32_t *part_idx, void *stream);

/* sb_argmax for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference.  The caller passes the logits and the output
 * only; the first stage's partial results go to a fixed device array of
 * 512 KB that every GPU the library runs on holds until the process ends, so
 * n_rows * sb_argmax_parts(vocab) may be at most sb_argmax_noalloc_max_entries()
 * (65,536; e.g. 1,724 rows of 152,064 logits); more is refused with
 * SB_ERR_UNSUPPORTED.  The call allocates and frees nothing.  Every call on a
 * GPU shares that GPU's array: the first stage overwrites every entry the second
 * stage reads, so nothing is cleared, and two calls that overlap on one GPU
 * (different streams, or threads) race.  Same results as sb_argmax. */
int sb_argmax_noalloc_max_entries(void);
int sb_argmax_noalloc(int32_t *ids, const float *logits, int n_rows, int vocab, void *stream);

/* Sampling penalties on the logits in place, for `n_items` (row, token, count)
 * triples: v = v>0 ? v/rp : v*rp (when rp != 1), then v -= freq*count + presence.
 * exact != 0 uses the single-rounding fma form of the sampled path. */
int sb_penalize(float *logits, int vocab, const int32_t *item_row, const int32_t *item_token,
                const int32_t *item_count, int n_items, float repeat_penalty,
                float presence_penalty, float frequency_penalty, int exact, void *stream);

/* The mask of constrained decoding on logits [n_rows, vocab] in place: -inf wherever
 * a row's bitmap (uint8 [n_rows, n_bytes]; bit i & 7 of byte i >> 3 for id i; ids past
 * the bitmap are not allowed) does not allow the id. */
int sb_mask_logits(float *logits, int n_rows, int vocab, const uint8_t *bitmaps, int n_bytes, void *stream);

/* The `k` (<= 256) candidates with the largest z = logit / temperature of every
 * row (ties toward the lower id), ordered by (z descending, id ascending).
 * cand_id int32 [n_rows,k], cand_z f32 [n_rows,k]; rows with vocab < k are
 * filled with id -1.  Long rows are cut into parts whose best go through
 * `scratch`: sb_top_candidates_scratch(...) 64-bit words (NULL when that is 0). */
size_t sb_top_candidates_scratch(int n_rows, int vocab);
int sb_top_candidates(int32_t *cand_id, float *cand_z, const float *logits, int n_rows, int vocab,
                      int k, float temperature, uint64_t *scratch, void *stream);

/* One token per row from its candidates as sb_top_candidates wrote them (k <= 256
 * per row): the window of 30 below the best z, top-k (0: off), min-p
 * (log_min_p = ln(min_p) as a float; use_min_p 0: off), top-p (use_top_p 0: off;
 * running sums in float64, in order) and the Gumbel-max draw with word 0 of
 * Philox4x32-10 of counter (position, id, 0) under `seed`; ties to the lower id.
 * position int64 [n_rows]: the absolute position of each row's new token.
 * token int32 [n_rows]: -1 for a row that keeps no candidate. */
int sb_draw(int32_t *token, const int32_t *cand_id, const float *cand_z, const int64_t *position,
            int n_rows, int k, int top_k, int use_min_p, float log_min_p, int use_top_p, double top_p,
            uint64_t seed, void *stream);
/* The same with the positions taken from a decode step's device bookkeeping:
 * row r's new token takes position length_before[r] + 1. */
int sb_draw_after(int32_t *token, const int32_t *cand_id, const float *cand_z, const int32_t *length_before,
                  int n_rows, int k, int top_k, int use_min_p, float log_min_p, int use_top_p, double top_p,
                  uint64_t seed, void *stream);

/* ---- bf16 products on the matrix cores ----------------------------------
 * X bf16 [n_rows, n_in] row-major, n_in a multiple of 8, operands 16-byte
 * aligned.  W bf16 [n_out, n_in] row-major, or (packed != 0, or always for the
 * stream kernel) re-laid in 16 x 32 tiles of 1 KB in MFMA fragment order, rows
 * padded to 16 and k to 32, tiles of a row block consecutive in k; gated: the two
 * halves [gate; up] packed one after the other, Y = act(X Wg^T) * (X Wu^T) with the activation
 * that `gated` names (an sb_gate).
 * Y f32 or bf16; bias [n_out] f32 or bf16 or NULL; resid f32 [n_rows, n_out] or
 * NULL (may be Y itself).  The *_partial_* forms write the raw product in K
 * slices, f32 [slices][n_rows][n_out], slices as the matching *_slices says. */
int sb_gemm_skinny_max_rows(void);                       /* up to 64 rows, waves split K */
size_t sb_gemm_skinny_scratch(int n_rows, int n_out, int n_in, int gated);
int sb_gemm_skinny_bf16(void *y, int y_dtype, const void *x, const void *w, const void *bias,
                        int bias_dtype, const float *resid, int n_rows, int n_out, int n_in, int gated,
                        int packed, float *scratch, size_t scratch_floats, void *stream);
int sb_gemm_skinny_slices(int n_rows, int n_out, int n_in);
int sb_gemm_skinny_partial_bf16(float *partial, const void *x, const void *w, int n_rows, int n_out,
                                int n_in, int packed, void *stream);
int sb_gemm_stream_max_rows(void);                       /* up to 128 rows, waves split the features */
/* `hint` (0: the launcher chooses; for tests and measurements): bits 0..7 waves per block (4..8),
 * bits 8..15 the K slices the partial form aims at (1..8).  `tile_shape`: -1 the launcher
 * chooses; else bits 0..3 the tile, 0 / 1 / 2 / 3 for 128 x 128, 256 x 128, 256 x 256, 128 x 256
 * outputs, and bits 4..5 the kernel: 0 the launcher's choice, 1 the one that stages tiles
 * through registers, 2 the one that loads them straight into LDS (packed weights, n_in a multiple
 * of 64; the only one with the 128 x 256 tile), 3 the same with a block for every tile. */
int sb_gemm_stream_bf16(void *y, int y_dtype, const void *x, const void *w, const void *bias,
                        int bias_dtype, const float *resid, int n_rows, int n_out, int n_in, int gated,
                        int hint, void *stream);
int sb_gemm_stream_slices(int n_rows, int n_out, int n_in, int hint);     /* up to 64 rows */
int sb_gemm_stream_partial_bf16(float *partial, const void *x, const void *w, int n_rows, int n_out,
                                int n_in, int hint, void *stream);
int sb_gemm_mfma_bf16(void *y, int y_dtype, const void *x, const void *w, const void *bias,   /* tiled */
                      int bias_dtype, const float *resid, int n_rows, int n_out, int n_in, int gated,
                      int packed, int tile_shape, void *stream);
int sb_gemm_mfma_slices(int n_rows, int n_out, int n_in, int packed);
int sb_gemm_mfma_partial_bf16(float *partial, const void *x, const void *w, int n_rows, int n_out,
                              int n_in, int packed, void *stream);

/* Seeded normal weights: elements first .. first + n - 1 (first a multiple of 4) of tensor number
 * `tensor_index` under `seed`, as float32(mean + std z) (out_kind 0), the same rounded to bfloat16
 * (1), or the float64 standard normals z themselves (2).  Element e comes from Philox4x32-10 with
 * the seed as key and the counter (e / 4 low, e / 4 high, tensor_index, 0), words 0 and 1 making the
 * normals of elements 4c and 4c + 1, words 2 and 3 those of 4c + 2 and 4c + 3 (Box and Muller).  The
 * host computes the same bits (sonicboom_amd/weights/random_stream.py). */
int sb_random_normal(void *out, int out_kind, uint64_t n, uint64_t first, uint64_t seed, int tensor_index,
                     double mean, double std, void *stream);

#ifdef __cplusplus
}
#endif
#endif
