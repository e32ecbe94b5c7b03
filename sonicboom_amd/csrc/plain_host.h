/* Plain C++ twins of the kernels on host memory (plain_host.cpp): the arguments of the sb_*
 * entry points without element types and stream; every array is float32 (int32 for indices) in
 * host memory, the cache paged as in sb_hip.h.  For tests; nothing on a step's path calls them.
 * Every function returns 0, or 1 for arguments it cannot take. */
#ifndef SONICBOOM_AMD_PLAIN_HOST_H
#define SONICBOOM_AMD_PLAIN_HOST_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

int sbp_embed(float *out, const float *table, const int32_t *ids, int n_rows, int width, int vocab);
int sbp_rmsnorm(float *y, const float *x, const float *w, const int32_t *rows, int n_rows, int width, float eps);
int sbp_reduce_resid_norm(float *y, float *x, const float *partial, int n_slices, const float *bias,
                          const float *w, int n_rows, int width, float eps, int do_norm);
int sbp_gemm(float *y, const float *x, const float *w, const float *bias, const float *resid, int n_rows,
             int n_out, int n_in);
int sbp_gate_mul(float *out, const float *gu, int n_rows, int width, int gate);   /* gate: an sb_gate */
int sbp_silu_mul(float *out, const float *gu, int n_rows, int width);
int sbp_add_into(float *resid, const float *y, size_t n);
int sbp_rope_kv_store(float *q_out, const float *qkv, int row_stride, const float *bias, const float *inv_freq,
                      const float *freq_factors, int rot_dims, const int32_t *row_pos, const int32_t *row_seq,
                      float *k_cache, float *v_cache, const int32_t *page_table, int max_pages,
                      int n_pages_total, int n_rows, int heads_q, int heads_kv, int head_dim);
int sbp_attention(float *out, const float *q, int q_stride, const float *k_cache, const float *v_cache,
                  const int32_t *page_table, int max_pages, int n_pages_total, const int32_t *row_pos,
                  const int32_t *row_seq, int n_rows, int heads_q, int heads_kv, int head_dim, float scale,
                  int window);
int sbp_argmax(int32_t *ids, const float *logits, int n_rows, int vocab);
int sbp_penalize(float *logits, int vocab, const int32_t *item_row, const int32_t *item_token,
                 const int32_t *item_count, int n_items, float repeat_penalty, float presence_penalty,
                 float frequency_penalty, int exact);
int sbp_mask_logits(float *logits, int n_rows, int vocab, const uint8_t *bitmaps, int n_bytes);
int sbp_top_candidates(int32_t *cand_id, float *cand_z, const float *logits, int n_rows, int vocab, int k,
                       float temperature);
int sbp_draw(int32_t *token, const int32_t *cand_id, const float *cand_z, const int64_t *position, int n_rows,
             int k, int top_k, int use_min_p, float log_min_p, int use_top_p, double top_p, uint64_t seed);

#ifdef __cplusplus
}
#endif
#endif
