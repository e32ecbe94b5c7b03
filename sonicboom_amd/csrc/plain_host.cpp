// Plain C++ twins of the kernels, on host memory.
//
// Every kernel of the library sits beside a function here that does the same
// work in the plainest way: float arrays in host memory, one loop per index, the
// formula as the reference writes it.  They take what the sb_* entry points take
// (without element types and stream: everything is float32) and are what the tests
// compare the kernels with, beside the NumPy implementation under tests/.  Nothing
// on the path of a step calls them: there is no CPU fallback.
//
// The reference pairs its device kernels with host functions of the same signature
// the same way (/root/reference/core/src/model/exec.cpp:73-78,
// /root/reference/tests/core/test_nn.cpp:100-127).  Formulas:
// norm /root/reference/core/src/nn/norm.cpp:25-42, rotation
// /root/reference/core/src/nn/rope.cpp:26-56, attention
// /root/reference/core/src/nn/attention.cpp:26-105, activation
// /root/reference/core/src/nn/activation.cpp:41-50, first maximum
// /root/reference/core/src/nn/sampling.cpp:238-244.
#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <limits>
#include <utility>
#include <vector>

#include "sb_hip.h"   // the cache's element order (sb_key_index, sb_value_index)

namespace {
constexpr int kPage = 64;   // SB_PAGE
}

extern "C" {

// out[t,:] = table[ids[t],:]; an id outside [0, vocab) gives a row of NaN.
int sbp_embed(float *out, const float *table, const int32_t *ids, int n_rows, int width, int vocab) {
  if (!out || !table || !ids || n_rows < 0 || width <= 0 || vocab <= 0) return 1;
  for (int t = 0; t < n_rows; ++t)
    for (int i = 0; i < width; ++i)
      out[size_t(t) * width + i] = (ids[t] < 0 || ids[t] >= vocab) ? std::numeric_limits<float>::quiet_NaN()
                                                                   : table[size_t(ids[t]) * width + i];
  return 0;
}

// y[r,:] = (x[src,:] * inv) * w, inv = 1 / sqrt(mean(x^2) + eps), src = rows ? rows[r] : r.
// Each square is a float product, the sum runs in double, the mean is rounded to float.
int sbp_rmsnorm(float *y, const float *x, const float *w, const int32_t *rows, int n_rows, int width, float eps) {
  if (!y || !x || n_rows < 0 || width <= 0 || eps < 0.f) return 1;
  for (int r = 0; r < n_rows; ++r) {
    const float *xr = x + size_t(rows ? rows[r] : r) * width;
    double sum = 0.0;
    for (int i = 0; i < width; ++i) sum += double(xr[i] * xr[i]);
    const float mean = float(sum / double(width));
    const float inv = 1.0f / std::sqrt(mean + eps);
    for (int i = 0; i < width; ++i) {
      float o = xr[i] * inv;
      if (w) o = o * w[i];
      y[size_t(r) * width + i] = o;
    }
  }
  return 0;
}

// x[t,:] += sum over slices of partial[s][t][:] (+ bias), slices in ascending order, then the
// bias, then the residual; with do_norm also y[t,:] = rmsnorm(x[t,:]) * w.
int sbp_reduce_resid_norm(float *y, float *x, const float *partial, int n_slices, const float *bias, const float *w,
                          int n_rows, int width, float eps, int do_norm) {
  if (!x || !partial || n_slices < 1 || n_rows < 0 || width <= 0 || (do_norm && !y)) return 1;
  for (int t = 0; t < n_rows; ++t)
    for (int i = 0; i < width; ++i) {
      float acc = partial[size_t(t) * width + i];
      for (int s = 1; s < n_slices; ++s) acc += partial[(size_t(s) * n_rows + t) * width + i];
      if (bias) acc += bias[i];
      x[size_t(t) * width + i] = acc + x[size_t(t) * width + i];
    }
  return do_norm ? sbp_rmsnorm(y, x, w, nullptr, n_rows, width, eps) : 0;
}

// Y[t,n] = sum_k X[t,k] W[n,k] (+ bias[n]) (+ resid[t,n]): one fused multiply-add per k in
// ascending order from zero, as the plain kernel does (so the two agree to the bit).
int sbp_gemm(float *y, const float *x, const float *w, const float *bias, const float *resid, int n_rows,
             int n_out, int n_in) {
  if (!y || !x || !w || n_rows < 0 || n_out <= 0 || n_in <= 0) return 1;
  for (int t = 0; t < n_rows; ++t)
    for (int n = 0; n < n_out; ++n) {
      float acc = 0.0f;
      for (int k = 0; k < n_in; ++k) acc = std::fmaf(x[size_t(t) * n_in + k], w[size_t(n) * n_in + k], acc);
      if (bias) acc = acc + bias[n];
      if (resid) acc = acc + resid[size_t(t) * n_out + n];
      y[size_t(t) * n_out + n] = acc;
    }
  return 0;
}

// out[t,i] = act(gu[t,i]) * gu[t,width+i]; gate 1: silu(g) = g / (1 + exp(-g)); gate 2: the tanh
// form of GELU, 0.5 g (1 + tanh(sqrt(2/pi) g (1 + 0.044715 g^2))).
int sbp_gate_mul(float *out, const float *gu, int n_rows, int width, int gate) {
  if (!out || !gu || n_rows < 0 || width <= 0 || (gate != 1 && gate != 2)) return 1;
  for (int t = 0; t < n_rows; ++t)
    for (int i = 0; i < width; ++i) {
      const float g = gu[size_t(t) * 2 * width + i];
      const float a = gate == 2 ? 0.5f * g * (1.0f + std::tanh(0.79788456080286535587989211986876f * g *
                                                              (1.0f + 0.044715f * g * g)))
                                : g / (1.0f + std::exp(-g));
      out[size_t(t) * width + i] = a * gu[size_t(t) * 2 * width + width + i];
    }
  return 0;
}
int sbp_silu_mul(float *out, const float *gu, int n_rows, int width) { return sbp_gate_mul(out, gu, n_rows, width, 1); }

int sbp_add_into(float *resid, const float *y, size_t n) {
  if (!resid || !y) return 1;
  for (size_t i = 0; i < n; ++i) resid[i] += y[i];
  return 0;
}

// Rotate the query and key heads of qkv rows [queries | keys | values] (+ bias first), write the
// queries and store keys [pages][kv heads][64][hd] and values [pages][kv heads][hd][64].
// Pair i of a head is (i, i + rot_dims / 2); theta = float(pos) * inv_freq[i] (/ freq_factors[i]).
int sbp_rope_kv_store(float *q_out, const float *qkv, int row_stride, const float *bias, const float *inv_freq,
                      const float *freq_factors, int rot_dims, const int32_t *row_pos, const int32_t *row_seq,
                      float *k_cache, float *v_cache, const int32_t *page_table, int max_pages, int n_pages_total,
                      int n_rows, int heads_q, int heads_kv, int head_dim) {
  if (!q_out || !qkv || !row_pos || n_rows < 0 || heads_q <= 0 || heads_kv < 0 || head_dim <= 0) return 1;
  if (heads_kv > 0 && (!k_cache || !v_cache || !page_table || !row_seq)) return 1;
  if (inv_freq && (rot_dims <= 0 || rot_dims % 2 || rot_dims > head_dim)) return 1;
  const int half = inv_freq ? rot_dims / 2 : 0;
  std::vector<float> head(static_cast<size_t>(head_dim), 0.0f);
  for (int t = 0; t < n_rows; ++t) {
    const float *r = qkv + size_t(t) * row_stride;
    const int pos = row_pos[t];
    int page = -1;
    if (heads_kv > 0) {
      const int lp = pos / kPage;
      page = (lp >= 0 && lp < max_pages) ? page_table[size_t(row_seq[t]) * max_pages + lp] : -1;
      if (page >= n_pages_total) page = -1;
    }
    for (int h = 0; h < heads_q + 2 * heads_kv; ++h) {
      const size_t hoff = size_t(h) * head_dim;
      for (int d = 0; d < head_dim; ++d) head[d] = r[hoff + d] + (bias ? bias[hoff + d] : 0.0f);
      if (h < heads_q + heads_kv)
        for (int i = 0; i < half; ++i) {
          float theta = float(pos) * inv_freq[i];
          if (freq_factors) theta = theta / freq_factors[i];
          const float c = std::cos(theta), s = std::sin(theta);
          const float x0 = head[i], x1 = head[i + half];
          head[i] = x0 * c - x1 * s;
          head[i + half] = x0 * s + x1 * c;
        }
      if (h < heads_q) {
        for (int d = 0; d < head_dim; ++d) q_out[size_t(t) * heads_q * head_dim + hoff + d] = head[d];
      } else if (page >= 0) {
        const bool is_k = h < heads_q + heads_kv;
        const int kh = is_k ? h - heads_q : h - heads_q - heads_kv;
        const size_t base = (size_t(page) * heads_kv + kh) * kPage * head_dim;
        for (int d = 0; d < head_dim; ++d) {
          if (is_k) k_cache[base + sb_key_index(pos % kPage, d, head_dim)] = head[d];
          else v_cache[base + sb_value_index(d, pos % kPage)] = head[d];
        }
      }
    }
  }
  return 0;
}

// Row r at position p of sequence s sees keys j <= p with (window == 0 or p - j < window); query
// head h reads kv head h / group; softmax with the maximum subtracted; a row that sees no key
// is zero.  Dot products and the mix accumulate in double, rounded once.
int sbp_attention(float *out, const float *q, int q_stride, const float *k_cache, const float *v_cache,
                  const int32_t *page_table, int max_pages, int n_pages_total, const int32_t *row_pos,
                  const int32_t *row_seq, int n_rows, int heads_q, int heads_kv, int head_dim, float scale,
                  int window) {
  if (!out || !q || !k_cache || !v_cache || !page_table || !row_pos || !row_seq) return 1;
  if (n_rows < 0 || heads_q <= 0 || heads_kv <= 0 || heads_q % heads_kv || head_dim <= 0 || window < 0) return 1;
  const int group = heads_q / heads_kv;
  std::vector<float> score;
  std::vector<int> key;
  for (int t = 0; t < n_rows; ++t) {
    const int pos = row_pos[t], seq = row_seq[t];
    const int lo = (window > 0 && pos >= window) ? pos - window + 1 : 0;
    for (int h = 0; h < heads_q; ++h) {
      const int kh = h / group;
      const float *qh = q + size_t(t) * q_stride + size_t(h) * head_dim;
      score.clear();
      key.clear();
      for (int j = lo; j <= pos; ++j) {
        const int lp = j / kPage;
        const int page = lp < max_pages ? page_table[size_t(seq) * max_pages + lp] : -1;
        if (page < 0 || page >= n_pages_total) continue;
        const float *kp = k_cache + (size_t(page) * heads_kv + kh) * kPage * head_dim;
        double dot = 0.0;
        for (int d = 0; d < head_dim; ++d) dot += double(qh[d]) * double(kp[sb_key_index(j % kPage, d, head_dim)]);
        score.push_back(float(dot) * scale);
        key.push_back(j);
      }
      float *o = out + (size_t(t) * heads_q + h) * head_dim;
      if (score.empty()) {
        for (int d = 0; d < head_dim; ++d) o[d] = 0.0f;
        continue;
      }
      float m = score[0];
      for (float s : score) m = s > m ? s : m;
      float sum = 0.0f;
      for (float &s : score) {
        s = std::exp(s - m);
        sum += s;
      }
      const float inv = 1.0f / sum;
      for (int d = 0; d < head_dim; ++d) {
        double acc = 0.0;
        for (size_t i = 0; i < score.size(); ++i) {
          const int j = key[i];
          const int page = page_table[size_t(seq) * max_pages + j / kPage];
          acc += double(score[i] * inv) *
                 double(v_cache[(size_t(page) * heads_kv + kh) * head_dim * kPage + sb_value_index(d, j % kPage)]);
        }
        o[d] = float(acc);
      }
    }
  }
  return 0;
}

// ids[r] = index of the first maximum of logits[r,:].
int sbp_argmax(int32_t *ids, const float *logits, int n_rows, int vocab) {
  if (!ids || !logits || n_rows < 0 || vocab <= 0) return 1;
  for (int r = 0; r < n_rows; ++r) {
    int best = 0;
    for (int i = 1; i < vocab; ++i)
      if (logits[size_t(r) * vocab + i] > logits[size_t(r) * vocab + best]) best = i;
    ids[r] = best;
  }
  return 0;
}

// Sampling penalties in place for (row, token, count) triples
// (/root/reference/core/src/nn/sampling.cpp:43-70 and, exact, :77-104): v = v > 0 ? v / rp : v * rp when rp != 1,
// then v -= freq * count + presence; exact: with one rounding where the sampled path has one.
int sbp_penalize(float *logits, int vocab, const int32_t *item_row, const int32_t *item_token,
                 const int32_t *item_count, int n_items, float rp, float presence, float freq, int exact) {
  if (!logits || vocab <= 0 || n_items < 0 || (n_items && (!item_row || !item_token || !item_count))) return 1;
  for (int it = 0; it < n_items; ++it) {
    const int tok = item_token[it];
    if (tok < 0 || tok >= vocab) continue;
    float &v = logits[size_t(item_row[it]) * vocab + tok];
    const float c = float(item_count[it]);
    if (rp != 1.0f) v = v > 0.0f ? v / rp : v * rp;
    if (exact) {
      v = std::fma(-1.0f, std::fma(freq, c, presence), v);
    } else {
      const float fc = freq * c;
      const float adjust = fc + presence;
      v = v - adjust;
    }
  }
  return 0;
}

// The mask of constrained decoding in place (/root/reference/core/src/nn/sampling.cpp:266-274): -inf
// wherever bit i & 7 of byte i >> 3 of the row's bitmap is clear or the bitmap ends before it.
int sbp_mask_logits(float *logits, int n_rows, int vocab, const uint8_t *bitmaps, int n_bytes) {
  if (!logits || !bitmaps || n_rows < 0 || vocab <= 0 || n_bytes <= 0) return 1;
  for (int r = 0; r < n_rows; ++r)
    for (int i = 0; i < vocab; ++i) {
      const int byte = i >> 3;
      const bool allowed = byte < n_bytes && ((bitmaps[size_t(r) * n_bytes + byte] >> (i & 7)) & 1u);
      if (!allowed) logits[size_t(r) * vocab + i] = -std::numeric_limits<float>::infinity();
    }
  return 0;
}

// The k best of every row by z = logit / temperature (one float32 division), ordered
// (z descending, id ascending); id -1 and z 0 past a short row's end
// (/root/reference/core/src/nn/sampling.cpp:257-285).
int sbp_top_candidates(int32_t *cand_id, float *cand_z, const float *logits, int n_rows, int vocab, int k,
                       float temperature) {
  if (!cand_id || !cand_z || !logits || n_rows < 0 || vocab <= 0 || k < 1 || !(temperature > 0.0f)) return 1;
  std::vector<std::pair<float, int>> row(static_cast<size_t>(vocab));
  for (int r = 0; r < n_rows; ++r) {
    for (int i = 0; i < vocab; ++i) row[i] = {logits[size_t(r) * vocab + i] / temperature + 0.0f, i};
    std::sort(row.begin(), row.end(), [](const std::pair<float, int> &a, const std::pair<float, int> &b) {
      return a.first != b.first ? a.first > b.first : a.second < b.second;
    });
    for (int i = 0; i < k; ++i) {
      cand_id[size_t(r) * k + i] = i < vocab ? row[i].second : -1;
      cand_z[size_t(r) * k + i] = i < vocab ? row[i].first : 0.0f;
    }
  }
  return 0;
}

namespace {
uint32_t philox_word0(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint64_t key) {
  uint32_t k0 = uint32_t(key), k1 = uint32_t(key >> 32);
  for (int round = 0; round < 10; ++round) {
    const uint64_t p0 = uint64_t(0xD2511F53u) * c0, p1 = uint64_t(0xCD9E8D57u) * c2;
    const uint32_t n0 = uint32_t(p1 >> 32) ^ c1 ^ k0, n1 = uint32_t(p1), n2 = uint32_t(p0 >> 32) ^ c3 ^ k1,
                   n3 = uint32_t(p0);
    c0 = n0, c1 = n1, c2 = n2, c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return c0;
}
}  // namespace

// One token per row from its ordered candidates: window 30, top-k, min-p, top-p, Gumbel-max
// (/root/reference/core/src/nn/sampling.cpp:157-203, :287-312); the arguments of sb_draw.
int sbp_draw(int32_t *token, const int32_t *cand_id, const float *cand_z, const int64_t *position, int n_rows,
             int k, int top_k, int use_min_p, float log_min_p, int use_top_p, double top_p, uint64_t seed) {
  if (!token || !cand_id || !cand_z || !position || n_rows < 0 || k < 1 || top_k < 0) return 1;
  for (int r = 0; r < n_rows; ++r) {
    const int32_t *id = cand_id + size_t(r) * k;
    const float *z = cand_z + size_t(r) * k;
    const float m = z[0], floor_z = m - 30.0f, cutoff = m + log_min_p;
    int keep = 0;
    for (int c = 0; c < k; ++c) keep += id[c] >= 0 && z[c] >= floor_z;
    if (top_k > 0 && keep > top_k) keep = top_k;
    if (use_min_p) {
      int kept = 0;
      for (int c = 0; c < keep; ++c) kept += !(z[c] < cutoff);
      keep = kept;
    }
    if (use_top_p && keep > 0) {
      double total = 0.0;
      for (int c = 0; c < keep; ++c) total += std::exp(double(z[c]) - double(m));
      if (total > 0.0) {
        double acc = 0.0;
        for (int c = 0; c < keep; ++c) {
          acc += std::exp(double(z[c]) - double(m));
          if (acc / total >= top_p) {
            keep = c + 1;
            break;
          }
        }
      }
    }
    int best = -1;
    double best_score = 0.0;
    const uint64_t pos = uint64_t(position[r]);
    for (int c = 0; c < keep; ++c) {
      const uint32_t w = philox_word0(uint32_t(pos), uint32_t(pos >> 32), uint32_t(id[c]), 0u, seed);
      const double u = (double(w) + 0.5) / 4294967296.0;
      const double score = double(z[c]) - std::log(-std::log(u));
      if (best < 0 || score > best_score || (score == best_score && id[c] < best)) best = id[c], best_score = score;
    }
    token[r] = best;
  }
  return 0;
}

}  // extern "C"
