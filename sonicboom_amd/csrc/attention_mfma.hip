// bf16 attention over the paged cache on the matrix cores, for one head size
// (compiled with -DSB_HEAD_DIM=N, N a multiple of 16 up to 256): a prefill
// kernel (many rows per sequence, causal) and a decode kernel (one row per
// sequence, keys split over blocks, the query heads of a kv head sharing its
// keys and values).
//
// Formula: /root/reference/core/src/nn/attention.cpp:26-105, :121-181 — query
// head h reads kv head h / group, s = dot(q, k) * scale, key j visible from
// position p when j <= p and (window == 0 or p - j < window), softmax with the
// maximum subtracted, in float32; probabilities are rounded to bf16 only as
// the operand of the P V product, which accumulates in float32.
//
// One wave owns 16 query columns (16 positions of one head in prefill, the
// heads of one kv head in decode) and walks its keys 32 at a time:
//   S^T[key][col] = K[key][:] . Q[col][:]     v_mfma_f32_16x16x32_bf16, A = K rows, B = Q rows
//   O^T[d][col]  += V^T[d][key] * P[key][col]  same instruction, A = V^T rows, B = P
// Row r = 4g + i of score tile t is fed key 8g + 4t + i of the 32, so that lane
// group g ends up holding the scores of keys 8g .. 8g+7 in order: exactly the
// eight k-slots of its B operand for the second product.  P therefore never
// leaves the registers; K fragments come straight from the cache ([key][d],
// 16 bytes per lane) and so do V fragments, because the cache keeps values
// transposed ([d][key]).  No LDS is used in the main loops.
//
// Order of summation: keys are visited in ascending order, 32 at a time, within
// a wave; decode merges waves (pages) and then blocks (chunks of 4 pages) in
// ascending order.  It depends on positions only, not on the batch.
#include <type_traits>

#include "mfma.h"

#ifndef SB_HEAD_DIM
#error "compile with -DSB_HEAD_DIM=<head size>"
#endif

namespace sb {
char *error_slot() {
  static thread_local char slot[kErrorLen] = {0};
  return slot;
}
}  // namespace sb

extern "C" const char *sb_attn_last_error(void) { return sb::error_slot(); }
extern "C" int sb_attn_head_dim(void) { return SB_HEAD_DIM; }

namespace {

constexpr int HD = SB_HEAD_DIM;
static_assert(HD % 16 == 0 && HD >= 16 && HD <= 256, "head size must be a multiple of 16 up to 256");
constexpr int KS = (HD + 31) / 32;   // k-steps of the score product
constexpr int DT = HD / 16;          // 16-row tiles of O^T
constexpr float kLog2e = 1.4426950408889634f;
constexpr int kPagesPerChunk = 4;
constexpr float kMaxSlack = 8.f;

// A wave's running softmax for NC groups of 16 query columns that share positions (and so the
// mask): in decode one group, the heads of a kv head; in prefill up to four heads of one kv head
// for the same 16 positions, so that every key and value fragment feeds NC products.
template <int NC>
struct WaveState {
  floatx4_t o[NC][DT];   // O^T[d = 16 dt + 4 g + i][col]
  float m[NC];           // running maximum of the column (log2 domain), same in the four lane groups
  float l[NC];           // this lane's share of the running sum
};

template <int NC>
__device__ __forceinline__ void init_state(WaveState<NC> &st) {
#pragma unroll
  for (int c = 0; c < NC; ++c) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) st.o[c][dt] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    st.m[c] = -__builtin_inff();
    st.l[c] = 0.f;
  }
}

// Zero the elements of a fragment of 8 consecutive keys from index n_keep on.
__device__ __forceinline__ uint4 keep_first(uint4 v, int n_keep) {
  uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int have = n_keep - 2 * i;   // elements of this word that stay
    w[i] = have >= 2 ? w[i] : (have == 1 ? (w[i] & 0xffffu) : 0u);
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}
// Zero the elements before index n_drop.
__device__ __forceinline__ uint4 drop_first(uint4 v, int n_drop) {
  uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gone = n_drop - 2 * i;
    w[i] = gone >= 2 ? 0u : (gone == 1 ? (w[i] & 0xffff0000u) : w[i]);
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// The fragments of one half page (32 keys): keys for both score tiles, values for all d tiles.
struct HalfPage {
  uint4 k[2][KS];
  uint4 v[DT];
};

constexpr int CPRK = HD / 8;                       // 16-byte chunks in a row of keys
constexpr int kPageChunks = SB_PAGE * HD / 8;      // 16-byte chunks of a page of keys (= of values)

// Where chunk `chunk` (8 elements) of key row `key` of a page lies, in chunks from the page's
// start: the cache's own order (sb_key_index), in which the sixteen rows a fragment read touches at
// once (key bits 0, 1, 3, 4) land in distinct LDS banks; a page is copied into LDS as it lies.
__device__ __forceinline__ int k_slot(int key, int chunk) { return key * CPRK + (chunk ^ sb_key_swizzle(key, HD)); }
// ... and of chunk `chunk` (8 keys) of value row d (sb_value_index).
__device__ __forceinline__ int v_slot(int d, int chunk) { return d * 8 + (chunk ^ ((d >> 1) & 7)); }

// The same for the fragments of a lane (row r = lane % 16, lane group g = lane / 16), written so
// that few registers hold addresses.  The keys a lane reads are 32 half + 8 (r / 4) + 4 t + r % 4:
// bits 0, 1, 3, 4 of every one of them are r's bits, so the permutation of its rows' chunks is
// the same for all of them, and a key's chunk 4 ks + g lies at
//   key_chunk(r, g, ks) + (32 half + 4 t) CPRK      (the second term a constant of the call).
// Likewise the value rows 16 dt + r of a lane share (d / 2) % 8 = (r / 2) % 8:
//   value_chunk(r, g, half) + 128 dt.
__device__ __forceinline__ int key_chunk(int r, int g, int ks) {
  const int key = 8 * (r >> 2) + (r & 3);            // the lane's key of half 0, score tile 0
  return key * CPRK + ((4 * ks + g) ^ sb_key_swizzle(key, HD));
}
__device__ __forceinline__ int value_chunk(int r, int g, int half) { return r * 8 + ((4 * half + g) ^ ((r >> 1) & 7)); }

__device__ __forceinline__ void load_half(HalfPage &hp, const bf16_t *__restrict__ kp,
                                          const bf16_t *__restrict__ vp, int half, int lane) {
  const int r = lane & 15, g = lane >> 4;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d = ks * 32 + g * 8;
    const int at = key_chunk(r, g, d < HD ? ks : 0);
#pragma unroll
    for (int t = 0; t < 2; ++t)   // A row r = 4 gg + i of score tile t is key 8 gg + 4 t + i of the 32
      hp.k[t][ks] = ld16(kp + size_t(at + (32 * half + 4 * t) * CPRK) * 8, d < HD);
  }
  const int vat = value_chunk(r, g, half);
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) hp.v[dt] = ld16(vp + size_t(vat + 128 * dt) * 8, true);
}

// The same without a branch around any load (a branch makes the compiler wait for every load in
// flight, which a loop that keeps the next half page's loads in flight cannot afford): a chunk
// past the head size is read from the row's start and replaced by zeros afterwards.
__device__ __forceinline__ void load_half_straight(HalfPage &hp, const bf16_t *__restrict__ kp,
                                                   const bf16_t *__restrict__ vp, int half, int lane) {
  const int r = lane & 15, g = lane >> 4;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d = ks * 32 + g * 8;
    const int at = key_chunk(r, g, d < HD ? ks : 0);
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const uint4 v = *reinterpret_cast<const uint4 *>(kp + size_t(at + (32 * half + 4 * t) * CPRK) * 8);
      hp.k[t][ks] = ((ks + 1) * 32 <= HD || d < HD) ? v : make_uint4(0u, 0u, 0u, 0u);
    }
  }
  const int vat = value_chunk(r, g, half);
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) hp.v[dt] = *reinterpret_cast<const uint4 *>(vp + size_t(vat + 128 * dt) * 8);
}

// 32 keys at absolute positions base .. base+31, their fragments in hp, for the wave's NC groups
// of 16 columns.  col_pos / col_lo: last and first visible key of this lane's column (col_pos < 0:
// the column is empty); the groups share them.  key_hi / key_lo: the same over all columns of the
// wave (uniform).
// MASKED = false: every key of the 32 is visible from every column (and so written): no score is
// tested and no value cut.
template <int NC, bool MASKED = true>
__device__ __forceinline__ void attend_half(WaveState<NC> &st, const bf16x8_t (&qf)[NC][KS], const HalfPage &hp,
                                            int base, int col_pos, int col_lo, int key_lo, int key_hi,
                                            float scale_log2, int lane) {
  const int g = lane >> 4;
  const int k0 = base + 8 * g;
  // values of keys outside [key_lo, key_hi] may be stale or never written: 0 * garbage must not
  // reach the accumulator, so such keys are cut out of the V fragments
  const bool cut_hi = MASKED && base + 31 > key_hi, cut_lo = MASKED && base < key_lo;
  uint4 vf[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    uint4 a = hp.v[dt];
    if (cut_hi) a = keep_first(a, key_hi - k0 + 1);
    if (cut_lo) a = drop_first(a, key_lo - k0);
    vf[dt] = a;
  }
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    floatx4_t s[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      s[t] = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) s[t] = mfma16(as_bf16x8(hp.k[t][ks]), qf[c][ks], s[t]);
    }
    // this lane: column lane % 16, keys base + 8 g + e, e = 0..7 (s[0] holds e = 0..3, s[1] e = 4..7)
    float sc[8];
    float mx = -__builtin_inff();
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int j = k0 + e;
      const bool vis = !MASKED || (j <= col_pos && j >= col_lo);
      const float v = (e < 4 ? s[0][e] : s[1][e - 4]) * scale_log2;
      sc[e] = vis ? v : -__builtin_inff();
      mx = fmaxf(mx, sc[e]);
    }
    mx = max_over_lane_groups(mx);
    const float m_new = fmaxf(st.m[c], mx);
    // a column that has seen no key yet keeps m = -inf: give it a finite stand-in
    const float m_use = m_new == -__builtin_inff() ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(st.m[c] - m_use);   // m = -inf gives 0
    float p[8];
    float psum = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      p[e] = __builtin_amdgcn_exp2f(sc[e] - m_use);                // -inf gives 0
      psum += p[e];
    }
    st.l[c] = st.l[c] * alpha + psum;
    st.m[c] = m_new;
    const uint4 pb = make_uint4(pack_bf16(p[0], p[1]), pack_bf16(p[2], p[3]), pack_bf16(p[4], p[5]),
                                pack_bf16(p[6], p[7]));
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      floatx4_t acc = st.o[c][dt];
      acc[0] *= alpha; acc[1] *= alpha; acc[2] *= alpha; acc[3] *= alpha;
      st.o[c][dt] = mfma16(as_bf16x8(vf[dt]), as_bf16x8(pb), acc);
    }
  }
}

// One page (64 keys at absolute positions page_pos .. page_pos+63).  With one column group and a
// head size up to 128 both halves' fragments are requested before the first product, so a page
// costs one round trip to memory (BOTH); otherwise half by half, to stay within the registers
// (or, when there are many more blocks than the GPU holds at once, to let more of them in).
template <int NC, bool BOTH = true>
__device__ __forceinline__ void attend_page(WaveState<NC> &st, const bf16x8_t (&qf)[NC][KS],
                                            const bf16_t *__restrict__ kp, const bf16_t *__restrict__ vp,
                                            int page_pos, int col_pos, int col_lo, int key_lo, int key_hi,
                                            float scale_log2, int lane) {
  const bool use0 = !(page_pos > key_hi || page_pos + 31 < key_lo);
  const bool use1 = !(page_pos + 32 > key_hi || page_pos + 63 < key_lo);
  if (BOTH && HD <= 128 && NC == 1) {
    HalfPage h0, h1;
    if (use0) load_half(h0, kp, vp, 0, lane);
    if (use1) load_half(h1, kp, vp, 1, lane);
    if (use0) attend_half<NC>(st, qf, h0, page_pos, col_pos, col_lo, key_lo, key_hi, scale_log2, lane);
    if (use1) attend_half<NC>(st, qf, h1, page_pos + 32, col_pos, col_lo, key_lo, key_hi, scale_log2, lane);
  } else {
    HalfPage h;
    if (use0) {
      load_half(h, kp, vp, 0, lane);
      attend_half<NC>(st, qf, h, page_pos, col_pos, col_lo, key_lo, key_hi, scale_log2, lane);
    }
    if (use1) {
      load_half(h, kp, vp, 1, lane);
      attend_half<NC>(st, qf, h, page_pos + 32, col_pos, col_lo, key_lo, key_hi, scale_log2, lane);
    }
  }
}

__device__ __forceinline__ void load_q(bf16x8_t (&qf)[KS], const bf16_t *qrow, bool col_ok, int lane) {
  const int g = lane >> 4;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d = ks * 32 + g * 8;
    qf[ks] = as_bf16x8(ld16(qrow + d, col_ok && d < HD));
  }
}

// ---------------------------------------------------------------------------------------------
// Prefill: a block takes a tile of up to 16 consecutive rows of one sequence and one kv head; its
// WAVES (4 or 8) waves take NC query heads of that kv head each (head tile WAVES * y + wave).
// Eight waves are two per SIMD: one's matrix products run under the other's softmax arithmetic.  Every page of
// keys and values is copied once per block into LDS (two buffers: the next page's loads are in
// flight while this one is multiplied) and read from there by all four waves.
// tiles: int32 [n_tiles][4] = (first row, rows, sequence, unused).  Grid: one dimension, the
// block number counting (kv head, group of four head tiles) fastest and row tiles from the last
// one down: the heavy (late) tiles of all heads start first and the short ones fill the gaps.

__device__ __forceinline__ void load_half_lds(HalfPage &hp, const uint4 *kl, const uint4 *vl, int half, int lane) {
  const int r = lane & 15, g = lane >> 4;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d = ks * 32 + g * 8;
    const int at = key_chunk(r, g, d < HD ? ks : 0);
#pragma unroll
    for (int t = 0; t < 2; ++t)
      hp.k[t][ks] = d < HD ? kl[at + (32 * half + 4 * t) * CPRK] : make_uint4(0u, 0u, 0u, 0u);
  }
  const int vat = value_chunk(r, g, half);
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) hp.v[dt] = vl[vat + 128 * dt];
}

// One page (64 keys at page_pos ..) out of LDS for the wave's NC groups of 16 columns, the softmax
// step taken over all 64 keys at once.  MASKED = false: every key of the page is visible from every
// column of the wave (the common case below the diagonal), so no score is tested and no value cut.
// PIN: keep the order written here (all fragments requested early), for a wave that has its SIMD
// to itself; otherwise the compiler reads each fragment where it is used and a second wave of
// the SIMD fills the waits.
template <int NC, bool MASKED, bool PIN>
__device__ __forceinline__ void attend_page64(WaveState<NC> &st, const bf16x8_t (&qf)[NC][KS], const uint4 *kl,
                                              const uint4 *vl, int page_pos, int col_pos, int col_lo, int key_lo,
                                              int key_hi, float scale_log2, int lane) {
  const int r = lane & 15, g = lane >> 4;
  auto read_k = [&](uint4 (&kf)[2][KS], int h) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = ks * 32 + g * 8;
      const int at = key_chunk(r, g, d < HD ? ks : 0);
#pragma unroll
      for (int t = 0; t < 2; ++t)   // A row r = 4 gg + i of score tile t is key 8 gg + 4 t + i of the 32
        kf[t][ks] = d < HD ? kl[at + (32 * h + 4 * t) * CPRK] : make_uint4(0u, 0u, 0u, 0u);
    }
  };
  floatx4_t s[NC][2][2];      // [group][half][score tile]
  auto scores = [&](const uint4 (&kf)[2][KS], int h) {
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        floatx4_t a = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) a = mfma16(as_bf16x8(kf[t][ks]), qf[c][ks], a);
        s[c][h][t] = a;
      }
  };
  uint4 vf[PIN ? DT : 1][2];
  if (PIN) {
    // All key fragments of the page are requested first, so that the wave waits for LDS once; the
    // second half's arrive while the first half is multiplied.
    uint4 kf[2][2][KS];
    read_k(kf[0], 0);
    read_k(kf[1], 1);
    __builtin_amdgcn_sched_barrier(0);
    scores(kf[0], 0);
    scores(kf[1], 1);
    __builtin_amdgcn_sched_barrier(0);
    // the value fragments travel while the softmax is worked out
#pragma unroll
    for (int dt = 0; dt < (PIN ? DT : 1); ++dt)
#pragma unroll
      for (int h = 0; h < 2; ++h) vf[dt][h] = vl[value_chunk(r, g, h) + 128 * dt];
    __builtin_amdgcn_sched_barrier(0);
  } else {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      uint4 kf[2][KS];
      read_k(kf, h);
      scores(kf, h);
    }
  }
  // this lane: column lane % 16, keys page_pos + 32 h + 8 g + e, e = 0..7
  // The running maximum only moves when a score exceeds it by more than kMaxSlack (in log2
  // units): until then the probabilities are taken relative to the old maximum (at most
  // 2^kMaxSlack, no trouble for float32 sums or bf16 operands) and the sums need no rescaling.
  // The quotient o / l at the end is the same; only the rounding differs.
  float alpha[NC];
  uint4 pb[NC][2];
  bool rescale = false;
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    float sc[16];
    float mx = -__builtin_inff();
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float v = e < 4 ? s[c][h][0][e] : s[c][h][1][e - 4];
        if (MASKED) {
          const int j = page_pos + 32 * h + 8 * g + e;
          v = (j <= col_pos && j >= col_lo) ? v : -__builtin_inff();
        }
        sc[8 * h + e] = v;
        mx = fmaxf(mx, v);
      }
    mx = max_over_lane_groups(mx);
    mx *= scale_log2;                                              // the scale is positive
    const float m_old = st.m[c];
    const bool move = mx > m_old + kMaxSlack;                      // also the first key of a column
    const float m_new = move ? mx : m_old;
    // a column that has seen no key yet keeps m = -inf: give it a finite stand-in
    const float m_use = m_new == -__builtin_inff() ? 0.f : m_new;
    alpha[c] = move ? __builtin_amdgcn_exp2f(m_old - m_use) : 1.f; // m_old = -inf gives 0
    rescale = rescale || move;
    float p[16];
    float psum = 0.f;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      p[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[e], scale_log2, -m_use));   // -inf gives 0
      psum += p[e];
    }
    st.l[c] = st.l[c] * alpha[c] + psum;
    st.m[c] = m_new;
#pragma unroll
    for (int h = 0; h < 2; ++h)
      pb[c][h] = make_uint4(pack_bf16(p[8 * h + 0], p[8 * h + 1]), pack_bf16(p[8 * h + 2], p[8 * h + 3]),
                            pack_bf16(p[8 * h + 4], p[8 * h + 5]), pack_bf16(p[8 * h + 6], p[8 * h + 7]));
  }
  // the old sums shrink by alpha; once the maxima have settled no column of the wave moves
  if (__any(rescale)) {
    // (two waves a SIMD: in place, so that the sums stay in their registers on the way that does not
    // come through here; a wave that has its SIMD to itself has registers to spare, and tying them
    // made its two-head form spill)
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (PIN) {
            st.o[c][dt][e] *= alpha[c];
          } else {
            float v = st.o[c][dt][e];
            asm volatile("v_mul_f32 %0, %0, %1" : "+v"(v) : "v"(alpha[c]));
            st.o[c][dt][e] = v;
          }
        }
  }
  if (PIN) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    uint4 va[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      uint4 a = PIN ? vf[PIN ? dt : 0][h] : vl[value_chunk(r, g, h) + 128 * dt];
      if (MASKED) {
        // values of keys outside [key_lo, key_hi] may be stale or never written: 0 * garbage must
        // not reach the accumulator
        const int k0 = page_pos + 32 * h + 8 * g;
        a = drop_first(keep_first(a, key_hi - k0 + 1), key_lo - k0);
      }
      va[h] = a;
    }
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      floatx4_t acc = mfma16(as_bf16x8(va[0]), as_bf16x8(pb[c][0]), st.o[c][dt]);
      st.o[c][dt] = mfma16(as_bf16x8(va[1]), as_bf16x8(pb[c][1]), acc);
    }
  }
}

template <int NC, int WAVES>
__global__ void __launch_bounds__(64 * WAVES, (WAVES == 8 || NC == 1) ? 2 : 1)
attn_prefill_kernel(bf16_t *__restrict__ out, const bf16_t *__restrict__ q,
                    const bf16_t *__restrict__ k_cache, const bf16_t *__restrict__ v_cache,
                    const int32_t *__restrict__ page_table, int max_pages, int n_pages_total,
                    const int32_t *__restrict__ row_pos, const int32_t *__restrict__ tiles, int n_tiles,
                    int heads_q, int heads_kv, int head_tiles, int y_per_kv, float scale_log2, int window,
                    int row_groups) {
  constexpr int kThreads = 64 * WAVES;
  constexpr int kStageLoads = (kPageChunks + kThreads - 1) / kThreads;
  extern __shared__ uint4 lds_pages[];               // [2 buffers][keys | values][kPageChunks]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n_y = heads_kv * y_per_kv;
  const int tile = n_tiles - 1 - int(blockIdx.x) / n_y, by = int(blockIdx.x) % n_y;
  const int group = heads_q / heads_kv;
  const int kvh = by / y_per_kv, yb = by - kvh * y_per_kv;
  // A block's waves cover the head tiles of its kv head; where those are fewer than half the
  // waves (groups of one or two heads), a tile is row_groups x 16 rows high and wave w takes
  // rows 16 * (w / heads_here) .. of head tile w % heads_here, so that the waves that would have
  // no head share the pages with rows of their own.
  const int heads_here = WAVES / row_groups;             // head tiles a block covers
  const int rw = wave / heads_here, hw = wave - rw * heads_here;
  const int ht = yb * heads_here + hw;                   // this wave's head tile
  const int tile_row0 = tiles[tile * 4 + 0], tile_rows = tiles[tile * 4 + 1], seq = tiles[tile * 4 + 2];
  const int n_rows = max(0, min(tile_rows - 16 * rw, 16));
  const int row0 = tile_row0 + (n_rows > 0 ? 16 * rw : 0);
  const bool active = ht < head_tiles && n_rows > 0;
  const int r = lane & 15, g = lane >> 4;
  const bool col_ok = r < n_rows;
  const int row = row0 + (col_ok ? r : 0);
  const int pos = row_pos[row];
  const int col_pos = col_ok ? pos : -1;
  const int col_lo = (window > 0 && pos >= window) ? pos - window + 1 : 0;
  // rows of a tile are consecutive positions: the first row has the lowest window start,
  // the last valid row the highest position.  tile_*: of the whole tile, which decide the pages
  // the block brings in; the others of this wave's rows, which decide what it multiplies.
  const int tile_first = row_pos[tile_row0], tile_last = row_pos[tile_row0 + tile_rows - 1];
  const int tile_lo = (window > 0 && tile_first >= window) ? tile_first - window + 1 : 0;
  const int pos_first = row_pos[row0], pos_last = row_pos[row0 + max(n_rows, 1) - 1];
  const int key_lo = (window > 0 && pos_first >= window) ? pos_first - window + 1 : 0;
  const int key_hi = pos_last;
  // first key that every row of the wave sees (the last row's window start)
  const int lo_last = (window > 0 && pos_last >= window) ? pos_last - window + 1 : 0;

  bf16x8_t qf[NC][KS];
  int head[NC];
  bool head_ok[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int hg = ht * NC + c;                      // query head within the kv head's group
    head_ok[c] = active && hg < group;
    head[c] = kvh * group + (head_ok[c] ? hg : 0);
    load_q(qf[c], q + (size_t(row) * heads_q + head[c]) * HD, col_ok && head_ok[c], lane);
  }
  WaveState<NC> st;
  init_state<NC>(st);

  const int32_t *pt = page_table + size_t(seq) * max_pages;
  const int pg_hi = min(tile_last / SB_PAGE, max_pages - 1);
  // the next page from pg on that the table holds (uniform over the block)
  auto next_valid = [&](int pg) {
    while (pg <= pg_hi) {
      const int page = pt[pg];
      if (page >= 0 && page < n_pages_total) break;
      ++pg;
    }
    return pg;
  };
  // Two register sets: while page p is multiplied out of LDS, page p + 1 waits in one set (its
  // loads went out a page earlier) and the loads of page p + 2 go out into the other.
  bf16x8_t stage_k[2][kStageLoads], stage_v[2][kStageLoads];
  auto issue = [&](auto SET, int pg) {
    constexpr int set = decltype(SET)::value;
    const size_t off = (size_t(pt[pg]) * heads_kv + kvh) * SB_PAGE * HD;
    const bf16x8_t *kp = reinterpret_cast<const bf16x8_t *>(k_cache + off);
    const bf16x8_t *vp = reinterpret_cast<const bf16x8_t *>(v_cache + off);
#pragma unroll
    for (int j = 0; j < kStageLoads; ++j) {
      const int id = tid + kThreads * j;
      if (kPageChunks % kThreads == 0 || id < kPageChunks) {
        stage_k[set][j] = kp[id];
        stage_v[set][j] = vp[id];
      }
    }
  };
  auto store = [&](auto SET, int buf) {
    constexpr int set = decltype(SET)::value;
    bf16x8_t *kl = reinterpret_cast<bf16x8_t *>(lds_pages) + buf * 2 * kPageChunks, *vl = kl + kPageChunks;
#pragma unroll
    for (int j = 0; j < kStageLoads; ++j) {
      const int id = tid + kThreads * j;
      if (kPageChunks % kThreads == 0 || id < kPageChunks) {
        kl[id] = stage_k[set][j];      // the cache keeps a page in the order LDS wants it
        vl[id] = stage_v[set][j];
      }
    }
  };
  using Set0 = std::integral_constant<int, 0>;
  using Set1 = std::integral_constant<int, 1>;
  // Page pg out of LDS buffer buf, for a wave that has a head.
  auto attend = [&](int pg, int buf) __attribute__((always_inline)) {
    const uint4 *kl = lds_pages + buf * 2 * kPageChunks, *vl = kl + kPageChunks;
    const int page_pos = pg * SB_PAGE;
    if (page_pos > key_hi || page_pos + SB_PAGE - 1 < key_lo) return;      // a page of other waves' rows only
    if (HD > 128) {
      // too many fragments for the registers at once: half a page at a time
      HalfPage h;
      if (!(page_pos > key_hi || page_pos + 31 < key_lo)) {
        load_half_lds(h, kl, vl, 0, lane);
        attend_half<NC>(st, qf, h, page_pos, col_pos, col_lo, key_lo, key_hi, scale_log2, lane);
      }
      if (!(page_pos + 32 > key_hi || page_pos + 63 < key_lo)) {
        load_half_lds(h, kl, vl, 1, lane);
        attend_half<NC>(st, qf, h, page_pos + 32, col_pos, col_lo, key_lo, key_hi, scale_log2, lane);
      }
    } else if (page_pos + SB_PAGE - 1 <= pos_first && page_pos >= lo_last) {
      attend_page64<NC, false, WAVES == 4 && NC != 1>(st, qf, kl, vl, page_pos, col_pos, col_lo, key_lo, key_hi,
                                                      scale_log2, lane);
    } else {
      attend_page64<NC, true, WAVES == 4 && NC != 1>(st, qf, kl, vl, page_pos, col_pos, col_lo, key_lo, key_hi,
                                                     scale_log2, lane);
    }
  };

  int pg = next_valid(tile_lo / SB_PAGE);                     // the page being multiplied
  // Waves without a head (the block's last ones, when the kv head's group does not fill it) bring
  // the pages in alone, straight into LDS (a load of 64 lanes x 16 bytes lands in 1 KB of
  // consecutive LDS, and a page lies in the cache as LDS wants it): the waves that multiply then
  // issue nothing for it, and a page comes through no registers.  While page p is multiplied out
  // of one buffer, page p + 1 arrives in the other.  Where every wave has a head, blocks of four
  // waves with one head per wave, or with heads of more than 128, share these loads among all
  // waves (measured against the path through registers below, 8,192 tokens, groups of 4: head
  // size 64 5 % faster, 96 22 %, 128 10 %, 144 12 %, 192 2.4 times, 256 7 times, whose two sets of
  // staging registers no longer fit; two and more heads per wave at head sizes up to 128, and eight
  // waves at those head sizes, are 5 to 11 % slower with them and keep the registers; eight waves
  // with bigger heads have no registers to keep pages in).
  constexpr bool kAllBring = (WAVES == 4 && (NC == 1 || HD > 128)) || (WAVES == 8 && HD > 128);
  // (tiles of several row groups: every wave has a head)
  const int n_busy = row_groups > 1 ? WAVES : min(head_tiles - yb * WAVES, WAVES), n_stagers = WAVES - n_busy;
  if (n_stagers > 0 || kAllBring) {
    typedef __attribute__((address_space(3))) uint4 *lds_ptr_t;
    constexpr int kWaveLoads = kPageChunks / 64;       // per page of keys, and of values
    auto bring = [&](int pg_in, int buf_in) __attribute__((always_inline)) {
      if (n_stagers > 0 && wave < n_busy) return;
      const int first_load = n_stagers > 0 ? wave - n_busy : wave, step_load = n_stagers > 0 ? n_stagers : WAVES;
      const size_t off = (size_t(pt[pg_in]) * heads_kv + kvh) * SB_PAGE * HD;
      const __amdgpu_buffer_rsrc_t rsrc_k = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<bf16_t *>(k_cache + off), 0, uint32_t(kPageChunks * 16), 0x00020000);
      const __amdgpu_buffer_rsrc_t rsrc_v = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<bf16_t *>(v_cache + off), 0, uint32_t(kPageChunks * 16), 0x00020000);
      for (int i = first_load; i < kWaveLoads; i += step_load) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_k, (lds_ptr_t)(lds_pages) + buf_in * 2 * kPageChunks + i * 64,
                                                 16, lane * 16, i * 1024, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rsrc_v, (lds_ptr_t)(lds_pages) + buf_in * 2 * kPageChunks + kPageChunks + i * 64, 16, lane * 16, i * 1024,
            0, 0);
      }
    };
    // a wave's own loads have landed, and after the barrier everybody's (a bare barrier between
    // two fences for the compiler: __syncthreads() says more than is needed)
    auto landed = [&]() __attribute__((always_inline)) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
    };
    if (pg <= pg_hi) bring(pg, 0);
    landed();
    int buf = 0;
    while (pg <= pg_hi) {
      const int pg_next = next_valid(pg + 1);
      if (pg_next <= pg_hi) bring(pg_next, buf ^ 1);
      if (active) attend(pg, buf);
      landed();
      pg = pg_next;
      buf ^= 1;
    }
  } else {
  int pg1 = pg <= pg_hi ? next_valid(pg + 1) : pg;            // the page after it
  if (pg <= pg_hi) issue(Set0{}, pg);
  if (pg1 <= pg_hi) issue(Set1{}, pg1);
  if (pg <= pg_hi) store(Set0{}, 0);
  __syncthreads();
  int buf = 0;
  // One page: FREE is the register set whose page already lies in LDS.
  auto step = [&](auto FREE) {
    constexpr int free_set = decltype(FREE)::value;
    using SetFree = std::integral_constant<int, free_set>;
    using SetHeld = std::integral_constant<int, free_set ^ 1>;
    const int pg2 = pg1 <= pg_hi ? next_valid(pg1 + 1) : pg1;
    if (pg2 <= pg_hi) issue(SetFree{}, pg2);
    if (active) attend(pg, buf);
    if (pg1 <= pg_hi) store(SetHeld{}, buf ^ 1);
    __syncthreads();
    pg = pg1;
    pg1 = pg2;
    buf ^= 1;
  };
  while (pg <= pg_hi) {
    step(Set0{});
    if (pg > pg_hi) break;
    step(Set1{});
  }
  }
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    float l = st.l[c];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (!col_ok || !head_ok[c]) continue;
    const float inv = l > 0.f ? 1.f / l : 0.f;
    bf16_t *orow = out + (size_t(row) * heads_q + head[c]) * HD;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const uint2 v = make_uint2(pack_bf16(st.o[c][dt][0] * inv, st.o[c][dt][1] * inv),
                                 pack_bf16(st.o[c][dt][2] * inv, st.o[c][dt][3] * inv));
      *reinterpret_cast<uint2 *>(orow + dt * 16 + 4 * g) = v;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Prefill in tiles of 32 rows, for long prompts: a block takes up to 32 consecutive rows of one
// sequence and one kv head, wave w of its eight the query head w of that kv head's group (waves
// past the group bring the pages in), and the products are v_mfma_f32_32x32x16_bf16:
//   S^T[32 keys][32 rows] = K[32 keys][16 d] . Q^T[16 d][32 rows]      A = K rows out of LDS, B = Q rows in registers
//   O^T[32 d][32 rows]   += V^T[32 d][16 keys] . P[16 keys][32 rows]   A = V^T rows out of LDS, B = P in registers
// A page that lies in LDS serves twice the rows it serves in the 16-row kernel above, and every
// fragment read from LDS feeds twice the products: per product half the LDS traffic, half the
// copies into LDS and half the barriers.
//
// Lane l of such a product holds for A row l % 32, k = 8 (l / 32) .. + 7, for B column l % 32 and
// the same k, and of the result column l % 32, rows 8 q + 4 (l / 32) + e for q, e = 0 .. 3
// (register 4 q + e).  Which key a row of the score product stands for is this kernel's choice.
// Row 8 q + 4 c + e of the tile of keys 32 t .. 32 t + 31 is key
//   32 t + 16 c + 8 (q & 1) + 4 (q >> 1) + e:
// the half of the wave c = l / 32 then holds, in registers 4 q .. 4 q + 3, the keys of the chunks
// of eight 4 t + 2 c and 4 t + 2 c + 1 (lower halves in q = 0 and 1, upper halves in q = 2 and 3),
// and a step of sixteen keys of the second product takes chunk 4 t + j from half 0 and 4 t + 2 + j
// from half 1 (j = 0, 1): the eight k of a lane are one chunk of the value row, as the cache keeps
// it, and P never leaves the registers.  The sixteen lanes that LDS serves together read key rows
// that differ in bits 0, 1, 3 and 4, which the cache's order of a row's chunks (sb_key_swizzle)
// spreads over all banks.
constexpr int DS32 = HD / 16;        // k-steps (16 d) of the score product
constexpr int DT32 = HD >= 32 ? HD / 32 : 1;        // 32-row tiles of O^T
constexpr bool kTallOk = HD % 32 == 0 && HD <= 128;

struct TallState {
  floatx16_t o[DT32];
  float m, l;               // running maximum of the lane's column (log2 domain), the lane's share of the sum
};

// The maximum of a value over the two halves of the wave (lanes l and l ^ 32), in both.
__device__ __forceinline__ float max_over_halves(float v) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const auto p = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const uint32_t p0 = p[0], p1 = p[1];
  return fmaxf(__builtin_bit_cast(float, p0), __builtin_bit_cast(float, p1));
}

// Key (within its page) of register i = 4 q + e of score tile t in half c of the wave.
__device__ __forceinline__ constexpr int tall_key(int t, int i, int c) {
  return 32 * t + 16 * c + 8 * ((i >> 2) & 1) + 4 * (i >> 3) + (i & 3);
}

// One page out of LDS.  masked (uniform over the block): some key of the page is hidden from some
// row, so every score is tested; the values of keys that no row of the tile may see have been
// zeroed in LDS by then (they may be stale or never written, and 0 * garbage must not reach the sums).
__device__ __forceinline__ void attend_page_tall(TallState &st, const bf16x8_t (&qf)[DS32], const uint4 *kl,
                                                 const uint4 *vl, int page_pos, bool masked, int col_pos, int col_lo,
                                                 float scale_log2, int lane) {
  const int m = lane & 31, c = lane >> 5;
  // this lane's key row of a tile: row m = 8 q + 4 cc + e of the product
  const int q_ = m >> 3, cc = (m >> 2) & 1;
  const int krow = 16 * cc + 8 * (q_ & 1) + 4 * (q_ >> 1) + (m & 3);
  const int kswz = sb_key_swizzle(krow, HD);             // bits 0, 1, 3, 4 of the key: the same for krow + 32
  floatx16_t s[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    floatx16_t acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
    for (int ds = 0; ds < DS32; ++ds)
      acc = mfma32(as_bf16x8(kl[(32 * t + krow) * CPRK + ((2 * ds + c) ^ kswz)]), qf[ds], acc);
    s[t] = acc;
  }
  // the first tile's fragments are asked for at once, the second tile's while the first is multiplied
  __builtin_amdgcn_sched_group_barrier(0x100, DS32, 0);
#pragma unroll
  for (int ds = 0; ds < DS32; ++ds) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
  }
  __builtin_amdgcn_sched_group_barrier(0x008, DS32, 0);
  __builtin_amdgcn_sched_barrier(0);          // (the value fragments are not asked for before the scores are done)
  if (masked) {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int j = page_pos + tall_key(t, i, c);
        s[t][i] = (j <= col_pos && j >= col_lo) ? s[t][i] : -__builtin_inff();
      }
  }
  float mx = -__builtin_inff();
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[t][i]);
  mx = max_over_halves(mx) * scale_log2;                 // the scale is positive
  // The running maximum only moves when a score exceeds it by more than kMaxSlack (see attend_page64).
  const float m_old = st.m;
  const bool move = mx > m_old + kMaxSlack;              // also the first key of a column
  const float m_new = move ? mx : m_old;
  const float m_use = m_new == -__builtin_inff() ? 0.f : m_new;
  const float alpha = move ? __builtin_amdgcn_exp2f(m_old - m_use) : 1.f;      // m_old = -inf gives 0
  float psum = 0.f;
  uint4 pb[2][2];                                        // [tile][j]: the chunk 4 t + 2 c + j of the page
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    float p[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      p[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][i], scale_log2, -m_use));    // -inf gives 0
      psum += p[i];
    }
#pragma unroll
    for (int j = 0; j < 2; ++j)
      pb[t][j] = make_uint4(pack_bf16(p[4 * j + 0], p[4 * j + 1]), pack_bf16(p[4 * j + 2], p[4 * j + 3]),
                            pack_bf16(p[8 + 4 * j + 0], p[8 + 4 * j + 1]), pack_bf16(p[8 + 4 * j + 2], p[8 + 4 * j + 3]));
  }
  st.l = st.l * alpha + psum;
  st.m = m_new;
  if (__any(move)) {
#pragma unroll
    for (int dt = 0; dt < DT32; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) st.o[dt][i] *= alpha;
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int dt = 0; dt < DT32; ++dt) {
    const int d = 32 * dt + m;
    floatx16_t acc = st.o[dt];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        acc = mfma32(as_bf16x8(vl[v_slot(d, 4 * t + 2 * c + j)]), as_bf16x8(pb[t][j]), acc);
    st.o[dt] = acc;
  }
  // four fragments ahead of the products
  __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
  for (int i = 0; i < 4 * DT32 - 4; ++i) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
  }
  __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
  __builtin_amdgcn_sched_barrier(0);
}

// tiles: int32 [n_tiles][4] = (first row, rows <= 32, sequence, unused).  Grid as above: the block
// number counts (kv head, group of eight heads) fastest and row tiles from the last one down.
template <bool OK>      // kTallOk: head sizes that this form does not take compile to nothing
__global__ void __launch_bounds__(512, 2)
attn_prefill_tall_kernel(bf16_t *__restrict__ out, const bf16_t *__restrict__ q, const bf16_t *__restrict__ k_cache,
                         const bf16_t *__restrict__ v_cache, const int32_t *__restrict__ page_table, int max_pages,
                         int n_pages_total, const int32_t *__restrict__ row_pos, const int32_t *__restrict__ tiles,
                         int n_tiles, int heads_q, int heads_kv, int y_per_kv, float scale_log2, int window) {
  if constexpr (OK) {
  constexpr int WAVES = 8;
  extern __shared__ uint4 lds_pages[];               // [2 buffers][keys | values][kPageChunks]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n_y = heads_kv * y_per_kv;
  const int tile = n_tiles - 1 - int(blockIdx.x) / n_y, by = int(blockIdx.x) % n_y;
  const int group = heads_q / heads_kv;
  const int kvh = by / y_per_kv, yb = by - kvh * y_per_kv;
  const int hg = yb * WAVES + wave;                  // this wave's query head within the group
  const int n_busy = min(group - yb * WAVES, WAVES), n_stagers = WAVES - n_busy;
  const bool active = wave < n_busy;
  const int head = kvh * group + (active ? hg : 0);
  const int tile_row0 = tiles[tile * 4 + 0], n_rows = tiles[tile * 4 + 1], seq = tiles[tile * 4 + 2];
  const int n = lane & 31, c = lane >> 5;
  const bool col_ok = n < n_rows;
  const int row = tile_row0 + (col_ok ? n : 0);
  const int pos = row_pos[row];
  const int col_pos = col_ok ? pos : -1;
  const int col_lo = (window > 0 && pos >= window) ? pos - window + 1 : 0;
  // rows of a tile are consecutive positions: the first row has the lowest window start, the
  // last one the highest position
  const int pos_first = row_pos[tile_row0], pos_last = row_pos[tile_row0 + n_rows - 1];
  const int key_lo = (window > 0 && pos_first >= window) ? pos_first - window + 1 : 0;
  const int key_hi = pos_last;
  const int lo_last = (window > 0 && pos_last >= window) ? pos_last - window + 1 : 0;

  bf16x8_t qf[DS32];
  {
    const bf16_t *qrow = q + (size_t(row) * heads_q + head) * HD;
#pragma unroll
    for (int ds = 0; ds < DS32; ++ds) qf[ds] = as_bf16x8(ld16(qrow + 16 * ds + 8 * c, col_ok && active));
  }
  TallState st;
#pragma unroll
  for (int dt = 0; dt < DT32; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) st.o[dt][i] = 0.f;
  st.m = -__builtin_inff();
  st.l = 0.f;

  const int32_t *pt = page_table + size_t(seq) * max_pages;
  const int pg_hi = min(pos_last / SB_PAGE, max_pages - 1);
  auto next_valid = [&](int pg) {
    while (pg <= pg_hi) {
      const int page = pt[pg];
      if (page >= 0 && page < n_pages_total) break;
      ++pg;
    }
    return pg;
  };
  // Pages come straight into LDS (a load of 64 lanes x 16 bytes lands in 1 KB of consecutive LDS,
  // and a page lies in the cache as LDS wants it): by the waves without a head when the group
  // leaves some, else by all waves in turns.  While page p is multiplied out of one buffer, page
  // p + 1 arrives in the other.
  typedef __attribute__((address_space(3))) uint4 *lds_ptr_t;
  constexpr int kWaveLoads = kPageChunks / 64;       // per page of keys, and of values
  auto bring = [&](int pg_in, int buf_in) __attribute__((always_inline)) {
    if (n_stagers > 0 && wave < n_busy) return;
    const int first_load = n_stagers > 0 ? wave - n_busy : wave, step_load = n_stagers > 0 ? n_stagers : WAVES;
    const size_t off = (size_t(pt[pg_in]) * heads_kv + kvh) * SB_PAGE * HD;
    const __amdgpu_buffer_rsrc_t rsrc_k = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16_t *>(k_cache + off), 0, uint32_t(kPageChunks * 16), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_v = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16_t *>(v_cache + off), 0, uint32_t(kPageChunks * 16), 0x00020000);
    for (int i = first_load; i < kWaveLoads; i += step_load) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_k, (lds_ptr_t)(lds_pages) + buf_in * 2 * kPageChunks + i * 64, 16,
                                               lane * 16, i * 1024, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rsrc_v, (lds_ptr_t)(lds_pages) + buf_in * 2 * kPageChunks + kPageChunks + i * 64, 16, lane * 16, i * 1024, 0, 0);
    }
  };
  auto landed = [&]() __attribute__((always_inline)) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  int pg = next_valid(key_lo / SB_PAGE);
  if (pg <= pg_hi) bring(pg, 0);
  landed();
  int buf = 0;
  while (pg <= pg_hi) {
    const int pg_next = next_valid(pg + 1);
    if (pg_next <= pg_hi) bring(pg_next, buf ^ 1);
    {
      uint4 *kl = lds_pages + buf * 2 * kPageChunks, *vl = kl + kPageChunks;
      const int page_pos = pg * SB_PAGE;
      const bool masked = !(page_pos + SB_PAGE - 1 <= pos_first && page_pos >= lo_last);
      if (masked) {
        // (rare: the pages on the diagonal and at a window's edge)  The values of keys outside
        // [key_lo, key_hi] go to zero in LDS, all threads of the block taking a share.
        for (int idx = tid; idx < kPageChunks; idx += 64 * WAVES) {
          const int d = idx >> 3, chunk = (idx & 7) ^ ((d >> 1) & 7);
          const int k0 = page_pos + 8 * chunk;
          vl[idx] = drop_first(keep_first(vl[idx], key_hi - k0 + 1), key_lo - k0);
        }
        __syncthreads();
      }
      if (active) attend_page_tall(st, qf, kl, vl, page_pos, masked, col_pos, col_lo, scale_log2, lane);
    }
    landed();
    pg = pg_next;
    buf ^= 1;
  }
  float l = st.l;
  {
    const uint32_t u = __builtin_bit_cast(uint32_t, l);
    const auto p = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const uint32_t p0 = p[0], p1 = p[1];
    l = __builtin_bit_cast(float, p0) + __builtin_bit_cast(float, p1);
  }
  if (!col_ok || !active) return;
  const float inv = l > 0.f ? 1.f / l : 0.f;
  bf16_t *orow = out + (size_t(row) * heads_q + head) * HD;
#pragma unroll
  for (int dt = 0; dt < DT32; ++dt)
#pragma unroll
    for (int qq = 0; qq < 4; ++qq) {
      const uint2 v = make_uint2(pack_bf16(st.o[dt][4 * qq + 0] * inv, st.o[dt][4 * qq + 1] * inv),
                                 pack_bf16(st.o[dt][4 * qq + 2] * inv, st.o[dt][4 * qq + 3] * inv));
      *reinterpret_cast<uint2 *>(orow + 32 * dt + 8 * qq + 4 * c) = v;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Decode: one row per sequence.  Block (chunk, kv head x head tile, sequence); wave w of the
// block takes page 4 * chunk + w; columns are the query heads of the kv head.
//
// Partial results, when a row's keys span several chunks, go to
//   part_o  float [seqs][tiles][n_chunks][HD][16]   (unnormalised sums, column fastest)
//   part_ml float [seqs][tiles][n_chunks][2][16]    (maximum, sum)
// and are merged by attn_decode_merge_kernel (up to 16 chunks, in ascending order) or
// attn_decode_merge_many_kernel.  (Merging in the block
// that finishes last was tried and dropped: the device-scope fences it needs write back and
// invalidate whole L2 caches on this multi-die GPU and cost far more than the second launch.)

// Decode grids have one dimension, the block number counting the (kv head x head tile) fastest,
// then the sequence, the chunk of pages slowest.  Blocks go to the GPU's eight dies in turn by
// their number; which chunks have work depends on the sequences' lengths, and with the chunk as
// the fastest dimension the chunks past a row's end would leave whole dies idle (nine busy chunks
// of sixteen put two ninths of the work on one die).
struct DecodeBlock {
  int chunk, seq, tile;   // tile = kv head * head tiles + head tile
};
__device__ __forceinline__ DecodeBlock decode_block(int tiles, int n_seqs) {
  const int per_chunk = tiles * n_seqs;
  DecodeBlock b;
  b.chunk = int(blockIdx.x) / per_chunk;
  const int rem = int(blockIdx.x) - b.chunk * per_chunk;
  b.seq = rem / tiles;
  b.tile = rem - b.seq * tiles;
  return b;
}

// The end of a decode block: the waves' running sums meet in LDS and are merged in wave order
// (thread e owns (d, column), column fastest); the result goes to `out` when the row's keys lie
// in this chunk alone, else to the chunk's place in the partial buffers.
__device__ __forceinline__ void finish_decode_block(const WaveState<1> &st, float (*lds_o)[HD * 16], float (*lds_m)[16],
                                                    float (*lds_l)[16], bf16_t *__restrict__ out,
                                                    float *__restrict__ part_o, float *__restrict__ part_ml,
                                                    int wave, int lane, int chunk, bool alone, int seq, int kvh,
                                                    int ht, int group, int heads_q, int n_chunks,
                                                    size_t tile_index) {
  const int r = lane & 15, g = lane >> 4;
  float l = st.l[0];
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 4; ++i) lds_o[wave][(dt * 16 + 4 * g + i) * 16 + r] = st.o[0][dt][i];
  if (g == 0) {
    lds_m[wave][r] = st.m[0];
    lds_l[wave][r] = l;
  }
  __syncthreads();
  // merge the four waves (pages in ascending order); thread e owns (d, col), column fastest
  float *po = part_o + (tile_index * n_chunks) * (HD * 16);
  float *pml = part_ml + (tile_index * n_chunks) * 32;
  for (int e = threadIdx.x; e < HD * 16; e += 256) {
    const int c = e & 15, d = e >> 4;
    float m = -__builtin_inff();
#pragma unroll
    for (int w = 0; w < 4; ++w) m = fmaxf(m, lds_m[w][c]);
    const float m_use = m == -__builtin_inff() ? 0.f : m;
    float o = 0.f, lsum = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = __builtin_amdgcn_exp2f(lds_m[w][c] - m_use);
      o += lds_o[w][e] * f;
      lsum += lds_l[w][c] * f;
    }
    if (alone) {
      const int hh = ht * 16 + c;
      if (hh < group)
        out[(size_t(seq) * heads_q + kvh * group + hh) * HD + d] = f32_to_bf16(lsum > 0.f ? o / lsum : 0.f);
    } else if (ht * 16 + c < group) {
      po[size_t(chunk) * (HD * 16) + e] = o;
      if (d == 0) {
        pml[size_t(chunk) * 32 + c] = m;
        pml[size_t(chunk) * 32 + 16 + c] = lsum;
      }
    }
  }
}

// ---- decode with the rotation and the store folded in ------------------------------------------
// A decode step's queries come out of the qkv product as float32 rows [queries | keys | values]
// (in K slices that are still to be added, plus a bias), have to be rotated and rounded, and the
// row's key and value have to go into the cache before the row attends.  Done by a kernel of its
// own that is a launch more per layer; folded in here, every block builds the queries of its heads
// itself (sums, bias, rotation: the arithmetic and the order of sb_rope_kv_store, so the same
// bits), and the block whose pages hold the row's own position also builds the new key and value,
// stores them, and only then reads that page (a fence and a barrier within the block: the
// stores and the loads come from the same CU).
struct RopeArgs {
  const float *qkv;            // [n_slices][n_seqs][row_stride]
  int row_stride, n_slices;
  size_t slice_stride;
  const float *bias;           // [row] or NULL
  const float *inv_freq;       // [rot_dims / 2] or NULL: no rotation
  const float *freq_factors;   // [rot_dims / 2] or NULL
  int rot_dims;                // a multiple of 16
  int store;                   // keys and values go into the cache (0: a layer that reads another's)
};

// Eight consecutive elements e0 .. e0+7 of sequence seq's qkv row, and the eight from p0 on (the
// partners in the rotation, or anything valid if there are none): slices in ascending order,
// then the bias.  The loads of four slices of both go out before the first sum (a loop that adds
// slice after slice waits for memory once per slice: three slices and a partner cost the kernel
// six trips to L2 in a row); a slice past the last is the last once more and is not added, so
// the sums have the bits of the loop.  More than four slices: a second round of four.
struct Row8 { float4 lo, hi; };
__device__ __forceinline__ void add_if(Row8 &a, const Row8 &c, bool use) {
  a.lo.x = use ? a.lo.x + c.lo.x : a.lo.x; a.lo.y = use ? a.lo.y + c.lo.y : a.lo.y;
  a.lo.z = use ? a.lo.z + c.lo.z : a.lo.z; a.lo.w = use ? a.lo.w + c.lo.w : a.lo.w;
  a.hi.x = use ? a.hi.x + c.hi.x : a.hi.x; a.hi.y = use ? a.hi.y + c.hi.y : a.hi.y;
  a.hi.z = use ? a.hi.z + c.hi.z : a.hi.z; a.hi.w = use ? a.hi.w + c.hi.w : a.hi.w;
}
__device__ __forceinline__ Row8 load8(const float *p) {
  return Row8{*reinterpret_cast<const float4 *>(p), *reinterpret_cast<const float4 *>(p + 4)};
}
// What qkv8x2_issue has asked for: the first four slices and the bias of both runs of eight.
struct Raw8x2 {
  Row8 cx[4], cp[4], bx, bp;
  size_t e0, p0;
};
__device__ __forceinline__ void qkv8x2_issue(Raw8x2 &raw, const RopeArgs &ra, int seq, size_t e0, size_t p0) {
  const float *rx = ra.qkv + size_t(seq) * ra.row_stride + e0, *rp = ra.qkv + size_t(seq) * ra.row_stride + p0;
  raw.e0 = e0;
  raw.p0 = p0;
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    const size_t so = size_t(min(s, ra.n_slices - 1)) * ra.slice_stride;
    raw.cx[s] = load8(rx + so);
    raw.cp[s] = load8(rp + so);
  }
  // 16-byte aligned like the row: e0 and p0 are multiples of 8 (without a bias: the row itself, not added)
  raw.bx = load8(ra.bias ? ra.bias + e0 : rx);
  raw.bp = load8(ra.bias ? ra.bias + p0 : rp);
}
__device__ __forceinline__ void qkv8x2_finish(float (&x)[8], float (&p)[8], const Raw8x2 &raw, const RopeArgs &ra, int seq) {
  Row8 ax = raw.cx[0], ap = raw.cp[0];
#pragma unroll
  for (int s = 1; s < 4; ++s) {
    add_if(ax, raw.cx[s], s < ra.n_slices);
    add_if(ap, raw.cp[s], s < ra.n_slices);
  }
  if (ra.n_slices > 4) {     // uniform
    const float *rx = ra.qkv + size_t(seq) * ra.row_stride + raw.e0, *rp = ra.qkv + size_t(seq) * ra.row_stride + raw.p0;
    Row8 cx[4], cp[4];
#pragma unroll
    for (int s = 4; s < 8; ++s) {
      const size_t so = size_t(min(s, ra.n_slices - 1)) * ra.slice_stride;
      cx[s - 4] = load8(rx + so);
      cp[s - 4] = load8(rp + so);
    }
#pragma unroll
    for (int s = 4; s < 8; ++s) {
      add_if(ax, cx[s - 4], s < ra.n_slices);
      add_if(ap, cp[s - 4], s < ra.n_slices);
    }
  }
  add_if(ax, raw.bx, ra.bias != nullptr);
  add_if(ap, raw.bp, ra.bias != nullptr);
  x[0] = ax.lo.x; x[1] = ax.lo.y; x[2] = ax.lo.z; x[3] = ax.lo.w; x[4] = ax.hi.x; x[5] = ax.hi.y; x[6] = ax.hi.z; x[7] = ax.hi.w;
  p[0] = ap.lo.x; p[1] = ap.lo.y; p[2] = ap.lo.z; p[3] = ap.lo.w; p[4] = ap.hi.x; p[5] = ap.hi.y; p[6] = ap.hi.z; p[7] = ap.hi.w;
}

// The same sums slice after slice, with few registers: for the items past a block's first 256,
// which are fetched while the page's fragments are held (only a group of fifteen or sixteen
// heads has any).
__device__ __forceinline__ void qkv8_in_turn(float (&v)[8], const RopeArgs &ra, int seq, size_t e0) {
  const float *r = ra.qkv + size_t(seq) * ra.row_stride + e0;
  Row8 a = load8(r);
  for (int s = 1; s < ra.n_slices; ++s) add_if(a, load8(r + s * ra.slice_stride), true);
  if (ra.bias) add_if(a, load8(ra.bias + e0), true);
  v[0] = a.lo.x; v[1] = a.lo.y; v[2] = a.lo.z; v[3] = a.lo.w; v[4] = a.hi.x; v[5] = a.hi.y; v[6] = a.hi.z; v[7] = a.hi.w;
}

// Eight floats rounded as sb_rope_kv_store rounds (to nearest even, a NaN stays one), packed.
__device__ __forceinline__ uint4 pack8(const float (&y)[8]) {
  return make_uint4(uint32_t(f32_to_bf16(y[0])) | uint32_t(f32_to_bf16(y[1])) << 16,
                    uint32_t(f32_to_bf16(y[2])) | uint32_t(f32_to_bf16(y[3])) << 16,
                    uint32_t(f32_to_bf16(y[4])) | uint32_t(f32_to_bf16(y[5])) << 16,
                    uint32_t(f32_to_bf16(y[6])) | uint32_t(f32_to_bf16(y[7])) << 16);
}

constexpr int kQStride = HD / 8 + 1;     // 16-byte units of a staged query row: one of padding against bank conflicts
constexpr int kPerHead = HD / 8;         // work items (of eight elements) per head

// LDS of the folded form: the block's cosines and sines, and the rotated, rounded queries of its
// (up to 16) heads, which the four waves then read as fragments.
struct RopeShared {
  float cs[HD / 2], sn[HD / 2];
  uint4 q[16 * kQStride];
  uint4 k[HD / 8];      // the row's own key, rotated and rounded
  bf16_t v[HD];         // and its value
  int page_of_wave[4];  // the page numbers the block's waves have looked up (kernels with a page a wave)
};

// Work item `it` of a block of the folded form: eight elements d0 .. d0+7 of one head of the qkv
// row; items [0, group * HD/8) are the queries of the block's heads, the next HD/8 the key of its
// kv head, the last HD/8 the value.  x: the elements, p: their partners in the rotation (d0 a
// multiple of 8, half and rot_dims multiples of 8: the eight lie on one side of every border).
struct RopeItem {
  float x[8], p[8];
};
__device__ __forceinline__ size_t item_head(int it, int n_q, int kvh, int group, int heads_q, int heads_kv) {
  if (it < n_q) return size_t(kvh * group + it / kPerHead) * HD;
  return size_t((it < n_q + kPerHead ? heads_q : heads_q + heads_kv) + kvh) * HD;
}
__device__ __forceinline__ void item_offsets(size_t &e0, size_t &p0, bool &paired, int it, int n_q, int kvh, int group,
                                             int heads_q, int heads_kv, int half) {
  const size_t hoff = item_head(it, n_q, kvh, group, heads_q, heads_kv);
  const int d0 = (it < n_q ? it % kPerHead : (it - n_q) % kPerHead) * 8;
  paired = it < n_q + kPerHead && d0 < 2 * half;
  e0 = hoff + d0;
  // an item without a partner (a value, an element past the rotated ones) stands in for it itself
  p0 = hoff + (!paired ? d0 : d0 < half ? d0 + half : d0 - half);
}
// a thread's first item: all its loads at once ...
__device__ __forceinline__ void fetch_item(RopeItem &v, const RopeArgs &ra, int seq, int it, int n_q, int kvh,
                                           int group, int heads_q, int heads_kv, int half) {
  size_t e0, p0;
  bool paired;
  item_offsets(e0, p0, paired, it, n_q, kvh, group, heads_q, heads_kv, half);
  Raw8x2 raw;
  qkv8x2_issue(raw, ra, seq, e0, p0);
  qkv8x2_finish(v.x, v.p, raw, ra, seq);
}
// ... and a later one, slice after slice
__device__ __forceinline__ void fetch_item_in_turn(RopeItem &v, const RopeArgs &ra, int seq, int it, int n_q, int kvh,
                                                   int group, int heads_q, int heads_kv, int half) {
  size_t e0, p0;
  bool paired;
  item_offsets(e0, p0, paired, it, n_q, kvh, group, heads_q, heads_kv, half);
  qkv8_in_turn(v.x, ra, seq, e0);
  if (paired) qkv8_in_turn(v.p, ra, seq, p0);
}
// The item's eight results: rotated queries and keys, the value as it is.
__device__ __forceinline__ void finish_item(float (&y)[8], const RopeItem &v, int it, int n_q, int half,
                                            const float *cs, const float *sn) {
  const int d0 = (it < n_q ? it % kPerHead : (it - n_q) % kPerHead) * 8;
  if (it >= n_q + kPerHead || d0 >= 2 * half) {
#pragma unroll
    for (int i = 0; i < 8; ++i) y[i] = v.x[i];
    return;
  }
  const bool low = d0 < half;
  const int i0 = low ? d0 : d0 - half;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    float y0, y1;
    if (low) rotate_pair(v.x[i], v.p[i], cs[i0 + i], sn[i0 + i], y0, y1);
    else rotate_pair(v.p[i], v.x[i], cs[i0 + i], sn[i0 + i], y0, y1);
    y[i] = low ? y0 : y1;
  }
}

// The block's queries into LDS, and in the block whose pages hold the row's own position (`mine`)
// the row's key and value into the cache and into LDS.  All threads of the block; `first` holds
// the thread's first item and `freq` the frequency of the angle it works out, whose loads went
// out at the kernel's start (they depend on the block's and the thread's number only).  Ends with
// a barrier after which the queries, the key and the value can be read from LDS; with
// `visible` the stored key and value are also visible to the block's own loads from the cache
// (a wait for the stores: the kernels that can patch their fragments from LDS do without).
__device__ __forceinline__ void rope_store(RopeShared &sh, const RopeItem &first, float freq, const RopeArgs &ra,
                                           int seq, int pos, int kvh, int group, int heads_q, int heads_kv,
                                           bool mine, bool visible, bf16_t *k_cache, bf16_t *v_cache,
                                           const int32_t *page_table, int max_pages, int n_pages_total,
                                           int first_page_of_block = -1) {
  const int half = ra.inv_freq ? ra.rot_dims / 2 : 0;
  if (int(threadIdx.x) < 2 * half) {
    const int j = threadIdx.x, i = j < half ? j : j - half;
    float theta = float(pos) * freq;
    if (ra.freq_factors) theta = theta / ra.freq_factors[i];       // as sb_rope_kv_store: the product first
    if (j < half) sh.cs[i] = cosf(theta);
    else sh.sn[i] = sinf(theta);
  }
  // The page that takes the row's own key and value.  first_page_of_block >= 0: wave w of the
  // block has looked up page first_page_of_block + w of the row already and left its number in
  // sh.page_of_wave[w], which saves a trip to memory that could only start once the position was known.
  int page = -1;
  const int lp = pos / SB_PAGE;
  if (ra.store && mine && first_page_of_block < 0) {
    page = lp < max_pages ? page_table[size_t(seq) * max_pages + lp] : -1;
    if (page >= n_pages_total) page = -1;
  }
  if (half > 0 || first_page_of_block >= 0) __syncthreads();
  if (ra.store && mine && first_page_of_block >= 0) {
    const int w = lp - first_page_of_block;
    page = (w >= 0 && w < 4 && lp < max_pages) ? sh.page_of_wave[w] : -1;
    if (page >= n_pages_total) page = -1;
  }
  const int n_q = group * kPerHead;
  const int n_items = n_q + (page >= 0 ? 2 * kPerHead : 0);
  for (int it = threadIdx.x; it < n_items; it += blockDim.x) {
    RopeItem later;
    if (it != int(threadIdx.x)) fetch_item_in_turn(later, ra, seq, it, n_q, kvh, group, heads_q, heads_kv, half);
    float y[8];
    finish_item(y, it == int(threadIdx.x) ? first : later, it, n_q, half, sh.cs, sh.sn);
    if (it < n_q) {
      sh.q[(it / kPerHead) * kQStride + it % kPerHead] = pack8(y);
      continue;
    }
    const size_t base = (size_t(page) * heads_kv + kvh) * SB_PAGE * HD;
    const int d0 = ((it - n_q) % kPerHead) * 8;
    if (it < n_q + kPerHead) {
      const uint4 packed = pack8(y);
      sh.k[d0 / 8] = packed;
      *reinterpret_cast<uint4 *>(k_cache + base + size_t(k_slot(pos % SB_PAGE, d0 / 8)) * 8) = packed;
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const bf16_t b = f32_to_bf16(y[i]);
        sh.v[d0 + i] = b;
        v_cache[base + sb_value_index(d0 + i, pos % SB_PAGE)] = b;
      }
    }
  }
  if (visible) __threadfence_block();
  __syncthreads();
}

// The frequency of the rotation that thread t of a block works out a cosine or sine for
// (threads [0, half) the cosines, [half, 2 half) the sines).
__device__ __forceinline__ float rope_freq(const RopeArgs &ra) {
  const int half = ra.inv_freq ? ra.rot_dims / 2 : 0;
  const int j = threadIdx.x;
  if (j >= 2 * half) return 0.f;
  const int i = j < half ? j : j - half;
  return ra.inv_freq[i];
}

// Half `half` of the page that holds the row's own position, as loaded from the cache before the
// row's key and value were stored: the fragments' elements of slot `slot` (the row's position in
// the page) replaced by the key and value in LDS.  A lane's key fragments are eight d of one key
// each, its value fragments eight consecutive keys of one d.
__device__ __forceinline__ void patch_half(HalfPage &hp, const RopeShared &sh, int half, int slot, int lane) {
  const int r = lane & 15, g = lane >> 4;
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int key = 32 * half + 8 * (r >> 2) + 4 * t + (r & 3);
    if (key == slot) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int d = ks * 32 + g * 8;
        if (d < HD) hp.k[t][ks] = sh.k[d / 8];
      }
    }
  }
  const int e = slot - (32 * half + 8 * g);
  if (e >= 0 && e < 8) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      uint32_t w[4] = {hp.v[dt].x, hp.v[dt].y, hp.v[dt].z, hp.v[dt].w};
      const uint32_t val = sh.v[dt * 16 + r];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (i == (e >> 1)) w[i] = (e & 1) ? ((w[i] & 0xffffu) | (val << 16)) : ((w[i] & 0xffff0000u) | val);
      hp.v[dt] = make_uint4(w[0], w[1], w[2], w[3]);
    }
  }
}

// A wave's query fragments from the staged queries.
__device__ __forceinline__ void staged_q(bf16x8_t (&qf)[KS], const RopeShared &sh, int hq, bool col_ok, int lane) {
  const int g = lane >> 4;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d = ks * 32 + g * 8;
    qf[ks] = as_bf16x8((col_ok && d < HD) ? sh.q[hq * kQStride + d / 8] : make_uint4(0u, 0u, 0u, 0u));
  }
}

template <bool BOTH, bool FUSED>
__global__ void __launch_bounds__(256)
attn_decode_kernel(bf16_t *__restrict__ out, float *__restrict__ part_o, float *__restrict__ part_ml,
                   const bf16_t *__restrict__ q, const RopeArgs ra,
                   const bf16_t *k_cache, const bf16_t *v_cache,
                   const int32_t *__restrict__ page_table, int max_pages, int n_pages_total,
                   const int32_t *__restrict__ row_pos, int heads_q, int heads_kv, int n_chunks,
                   float scale_log2, int window, int n_seqs) {
  __shared__ float lds_o[4][HD * 16];   // [wave][d][col]
  __shared__ float lds_m[4][16], lds_l[4][16];
  __shared__ std::conditional_t<FUSED, RopeShared, int> rope_sh;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int group = heads_q / heads_kv;
  const int head_tiles = (group + 15) / 16;
  const int tiles = heads_kv * head_tiles;
  const DecodeBlock blk = decode_block(tiles, n_seqs);
  const int chunk = blk.chunk, seq = blk.seq;
  const int kvh = blk.tile / head_tiles, ht = blk.tile - kvh * head_tiles;
  // the wave's page number does not depend on the position: both look-ups go out together, and
  // before everything else, since the page's loads wait for them
  const int pg = chunk * kPagesPerChunk + wave;
  const int page_looked_up = page_table[size_t(seq) * max_pages + min(pg, max_pages - 1)];
  const int pos = row_pos[seq];
  // the folded form: this thread's share of the qkv row depends on the block's number only, so
  // its loads go out right behind them
  RopeItem first;
  if constexpr (FUSED) {
    const int n_q = group * kPerHead, n_all = n_q + (ra.store ? 2 * kPerHead : 0);
    if (int(threadIdx.x) < n_all)
      fetch_item(first, ra, seq, threadIdx.x, n_q, kvh, group, heads_q, heads_kv, ra.inv_freq ? ra.rot_dims / 2 : 0);
  }
  const float freq = FUSED ? rope_freq(ra) : 0.f;
  const int key_lo = (window > 0 && pos >= window) ? pos - window + 1 : 0;
  const int first_chunk = key_lo / (SB_PAGE * kPagesPerChunk);
  const int last_chunk = min(pos / (SB_PAGE * kPagesPerChunk), n_chunks - 1);
  if (chunk < first_chunk || chunk > last_chunk) return;   // uniform over the block

  const int r = lane & 15, g = lane >> 4;
  const int hq = ht * 16 + r;                 // query head within the group
  const bool col_ok = hq < group;
  const int head = kvh * group + (col_ok ? hq : 0);
  const bool have_page = pg >= key_lo / SB_PAGE && pg <= pos / SB_PAGE && pg < max_pages && page_looked_up >= 0 &&
                         page_looked_up < n_pages_total;
  const size_t off = (size_t(have_page ? page_looked_up : 0) * heads_kv + kvh) * SB_PAGE * HD;
  const int col_pos = col_ok ? pos : -1;
  bf16x8_t qf[1][KS];
  WaveState<1> st;
  init_state<1>(st);
  if constexpr (!FUSED) {
    load_q(qf[0], q + (size_t(seq) * heads_q + head) * HD, col_ok, lane);
    if (have_page)
      attend_page<1, BOTH>(st, qf, k_cache + off, v_cache + off, pg * SB_PAGE, col_pos, key_lo, key_lo, pos, scale_log2,
                           lane);
  } else {
    // The page's keys and values do not depend on the queries: their loads go out first and are
    // in flight while the block builds its queries.  The page that receives the row's own key
    // and value is read like the others, before they are stored, and its fragments are patched
    // from LDS afterwards.
    const int page_pos = pg * SB_PAGE;
    const bool use0 = have_page && !(page_pos > pos || page_pos + 31 < key_lo);
    const bool use1 = have_page && !(page_pos + 32 > pos || page_pos + 63 < key_lo);
    const bool own_page = ra.store && have_page && pg == pos / SB_PAGE;
    constexpr bool kEarly = BOTH && HD <= 128;
    HalfPage h0, h1;
    if (kEarly) {
      if (use0) load_half(h0, k_cache + off, v_cache + off, 0, lane);
      if (use1) load_half(h1, k_cache + off, v_cache + off, 1, lane);
    }
    if (lane == 0) rope_sh.page_of_wave[wave] = page_looked_up;
    rope_store(rope_sh, first, freq, ra, seq, pos, kvh, group, heads_q, heads_kv, chunk == last_chunk, !kEarly,
               const_cast<bf16_t *>(k_cache), const_cast<bf16_t *>(v_cache), page_table, max_pages, n_pages_total,
               chunk * kPagesPerChunk);
    staged_q(qf[0], rope_sh, hq, col_ok, lane);
    if (kEarly) {
      const int slot = pos % SB_PAGE;
      if (own_page && slot < 32 && use0) patch_half(h0, rope_sh, 0, slot, lane);
      if (own_page && slot >= 32 && use1) patch_half(h1, rope_sh, 1, slot, lane);
      if (use0) attend_half<1>(st, qf, h0, page_pos, col_pos, key_lo, key_lo, pos, scale_log2, lane);
      if (use1) attend_half<1>(st, qf, h1, page_pos + 32, col_pos, key_lo, key_lo, pos, scale_log2, lane);
    } else if (have_page) {
      attend_page<1, BOTH>(st, qf, k_cache + off, v_cache + off, page_pos, col_pos, key_lo, key_lo, pos, scale_log2,
                           lane);
    }
  }
  finish_decode_block(st, lds_o, lds_m, lds_l, out, part_o, part_ml, wave, lane, chunk, first_chunk == last_chunk,
                      seq, kvh, ht, group, heads_q, n_chunks, size_t(seq) * tiles + blk.tile);
}

// Decode with many more blocks than the GPU holds at once (long contexts, large batches): a wave
// takes `ppw` consecutive pages instead of one and keeps the next half page's keys and values in
// flight while it multiplies the current one, so that a block lives long enough to stream and the
// fixed costs of a block (look-ups, queries, the merge through LDS, the partial results) are paid
// once per 4 * ppw pages.  Block (chunk of 4 * ppw pages, kv head x head tile, sequence); wave w
// takes pages chunk * 4 * ppw + w * ppw + 0 .. ppw-1.  Head sizes up to 128.
template <bool FUSED>
__global__ void __launch_bounds__(256, 2)
attn_decode_long_kernel(bf16_t *__restrict__ out, float *__restrict__ part_o, float *__restrict__ part_ml,
                        const bf16_t *__restrict__ q, const RopeArgs ra,
                        const bf16_t *k_cache, const bf16_t *v_cache,
                        const int32_t *__restrict__ page_table, int max_pages, int n_pages_total,
                        const int32_t *__restrict__ row_pos, int heads_q, int heads_kv, int n_chunks,
                        float scale_log2, int window, int ppw, int n_seqs) {
  __shared__ float lds_o[4][HD * 16];   // [wave][d][col]
  __shared__ float lds_m[4][16], lds_l[4][16];
  __shared__ std::conditional_t<FUSED, RopeShared, int> rope_sh;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int group = heads_q / heads_kv;
  const int head_tiles = (group + 15) / 16;
  const int tiles = heads_kv * head_tiles;
  const DecodeBlock blk = decode_block(tiles, n_seqs);
  const int chunk = blk.chunk, seq = blk.seq;
  const int kvh = blk.tile / head_tiles, ht = blk.tile - kvh * head_tiles;
  const int pos = row_pos[seq];
  RopeItem first;       // the folded form: see attn_decode_kernel
  if constexpr (FUSED) {
    const int n_q = group * kPerHead, n_all = n_q + (ra.store ? 2 * kPerHead : 0);
    if (int(threadIdx.x) < n_all)
      fetch_item(first, ra, seq, threadIdx.x, n_q, kvh, group, heads_q, heads_kv, ra.inv_freq ? ra.rot_dims / 2 : 0);
  }
  const float freq = FUSED ? rope_freq(ra) : 0.f;
  const int pages_per_chunk = kPagesPerChunk * ppw;
  const int key_lo = (window > 0 && pos >= window) ? pos - window + 1 : 0;
  const int first_chunk = key_lo / (SB_PAGE * pages_per_chunk);
  const int last_chunk = min(pos / (SB_PAGE * pages_per_chunk), n_chunks - 1);
  if (chunk < first_chunk || chunk > last_chunk) return;   // uniform over the block

  const int r = lane & 15;
  const int hq = ht * 16 + r;                 // query head within the group
  const bool col_ok = hq < group;
  const int head = kvh * group + (col_ok ? hq : 0);
  bf16x8_t qf[1][KS];
  WaveState<1> st;
  init_state<1>(st);

  const int32_t *pt = page_table + size_t(seq) * max_pages;
  const int pg_begin = max(chunk * pages_per_chunk + wave * ppw, key_lo / SB_PAGE);
  const int pg_end = min(min(chunk * pages_per_chunk + (wave + 1) * ppw, pos / SB_PAGE + 1), max_pages);
  const size_t page_elems = size_t(heads_kv) * SB_PAGE * HD;
  const size_t head_off = size_t(kvh) * SB_PAGE * HD;
  // a page number outside the cache: read page 0 and see none of its keys
  auto page_of = [&](int pg, bool &ok) {
    const int page = pt[pg];
    ok = page >= 0 && page < n_pages_total;
    return size_t(ok ? page : 0) * page_elems + head_off;
  };
  HalfPage h0, h1;
  bool ok = false;
  size_t off = 0;
  // The folded form: the first half page's loads go out before the block builds its queries.  The
  // page that receives the row's own key and value is read like the others (before or after they
  // are stored: the stores are not waited for) and its fragments are patched from LDS.
  if (pg_begin < pg_end) {
    off = page_of(pg_begin, ok);
    load_half_straight(h0, k_cache + off, v_cache + off, 0, lane);
  }
  if constexpr (FUSED) {
    rope_store(rope_sh, first, freq, ra, seq, pos, kvh, group, heads_q, heads_kv, chunk == last_chunk, false,
               const_cast<bf16_t *>(k_cache), const_cast<bf16_t *>(v_cache), page_table, max_pages, n_pages_total);
    staged_q(qf[0], rope_sh, hq, col_ok, lane);
  } else {
    load_q(qf[0], q + (size_t(seq) * heads_q + head) * HD, col_ok, lane);
  }
  if (pg_begin < pg_end) {
    // 32 keys from `base` on: all visible and written (the common case), or tested one by one
    const int own_base = (FUSED && ra.store) ? (pos / 32) * 32 : -1;     // the half page of the row's own slot
    auto attend = [&](HalfPage &h, int base, bool ok) {
      if constexpr (FUSED) {
        if (ok && base == own_base) patch_half(h, rope_sh, (base >> 5) & 1, pos % SB_PAGE, lane);
      }
      if (ok && base >= key_lo && base + 31 <= pos) {
        attend_half<1, false>(st, qf, h, base, pos, key_lo, key_lo, pos, scale_log2, lane);
      } else {
        // hi < lo for a page that is not there: every value is cut, no key seen
        attend_half<1, true>(st, qf, h, base, (ok && col_ok) ? pos : -1, key_lo, key_lo, ok ? pos : -1, scale_log2,
                             lane);
      }
    };
    int pg = pg_begin;
    // every page but the last: the loads of the next half page go out before this half's
    // products, with no branch between a load and its use
    for (; pg + 1 < pg_end; ++pg) {
      load_half_straight(h1, k_cache + off, v_cache + off, 1, lane);
      attend(h0, pg * SB_PAGE, ok);
      bool ok_next;
      off = page_of(pg + 1, ok_next);
      load_half_straight(h0, k_cache + off, v_cache + off, 0, lane);
      attend(h1, pg * SB_PAGE + 32, ok);
      ok = ok_next;
    }
    load_half_straight(h1, k_cache + off, v_cache + off, 1, lane);
    attend(h0, pg * SB_PAGE, ok);
    attend(h1, pg * SB_PAGE + 32, ok);
  }
  finish_decode_block(st, lds_o, lds_m, lds_l, out, part_o, part_ml, wave, lane, chunk, first_chunk == last_chunk,
                      seq, kvh, ht, group, heads_q, n_chunks, size_t(seq) * tiles + blk.tile);
}

// Merge the chunks of a (sequence, tile), at most kAtOnce of them, in ascending order: one thread
// per element e = d * 16 + column.  Grid (HD * 16 / 256, tiles, sequences).
__global__ void __launch_bounds__(256)
attn_decode_merge_kernel(bf16_t *__restrict__ out, const float *__restrict__ part_o,
                         const float *__restrict__ part_ml, const int32_t *__restrict__ row_pos,
                         int heads_q, int heads_kv, int n_chunks, int window, int pages_per_chunk) {
  const int seq = blockIdx.z;
  const int group = heads_q / heads_kv;
  const int head_tiles = (group + 15) / 16;
  const int kvh = blockIdx.y / head_tiles, ht = blockIdx.y - kvh * head_tiles;
  const int pos = row_pos[seq];
  const int e = blockIdx.x * 256 + threadIdx.x;
  const size_t tile_index = size_t(seq) * gridDim.y + blockIdx.y;
  const float *po = part_o + (tile_index * n_chunks) * (HD * 16), *pml = part_ml + (tile_index * n_chunks) * 32;
  // Up to kAtOnce chunks: the partial results of all of them are asked for together with the
  // position, which says which of them count (a chunk past the last is the last once more);
  // waiting for the position first costs this short kernel a trip to memory of its two.
  constexpr int kAtOnce = 16;
  float mv[kAtOnce], lv[kAtOnce], ov[kAtOnce];
  {
    const int c = e & 15;
#pragma unroll
    for (int ch = 0; ch < kAtOnce; ++ch) {
      const size_t cc = size_t(min(ch, n_chunks - 1));
      mv[ch] = pml[cc * 32 + c];
      lv[ch] = pml[cc * 32 + 16 + c];
      ov[ch] = po[cc * (HD * 16) + e];
    }
  }
  const int key_lo = (window > 0 && pos >= window) ? pos - window + 1 : 0;
  const int first = key_lo / (SB_PAGE * pages_per_chunk), last = min(pos / (SB_PAGE * pages_per_chunk), n_chunks - 1);
  if (first == last) return;      // the decode kernel has written the result itself
  // rescaled to the common maximum and added in ascending chunk order
  const int c = e & 15, d = e >> 4;
  const int hh = ht * 16 + c;
  if (hh >= group) return;
  float m = -__builtin_inff();
#pragma unroll
  for (int ch = 0; ch < kAtOnce; ++ch) m = (ch >= first && ch <= last) ? fmaxf(m, mv[ch]) : m;
  const float m_use = m == -__builtin_inff() ? 0.f : m;
  float o = 0.f, l = 0.f;
#pragma unroll
  for (int ch = 0; ch < kAtOnce; ++ch) {
    const bool use = ch >= first && ch <= last;
    const float f = __builtin_amdgcn_exp2f(mv[ch] - m_use);
    o = use ? o + ov[ch] * f : o;
    l = use ? l + lv[ch] * f : l;
  }
  out[(size_t(seq) * heads_q + kvh * group + hh) * HD + d] = f32_to_bf16(l > 0.f ? o / l : 0.f);
}

// The same for rows of many chunks: a block takes 64 elements, its four waves every fourth
// chunk each, eight chunks' partial results in flight at a time (one thread walking all chunks
// waits for memory once per few chunks: 128 chunks took it longer than the decode kernel took to
// read the keys).  A wave keeps a running maximum of its own; the four meet in LDS and are folded
// in wave order.  Grid (HD * 16 / 64, tiles, sequences).
__global__ void __launch_bounds__(256)
attn_decode_merge_many_kernel(bf16_t *__restrict__ out, const float *__restrict__ part_o,
                              const float *__restrict__ part_ml, const int32_t *__restrict__ row_pos,
                              int heads_q, int heads_kv, int n_chunks, int window, int pages_per_chunk) {
  __shared__ float lds_m[4][64], lds_l[4][64], lds_o[4][64];
  const int seq = blockIdx.z;
  const int group = heads_q / heads_kv;
  const int head_tiles = (group + 15) / 16;
  const int kvh = blockIdx.y / head_tiles, ht = blockIdx.y - kvh * head_tiles;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int e = blockIdx.x * 64 + lane;                 // < HD * 16: 64 divides it
  const int c = e & 15, d = e >> 4;
  const size_t tile_index = size_t(seq) * gridDim.y + blockIdx.y;
  const float *po = part_o + (tile_index * n_chunks) * (HD * 16), *pml = part_ml + (tile_index * n_chunks) * 32;
  constexpr int kAtOnce = 8;
  float mv[kAtOnce], lv[kAtOnce], ov[kAtOnce];
  auto ask = [&](int base) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < kAtOnce; ++i) {
      const size_t cc = size_t(min(base + 4 * i, n_chunks - 1));   // (past the end: the last once more, not used)
      mv[i] = pml[cc * 32 + c];
      lv[i] = pml[cc * 32 + 16 + c];
      ov[i] = po[cc * (HD * 16) + e];
    }
  };
  // the first round goes out together with the position, which says which chunks count
  ask(wave);
  const int pos = row_pos[seq];
  const int key_lo = (window > 0 && pos >= window) ? pos - window + 1 : 0;
  const int first = key_lo / (SB_PAGE * pages_per_chunk), last = min(pos / (SB_PAGE * pages_per_chunk), n_chunks - 1);
  if (first == last) return;      // the decode kernel has written the result itself
  float m = -__builtin_inff(), o = 0.f, l = 0.f;
  for (int base = wave;; base += 4 * kAtOnce) {
    if (base + 4 * (kAtOnce - 1) >= first) {
#pragma unroll
      for (int i = 0; i < kAtOnce; ++i) {
        const int ch = base + 4 * i;
        const bool use = ch >= first && ch <= last;
        const float m_new = use ? fmaxf(m, mv[i]) : m;
        const float m_use = m_new == -__builtin_inff() ? 0.f : m_new;
        const float keep = __builtin_amdgcn_exp2f(m - m_use), f = use ? __builtin_amdgcn_exp2f(mv[i] - m_use) : 0.f;
        o = o * keep + (use ? ov[i] * f : 0.f);
        l = l * keep + (use ? lv[i] * f : 0.f);
        m = m_new;
      }
    }
    if (base + 4 * kAtOnce > last) break;
    ask(base + 4 * kAtOnce);
  }
  lds_m[wave][lane] = m;
  lds_l[wave][lane] = l;
  lds_o[wave][lane] = o;
  __syncthreads();
  if (wave != 0) return;
  const int hh = ht * 16 + c;
  if (hh >= group) return;
  float m_all = fmaxf(fmaxf(lds_m[0][lane], lds_m[1][lane]), fmaxf(lds_m[2][lane], lds_m[3][lane]));
  if (m_all == -__builtin_inff()) m_all = 0.f;
  float o_all = 0.f, l_all = 0.f;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const float f = __builtin_amdgcn_exp2f(lds_m[w][lane] - m_all);
    o_all += lds_o[w][lane] * f;
    l_all += lds_l[w][lane] * f;
  }
  out[(size_t(seq) * heads_q + kvh * group + hh) * HD + d] = f32_to_bf16(l_all > 0.f ? o_all / l_all : 0.f);
}

int check_common(const void *out, const void *q, const void *k, const void *v, const void *pt,
                 const void *row_pos, int max_pages, int n_pages_total, int heads_q, int heads_kv,
                 int window, const char *who) {
  SB_REQUIRE(out && q && k && v && pt && row_pos, "%s: null pointer", who);
  SB_REQUIRE(max_pages > 0 && n_pages_total > 0 && heads_q > 0 && heads_kv > 0 && window >= 0,
             "%s: bad sizes", who);
  SB_REQUIRE(heads_q % heads_kv == 0, "%s: %d query heads are not a multiple of %d kv heads", who, heads_q,
             heads_kv);
  SB_SUPPORT(heads_q <= 65535, "%s: more than 65535 query heads", who);
  SB_SUPPORT(((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) |
               reinterpret_cast<uintptr_t>(v) | reinterpret_cast<uintptr_t>(out)) % 16) == 0,
             "%s: operands must be 16-byte aligned", who);
  return SB_OK;
}

}  // namespace

// Chunks the decode kernel splits `max_pages` pages into (the third size of its partial buffers).
extern "C" int sb_attn_decode_chunks(int max_pages) {
  return (max_pages + kPagesPerChunk - 1) / kPagesPerChunk;
}

// Floats of part_o and of part_ml that sb_attn_decode_bf16 needs for these sizes.
extern "C" size_t sb_attn_decode_part_o(int n_seqs, int heads_q, int heads_kv, int max_pages) {
  const int tiles = heads_kv * ((heads_q / heads_kv + 15) / 16);
  return size_t(n_seqs) * tiles * sb_attn_decode_chunks(max_pages) * HD * 16;
}
extern "C" size_t sb_attn_decode_part_ml(int n_seqs, int heads_q, int heads_kv, int max_pages) {
  const int tiles = heads_kv * ((heads_q / heads_kv + 15) / 16);
  return size_t(n_seqs) * tiles * sb_attn_decode_chunks(max_pages) * 32;
}

namespace {

// The decode launch, for queries that are given (q) or still to be built (ra.qkv).
int decode_launch(const char *who, void *out, const void *q, const RopeArgs &ra, const void *k_cache,
                  const void *v_cache, const int32_t *page_table, int max_pages, int n_pages_total,
                  const int32_t *row_pos, float *part_o, float *part_ml, int n_seqs, int heads_q, int heads_kv,
                  float scale, int window, int pages_per_wave, void *stream) {
  const bool fused = ra.qkv != nullptr;
  const int chunks_1 = sb_attn_decode_chunks(max_pages);      // what the partial buffers are sized for
  SB_REQUIRE(chunks_1 == 1 || (part_o && part_ml), "%s: no buffers for the partial results", who);
  const int group = heads_q / heads_kv;
  const int head_tiles = (group + 15) / 16;
  hipStream_t s = (hipStream_t)stream;
  SB_SUPPORT(heads_kv * head_tiles <= 65535, "%s: too many heads", who);
  // A wave takes one page and asks for all of it at once (one round trip to memory), or, when
  // two pages per wave still leave a block for every CU, several pages in a row with half a page
  // in flight while the half before it is multiplied.
  const long long per_chunk = (long long)heads_kv * head_tiles * n_seqs;
  int ppw = 1;
  if (HD <= 128 && (long long)((max_pages + 7) / 8) * per_chunk >= 256) {
    // How many pages in a row: the count with the least estimated time, in microseconds, from
    // what was measured (MI355X, cold caches).  A wave gets through a page in about 3.3 us
    // whatever the head size (two round trips to memory); a CU streams about 27 GB/s, all of
    // them together 5.3 TB/s; a block costs about 2 us besides (fitted: with 4 the choices lost 42 us over
    // 29 measured cases of 1 to 128 sequences and 2,000 to 131,000 keys, with 2 they lose 5); more than one chunk costs the
    // partial results and the second kernel, about 8 us.  The table's width is taken for the rows' length less half of the 16
    // pages it is rounded up by.  One chunk (a quarter of the width per wave) is among the
    // candidates: it wins when sequences x kv heads alone fill most of the GPU.
    const double page_bytes = 2.0 * SB_PAGE * HD * 2;
    const int pages = max_pages > 8 ? max_pages - 8 : 1;
    const int whole = (max_pages + kPagesPerChunk - 1) / kPagesPerChunk;
    const int candidates[5] = {2, 4, 8, 16, whole < 2 ? 2 : whole};
    double best = -1.0;
    for (int c : candidates) {
      const int chunks = (max_pages + 4 * c - 1) / (4 * c);
      const int full = pages / (4 * c) > 1 ? pages / (4 * c) : 1;
      const double busy = double(per_chunk) * full < 256.0 ? double(per_chunk) * full : 256.0;
      const double rate = busy * 27e3 < 5.3e6 ? busy * 27e3 : 5.3e6;            // bytes per us
      const int run = c < pages ? c : pages;
      // a block spends about 2 us on what is not streaming (look-ups, queries, the merge)
      // blocks that a CU holds together share its rate, so the CU with the most blocks sets the
      // time: 260 equal blocks take as long as 512 (measured: 65 sequences x 4 kv heads x 2,048
      // keys 77 us in one chunk against 45 for 64 sequences, 63 in chunks of eight pages)
      const long long n_busy = per_chunk * full;
      // (blocks of few pages in a row pay less of it, the CU's second block being short: 260
      // blocks of two pages a wave took 22.7 us where 130 of four took 25.7)
      const double rounds = n_busy > 256 ? double((n_busy + 255) / 256) * 256.0 / double(n_busy) : 1.0;
      const double uneven = 1.0 + (rounds - 1.0) * (run < 8 ? run / 8.0 : 1.0);
      const double stream_us =
          double(per_chunk) * pages * page_bytes / rate * (1.0 + 2.0 / (run * 3.3)) * uneven;
      const double in_a_row = run * 3.3 + 2.0;
      const double t = (stream_us > in_a_row ? stream_us : in_a_row) + (chunks > 1 ? 8.0 : 0.0);
      if (best < 0.0 || t < best) best = t, ppw = c;
    }
  }
  // a test's or a measurement's choice (0: the launcher's own)
  if (pages_per_wave > 0 && (pages_per_wave == 1 || HD <= 128)) ppw = pages_per_wave;
  const int pages_per_chunk = kPagesPerChunk * ppw;
  const int n_chunks = (max_pages + pages_per_chunk - 1) / pages_per_chunk;
  SB_SUPPORT((long long)n_chunks * per_chunk <= 0x7fffffffLL, "%s: too many blocks", who);
  const unsigned grid = unsigned((long long)n_chunks * per_chunk);
#define SB_ARGS                                                                                           \
  (bf16_t *)out, part_o, part_ml, (const bf16_t *)q, ra, (const bf16_t *)k_cache, (const bf16_t *)v_cache, \
      page_table, max_pages, n_pages_total, row_pos, heads_q, heads_kv, n_chunks, scale *kLog2e, window
  if (ppw > 1) {
    // (only head sizes up to 128 get here, and only they hold this kernel)
    if constexpr (HD <= 128) {
      if (fused) attn_decode_long_kernel<true><<<grid, 256, 0, s>>>(SB_ARGS, ppw, n_seqs);
      else attn_decode_long_kernel<false><<<grid, 256, 0, s>>>(SB_ARGS, ppw, n_seqs);
    }
  } else if ((long long)n_chunks * per_chunk <= 1536) {
    if (fused) attn_decode_kernel<true, true><<<grid, 256, 0, s>>>(SB_ARGS, n_seqs);
    else attn_decode_kernel<true, false><<<grid, 256, 0, s>>>(SB_ARGS, n_seqs);
  } else {
    if (fused) attn_decode_kernel<false, true><<<grid, 256, 0, s>>>(SB_ARGS, n_seqs);
    else attn_decode_kernel<false, false><<<grid, 256, 0, s>>>(SB_ARGS, n_seqs);
  }
#undef SB_ARGS
  int rc = sb::check_launch(who);
  if (rc != SB_OK || n_chunks == 1) return rc;
  if (n_chunks <= 16)
    attn_decode_merge_kernel<<<dim3((HD * 16 + 255) / 256, heads_kv * head_tiles, n_seqs), 256, 0, s>>>(
        (bf16_t *)out, part_o, part_ml, row_pos, heads_q, heads_kv, n_chunks, window, pages_per_chunk);
  else
    attn_decode_merge_many_kernel<<<dim3(HD * 16 / 64, heads_kv * head_tiles, n_seqs), 256, 0, s>>>(
        (bf16_t *)out, part_o, part_ml, row_pos, heads_q, heads_kv, n_chunks, window, pages_per_chunk);
  return sb::check_launch(who);
}

}  // namespace

// q, out: bf16 [n_seqs, heads_q * HD], one row per sequence; k_cache bf16 [pages][heads_kv][64][HD],
// v_cache bf16 [pages][heads_kv][HD][64].  part_o / part_ml: float buffers of the sizes the two
// functions above give (may be NULL when max_pages fits one chunk).  pages_per_wave: 0, or a
// test's or a measurement's choice of how many pages in a row a wave takes.
extern "C" int sb_attn_decode_bf16(void *out, const void *q, const void *k_cache, const void *v_cache,
                                   const int32_t *page_table, int max_pages, int n_pages_total,
                                   const int32_t *row_pos, float *part_o, float *part_ml, int n_seqs,
                                   int heads_q, int heads_kv, float scale, int window, int pages_per_wave,
                                   void *stream) {
  int rc = check_common(out, q, k_cache, v_cache, page_table, row_pos, max_pages, n_pages_total, heads_q,
                        heads_kv, window, "sb_attn_decode_bf16");
  if (rc != SB_OK) return rc;
  SB_REQUIRE(n_seqs >= 0, "sb_attn_decode_bf16: bad batch");
  SB_SUPPORT(n_seqs <= 65535, "sb_attn_decode_bf16: more than 65535 sequences in a step");
  if (n_seqs == 0) return SB_OK;
  const RopeArgs none{nullptr, 0, 0, 0, nullptr, nullptr, nullptr, 0, 0};
  return decode_launch("sb_attn_decode_bf16", out, q, none, k_cache, v_cache, page_table, max_pages, n_pages_total,
                       row_pos, part_o, part_ml, n_seqs, heads_q, heads_kv, scale, window, pages_per_wave, stream);
}

// 1 when sb_attn_decode_rope_bf16 takes these sizes (else: sb_rope_kv_store, then sb_attn_decode_bf16).
extern "C" int sb_attn_decode_rope_ok(int heads_q, int heads_kv, int rot_dims, int row_stride) {
  return heads_kv > 0 && heads_q % heads_kv == 0 && heads_q / heads_kv <= 16 && rot_dims >= 0 && rot_dims % 16 == 0 &&
         rot_dims <= HD && row_stride % 4 == 0;
}

// The same attention for a step whose queries, keys and values are still the float32 rows of the
// qkv product: qkv [n_slices][n_seqs][row_stride], a row [heads_q*HD queries | heads_kv*HD keys |
// heads_kv*HD values], the slices added in ascending order, then `bias` (float [row] or NULL).
// Queries and keys are rotated as sb_rope_kv_store rotates them (inv_freq NULL: not at all), the
// row's key and value are stored at its position (store_kv = 0: nothing is stored, for a layer
// that reads another layer's cache), and the row attends over the cache including itself: the
// results and the cache contents are those of sb_rope_kv_store followed by sb_attn_decode_bf16,
// bit for bit, in one launch less.  Sizes: sb_attn_decode_rope_ok.
extern "C" int sb_attn_decode_rope_bf16(void *out, const float *qkv, int row_stride, int n_slices, const float *bias,
                                        const float *inv_freq, const float *freq_factors, int rot_dims,
                                        int store_kv, void *k_cache, void *v_cache, const int32_t *page_table,
                                        int max_pages, int n_pages_total, const int32_t *row_pos, float *part_o,
                                        float *part_ml, int n_seqs, int heads_q, int heads_kv, float scale,
                                        int window, int pages_per_wave, void *stream) {
  int rc = check_common(out, qkv, k_cache, v_cache, page_table, row_pos, max_pages, n_pages_total, heads_q,
                        heads_kv, window, "sb_attn_decode_rope_bf16");
  if (rc != SB_OK) return rc;
  SB_REQUIRE(n_seqs >= 0 && n_slices >= 1 && n_slices <= 8, "sb_attn_decode_rope_bf16: bad batch or slice count");
  SB_SUPPORT(n_seqs <= 65535, "sb_attn_decode_rope_bf16: more than 65535 sequences in a step");
  SB_REQUIRE(row_stride >= (heads_q + (store_kv ? 2 * heads_kv : 0)) * HD,
             "sb_attn_decode_rope_bf16: row stride %d is shorter than a row of queries%s", row_stride,
             store_kv ? ", keys and values" : "");
  if (!inv_freq) rot_dims = 0;
  SB_SUPPORT(sb_attn_decode_rope_ok(heads_q, heads_kv, rot_dims, row_stride),
             "sb_attn_decode_rope_bf16: takes up to 16 query heads per kv head, a rotary width in steps of 16 and a "
             "row stride in steps of 4 (heads %d / %d, rotary width %d, stride %d)", heads_q, heads_kv, rot_dims,
             row_stride);
  SB_SUPPORT(!bias || reinterpret_cast<uintptr_t>(bias) % 4 == 0, "sb_attn_decode_rope_bf16: unaligned bias");
  if (n_seqs == 0) return SB_OK;
  const RopeArgs ra{qkv, row_stride, n_slices, size_t(n_seqs) * row_stride, bias, inv_freq, freq_factors, rot_dims,
                    store_kv ? 1 : 0};
  return decode_launch("sb_attn_decode_rope_bf16", out, nullptr, ra, k_cache, v_cache, page_table, max_pages,
                       n_pages_total, row_pos, part_o, part_ml, n_seqs, heads_q, heads_kv, scale, window,
                       pages_per_wave, stream);
}

// 1 when the prefill kernel also takes tiles of 32 rows for these heads (head sizes that 32 divides,
// up to 128; groups of three and more query heads per kv head): the form for long prompts.
extern "C" int sb_attn_prefill_tall_ok(int heads_q, int heads_kv) {
  return kTallOk && heads_kv > 0 && heads_q % heads_kv == 0 && heads_q / heads_kv >= 3;
}

// The tile height that suits these heads: 16 rows, or 64 and 32 for groups of one and two query
// heads per kv head, whose blocks would otherwise have waves without a head.
extern "C" int sb_attn_prefill_tile_rows(int heads_q, int heads_kv) {
  if (heads_kv <= 0 || heads_q % heads_kv) return 16;
  const int group = heads_q / heads_kv;
  return group == 1 ? 64 : (group == 2 ? 32 : 16);
}

// q, out: bf16 [n_rows, heads_q * HD]; tiles int32 [n_tiles][4] = (first row, rows <= tile_rows,
// sequence, 0), every tile inside one sequence and its rows at consecutive positions.  tile_rows:
// 16, or what sb_attn_prefill_tile_rows gives for these heads.
extern "C" int sb_attn_prefill_bf16(void *out, const void *q, const void *k_cache, const void *v_cache,
                                    const int32_t *page_table, int max_pages, int n_pages_total,
                                    const int32_t *row_pos, const int32_t *tiles, int n_tiles, int heads_q,
                                    int heads_kv, float scale, int window, int tile_rows, void *stream) {
  int rc = check_common(out, q, k_cache, v_cache, page_table, row_pos, max_pages, n_pages_total, heads_q,
                        heads_kv, window, "sb_attn_prefill_bf16");
  if (rc != SB_OK) return rc;
  SB_REQUIRE(tiles && n_tiles >= 0, "sb_attn_prefill_bf16: no tiles");
  if (n_tiles == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  const int group = heads_q / heads_kv;
  // Waves of a block and query heads of a kv head that one wave takes together: the block's
  // waves cover the group, eight of them (two per SIMD) when the group is big enough to use them,
  // as far as the accumulators fit the registers.  Heads of more than 128 take eight waves with
  // one head each for every group from 5 on (a page of theirs fills so much of LDS that a CU holds
  // one block, and four waves would leave it half empty: measured 1.3 to 2.2 times slower).
  int waves = (group >= 5 && (group <= 8 || HD > 128)) ? 8 : 4;
  int nc = (group + waves - 1) / waves;
  const int nc_max = waves == 8 ? 1 : (DT <= 4 ? 4 : (DT <= 12 ? 2 : 1));
  if (nc > nc_max) nc = nc_max;
  const int head_tiles = (group + nc - 1) / nc;
  const int y_per_kv = (head_tiles + waves - 1) / waves;
  if (tile_rows == 32 && sb_attn_prefill_tall_ok(heads_q, heads_kv)) {
    const int y_tall = (group + 7) / 8;
    SB_SUPPORT((long long)n_tiles * heads_kv * y_tall <= 0x7fffffffLL, "sb_attn_prefill_bf16: too many blocks");
    constexpr int lds_tall = 2 * 2 * kPageChunks * 16;
    static bool raised_tall = false;
    if (lds_tall > 48 * 1024 && !raised_tall) {
      const hipError_t e = hipFuncSetAttribute((const void *)attn_prefill_tall_kernel<kTallOk>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, lds_tall);
      SB_REQUIRE(e == hipSuccess, "sb_attn_prefill_bf16: cannot reserve %d bytes of LDS: %s", lds_tall,
                 hipGetErrorString(e));
      raised_tall = true;
    }
    attn_prefill_tall_kernel<kTallOk><<<dim3(unsigned(n_tiles) * unsigned(heads_kv * y_tall)), 512, lds_tall, s>>>(
        (bf16_t *)out, (const bf16_t *)q, (const bf16_t *)k_cache, (const bf16_t *)v_cache, page_table, max_pages,
        n_pages_total, row_pos, tiles, n_tiles, heads_q, heads_kv, y_tall, scale * kLog2e, window);
    return sb::check_launch("sb_attn_prefill_bf16");
  }
  SB_REQUIRE(tile_rows == 16 || tile_rows == sb_attn_prefill_tile_rows(heads_q, heads_kv),
             "sb_attn_prefill_bf16: tiles of %d rows do not suit %d heads on %d kv heads", tile_rows, heads_q, heads_kv);
  const int row_groups = tile_rows / 16;       // more than one: waves == 4, nc == 1, head_tiles * row_groups == 4
  SB_SUPPORT((long long)n_tiles * heads_kv * y_per_kv <= 0x7fffffffLL, "sb_attn_prefill_bf16: too many blocks");
  dim3 grid(unsigned(n_tiles) * unsigned(heads_kv * y_per_kv));
  constexpr int lds_bytes = 2 * 2 * kPageChunks * 16;
#define SB_GO(NC, WAVES)                                                                                 \
  do {                                                                                                   \
    static bool raised = false;                                                                          \
    if (lds_bytes > 48 * 1024 && !raised) {                                                              \
      const hipError_t e = hipFuncSetAttribute((const void *)attn_prefill_kernel<NC, WAVES>,             \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);   \
      SB_REQUIRE(e == hipSuccess, "sb_attn_prefill_bf16: cannot reserve %d bytes of LDS: %s", lds_bytes, \
                 hipGetErrorString(e));                                                                  \
      raised = true;                                                                                     \
    }                                                                                                    \
    attn_prefill_kernel<NC, WAVES><<<grid, 64 * WAVES, lds_bytes, s>>>(                                  \
        (bf16_t *)out, (const bf16_t *)q, (const bf16_t *)k_cache, (const bf16_t *)v_cache, page_table,  \
        max_pages, n_pages_total, row_pos, tiles, n_tiles, heads_q, heads_kv, head_tiles, y_per_kv,      \
        scale * kLog2e, window, row_groups);                                                             \
  } while (0)
  // (forms that nc_max rules out for this head size are not compiled)
  if (waves == 8) {
    SB_GO(1, 8);
  } else if (nc == 4) {
    if constexpr (DT <= 4) SB_GO(4, 4);
  } else if (nc == 3) {
    if constexpr (DT <= 4) SB_GO(3, 4);
  } else if (nc == 2) {
    if constexpr (DT <= 12) SB_GO(2, 4);
  } else {
    SB_GO(1, 4);
  }
#undef SB_GO
  return sb::check_launch("sb_attn_prefill_bf16");
}
