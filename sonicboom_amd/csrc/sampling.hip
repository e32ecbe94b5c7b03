// Token selection on the device: greedy argmax, sampling penalties, and the
// candidate stage of seeded sampling.
//
// Behaviour follows /root/reference/core/src/nn/sampling.cpp: argmax takes the
// first maximum (:238-244); penalties are v>0 ? v/rp : v*rp, then
// v -= freq*count + presence, in the float form for the greedy path (:43-70)
// and the single-rounding fma form for the sampled path (:77-104); candidates
// are z = l/T as one float division, the 256 largest by (z descending, id
// ascending) (:257-285).  The filters and the Gumbel draw run on the host.
#include "common.h"

#include <mutex>

namespace {

constexpr int kSelThreads = 1024;
constexpr int kSelWaves = kSelThreads / 64;
constexpr int kMaxCand = 256;

// Larger value wins; equal values go to the lower index; an index of INT_MAX marks "nothing".
__device__ __forceinline__ void take_better(float &bv, int &bi, float ov, int oi) {
  if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi))) {
    bv = ov;
    bi = oi;
  }
}

constexpr int kArgThreads = 256;

// Stage 1: block (part, row) scans elements [part * span, (part + 1) * span) of its row, four per
// thread and round, all four loads in flight together.  Stage 2 (n_parts partials per row) runs
// with span covering the partial arrays.  Within a thread indices ascend, so "first maximum"
// needs only strict comparison there; across threads take_better breaks ties.
__global__ void __launch_bounds__(kArgThreads)
argmax_kernel(int32_t *__restrict__ ids, float *__restrict__ part_val, int32_t *__restrict__ part_idx,
              const float *__restrict__ vals, const int32_t *__restrict__ idxs, int row_len, int span) {
  const int row = blockIdx.y, part = blockIdx.x;
  const float *x = vals + size_t(row) * row_len;
  const int32_t *xi = idxs ? idxs + size_t(row) * row_len : nullptr;
  const int begin = part * span, end = min(begin + span, row_len);
  float best_v = -__builtin_inff();
  int best_i = 0x7fffffff;
  for (int i0 = begin + threadIdx.x; i0 < end; i0 += 4 * kArgThreads) {
    float v[4];
    int id[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = i0 + u * kArgThreads;
      const bool ok = i < end;
      v[u] = ok ? x[i] : -__builtin_inff();
      id[u] = ok ? (xi ? xi[i] : i) : 0x7fffffff;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) take_better(best_v, best_i, v[u], id[u]);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(best_v, off, 64);
    const int oi = __shfl_xor(best_i, off, 64);
    take_better(best_v, best_i, ov, oi);
  }
  __shared__ float wv[kArgThreads / 64];
  __shared__ int wi[kArgThreads / 64];
  if ((threadIdx.x & 63) == 0) {
    wv[threadIdx.x >> 6] = best_v;
    wi[threadIdx.x >> 6] = best_i;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    float bv = wv[0];
    int bi = wi[0];
    for (int k = 1; k < kArgThreads / 64; ++k) take_better(bv, bi, wv[k], wi[k]);
    if (ids) {
      ids[row] = bi == 0x7fffffff ? 0 : bi;
    } else {
      part_val[size_t(row) * gridDim.x + part] = bv;
      part_idx[size_t(row) * gridDim.x + part] = bi;
    }
  }
}

__global__ void penalize_kernel(float *__restrict__ logits, int vocab,
                                const int32_t *__restrict__ item_row,
                                const int32_t *__restrict__ item_token,
                                const int32_t *__restrict__ item_count, int n_items, float rp,
                                float presence, float freq, int exact) {
  const int it = blockIdx.x * blockDim.x + threadIdx.x;
  if (it >= n_items) return;
  const int tok = item_token[it];
  if (tok < 0 || tok >= vocab) return;
  float *p = logits + size_t(item_row[it]) * vocab + tok;
  const float c = float(item_count[it]);
  float v = *p;
  if (exact) {
    if (rp != 1.0f) v = v > 0.0f ? __fdiv_rn(v, rp) : __fmul_rn(v, rp);
    const float adjust = __fmaf_rn(freq, c, presence);
    v = __fmaf_rn(-1.0f, adjust, v);
  } else {
    if (rp != 1.0f) v = v > 0.0f ? __fdiv_rn(v, rp) : __fmul_rn(v, rp);
    v = __fsub_rn(v, __fadd_rn(__fmul_rn(freq, c), presence));
  }
  *p = v;
}

// The mask of constrained decoding (/root/reference/core/src/nn/sampling.cpp:266-274, :334-339): bit
// i & 7 of byte i >> 3 of a row's bitmap says whether id i may be chosen; an id past the bitmap
// may not.  What may not be chosen gets -inf, which neither the argmax nor the candidates' window
// ever takes while one id is allowed.
__global__ void mask_logits_kernel(float *__restrict__ logits, int vocab, const uint8_t *__restrict__ bitmaps,
                                   int n_bytes) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x, row = blockIdx.y;
  if (i >= vocab) return;
  const int byte = i >> 3;
  const bool allowed = byte < n_bytes && ((bitmaps[size_t(row) * n_bytes + byte] >> (i & 7)) & 1u);
  if (!allowed) logits[size_t(row) * vocab + i] = -__builtin_inff();
}

// Order-preserving map of a float to an unsigned key (larger float, larger key).
__device__ __forceinline__ uint32_t float_key(float z) {
  z = z + 0.0f;  // -0 and +0 are one value
  const uint32_t u = __float_as_uint(z);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_float(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}
// (z descending, id ascending) as one descending 64-bit order; all keys differ.
__device__ __forceinline__ uint64_t cand_key(float logit, float temperature, int id) {
  return (uint64_t(float_key(__fdiv_rn(logit, temperature))) << 32) | uint64_t(0xffffffffu - uint32_t(id));
}

// The key of rank `want` (1 = largest) among the keys a block's threads hold in registers, PER per
// thread: up to eight radix passes from the top byte down, each a histogram of the keys that share
// the bytes found so far (one histogram per wave, then added up), and a look for the bucket that
// holds the rank.  When that bucket holds exactly the keys still wanted, its lowest possible key
// cuts as the key of the rank would, and the passes end there: with keys that differ in their
// upper half (z) this is after four passes or fewer; the lower half (the id) only matters among
// equal z at the cut.  A key of 0 stands for "nothing" and lies below every real key; `want` must
// not exceed the number of real keys.  Every thread of the block calls it and gets the same key:
// exactly `want` of the real keys are greater or equal.
struct SelectShared {
  uint32_t hist[kSelWaves][256];
  uint32_t wave_total[4];
  uint64_t prefix;
  int remaining;
};

template <int PER>
__device__ __forceinline__ uint64_t select_kth(const uint64_t (&mine)[PER], int want, SelectShared &sh) {
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  if (tid == 0) {
    sh.prefix = 0;
    sh.remaining = want;
  }
  for (int pass = 7; pass >= 0; --pass) {
    const int shift = pass * 8;
    for (int i = tid; i < kSelWaves * 256; i += kSelThreads) (&sh.hist[0][0])[i] = 0;
    __syncthreads();
    const uint64_t prefix = sh.prefix;
    const uint32_t remaining = uint32_t(sh.remaining);
    if (remaining == 0) break;          // (uniform) the cut is found
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const uint64_t key = mine[j];
      if (pass == 7 || (key >> (shift + 8)) == (prefix >> (shift + 8)))
        atomicAdd(&sh.hist[wave][(key >> shift) & 0xffu], 1u);
    }
    __syncthreads();
    // thread b < 256 owns bucket b: its count, and by a suffix sum over the wave and the waves
    // above the count of all higher buckets; the bucket that holds the rank is the one with
    // fewer than `remaining` keys above it and at least that many with its own
    uint32_t mine_n = 0;
    if (tid < 256)
      for (int wv = 0; wv < kSelWaves; ++wv) mine_n += sh.hist[wv][tid];
    uint32_t suffix = mine_n;           // buckets tid .. end of the wave
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const uint32_t other = __shfl_down(suffix, off, 64);
      if (lane + off < 64) suffix += other;
    }
    if (tid < 256 && lane == 0) sh.wave_total[wave] = suffix;
    __syncthreads();
    if (tid < 256) {
      uint32_t above = suffix - mine_n;
      for (int wv = wave + 1; wv < 4; ++wv) above += sh.wave_total[wv];
      if (above < remaining && above + mine_n >= remaining) {
        // the whole bucket is wanted: its lowest key cuts where the key of the rank would
        sh.remaining = above + mine_n == remaining ? 0 : int(remaining - above);
        sh.prefix = prefix | (uint64_t(tid) << shift);
      }
    }
    __syncthreads();
  }
  return sh.prefix;
}

// Stage 1 for long rows: block (part, row) finds the kMaxCand largest keys among kPartElems
// elements of its row and writes them, in no order, to part_keys [row][part][kMaxCand] (zeros fill
// what a short part leaves); the row's kMaxCand largest are among them.
constexpr int kPartElems = 4096;
__global__ void __launch_bounds__(kSelThreads)
top_part_kernel(uint64_t *__restrict__ part_keys, const float *__restrict__ logits, int vocab, float temperature) {
  __shared__ SelectShared sh;
  __shared__ int count_s;
  constexpr int PER = kPartElems / kSelThreads;
  const int tid = threadIdx.x;
  const float *x = logits + size_t(blockIdx.y) * vocab;
  const int first = blockIdx.x * kPartElems;
  uint64_t mine[PER];
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int i = first + j * kSelThreads + tid;
    mine[j] = i < vocab ? cand_key(x[i], temperature, i) : 0ull;
  }
  uint64_t *out = part_keys + (size_t(blockIdx.y) * gridDim.x + blockIdx.x) * kMaxCand;
  if (tid < kMaxCand) out[tid] = 0;
  if (tid == 0) count_s = 0;
  const int real = min(kPartElems, vocab - first);
  const uint64_t kth = select_kth<PER>(mine, min(kMaxCand, real), sh);   // syncs inside
#pragma unroll
  for (int j = 0; j < PER; ++j)
    if (mine[j] >= kth && mine[j] != 0) {
      const int slot = atomicAdd(&count_s, 1);
      if (slot < kMaxCand) out[slot] = mine[j];
    }
}

// Stage 2, or the only stage of a short row: one block per row finds the k largest keys among the
// row's (FROM_KEYS: among the n_keys that stage 1 left in part_keys, at most kRowKeys * 1024; else
// among the keys of its vocab <= kRowKeys * 1024 logits), sorts them (bitonic, in shared memory)
// and writes ids and z.
constexpr int kRowKeys = 16;
template <bool FROM_KEYS>
__global__ void __launch_bounds__(kSelThreads)
top_candidates_kernel(int32_t *__restrict__ cand_id, float *__restrict__ cand_z,
                      const float *__restrict__ logits, const uint64_t *__restrict__ part_keys, int n_keys,
                      int vocab, int k, float temperature) {
  __shared__ SelectShared sh;
  __shared__ uint64_t sel[kMaxCand];
  __shared__ int count_s;
  const float *x = logits + size_t(blockIdx.x) * vocab;
  const uint64_t *pk = part_keys + size_t(blockIdx.x) * n_keys;
  const int n_scan = FROM_KEYS ? n_keys : vocab;
  const int tid = threadIdx.x;
  const int want = min(k, vocab);
  uint64_t mine[kRowKeys];
#pragma unroll
  for (int j = 0; j < kRowKeys; ++j) {
    const int i = j * kSelThreads + tid;
    mine[j] = i < n_scan ? (FROM_KEYS ? pk[i] : cand_key(x[i], temperature, i)) : 0ull;
  }
  if (tid == 0) count_s = 0;
  for (int i = tid; i < kMaxCand; i += kSelThreads) sel[i] = 0;
  const uint64_t kth = select_kth<kRowKeys>(mine, want, sh);              // syncs inside
#pragma unroll
  for (int j = 0; j < kRowKeys; ++j)
    if (mine[j] >= kth && mine[j] != 0) {
      const int slot = atomicAdd(&count_s, 1);
      if (slot < kMaxCand) sel[slot] = mine[j];
    }
  __syncthreads();

  // Bitonic sort of 256 keys, descending; empty slots (0) sink to the end.
  for (int size = 2; size <= kMaxCand; size <<= 1) {
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      if (tid < kMaxCand / 2) {
        const int lo = ((tid / stride) * stride * 2) + (tid % stride);
        const int hi = lo + stride;
        const bool descending = ((lo & size) == 0);
        const uint64_t a = sel[lo], b = sel[hi];
        if (descending ? (a < b) : (a > b)) {
          sel[lo] = b;
          sel[hi] = a;
        }
      }
      __syncthreads();
    }
  }
  for (int i = tid; i < k; i += kSelThreads) {
    const uint64_t key = sel[i];
    const bool real = i < want;
    cand_id[size_t(blockIdx.x) * k + i] = real ? int32_t(0xffffffffu - uint32_t(key)) : -1;
    cand_z[size_t(blockIdx.x) * k + i] = real ? key_float(uint32_t(key >> 32)) : 0.0f;
  }
}


// ---------------------------------------------------------------------------------------------
// The filters and the draw over a row's candidates (/root/reference/core/src/nn/sampling.cpp:157-203,
// :287-312): window of 30 below the best z, top-k, min-p, the shortest prefix whose probability
// reaches top_p (running sums in float64, in order), then Gumbel-max: the candidate with the
// largest z + g, g = -ln(-ln u), u = (w + 0.5) / 2^32 for word 0 of Philox4x32-10 of counter
// (position low, position high, id, 0) under the 64-bit seed; ties to the lower id.  One wave
// per row; the candidates are ordered (z descending, id ascending), so what every filter keeps
// is a prefix and a count stands for it.
__device__ __forceinline__ uint32_t philox_word0(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint64_t key) {
  uint32_t k0 = uint32_t(key), k1 = uint32_t(key >> 32);
#pragma unroll
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

constexpr int kDrawPerLane = kMaxCand / 64;

template <typename POS>    // int64 positions, or int32 lengths to which position_offset is added
__global__ void __launch_bounds__(64)
draw_kernel(int32_t *__restrict__ token, const int32_t *__restrict__ cand_id, const float *__restrict__ cand_z,
            const POS *__restrict__ position, int64_t position_offset, int k, int top_k, int use_min_p,
            float log_min_p, int use_top_p, double top_p, uint64_t seed) {
  __shared__ double e_of[kMaxCand];
  __shared__ int n_keep_sh;
  const int row = blockIdx.x, lane = threadIdx.x;
  const int32_t *ids = cand_id + size_t(row) * k;
  const float *zs = cand_z + size_t(row) * k;
  const float m = zs[0];
  const float floor_z = m - 30.0f;
  const float cutoff = m + log_min_p;
  float z[kDrawPerLane];
  int id[kDrawPerLane];
  int keep = 0;            // candidates inside the window, then after top-k and min-p: a prefix
#pragma unroll
  for (int j = 0; j < kDrawPerLane; ++j) {
    const int c = lane + 64 * j;
    z[j] = c < k ? zs[c] : -__builtin_inff();
    id[j] = c < k ? ids[c] : -1;
    keep += int(__popcll(__ballot(c < k && id[j] >= 0 && z[j] >= floor_z)));
  }
  if (top_k > 0) keep = min(keep, top_k);
  if (use_min_p) {
    int kept = 0;
#pragma unroll
    for (int j = 0; j < kDrawPerLane; ++j) kept += int(__popcll(__ballot(lane + 64 * j < keep && !(z[j] < cutoff))));
    keep = kept;
  }
  if (use_top_p && keep > 0) {
#pragma unroll
    for (int j = 0; j < kDrawPerLane; ++j) {
      const int c = lane + 64 * j;
      if (c < keep) e_of[c] = exp(double(z[j]) - double(m));
    }
    __syncthreads();
    if (lane == 0) {
      double total = 0.0;
      for (int c = 0; c < keep; ++c) total += e_of[c];
      int n = keep;
      if (total > 0.0) {
        double acc = 0.0;
        for (int c = 0; c < keep; ++c) {
          acc += e_of[c];
          if (acc / total >= top_p) {
            n = c + 1;
            break;
          }
        }
      }
      n_keep_sh = n;
    }
    __syncthreads();
    keep = n_keep_sh;
  }
  double best = -__builtin_inf();
  int best_id = 0x7fffffff;
  const uint64_t pos = uint64_t(int64_t(position[row]) + position_offset);
#pragma unroll
  for (int j = 0; j < kDrawPerLane; ++j) {
    const int c = lane + 64 * j;
    if (c >= keep) continue;
    const uint32_t w = philox_word0(uint32_t(pos), uint32_t(pos >> 32), uint32_t(id[j]), 0u, seed);
    const double u = (double(w) + 0.5) / 4294967296.0;
    const double score = double(z[j]) - log(-log(u));
    if (score > best || (score == best && id[j] < best_id)) best = score, best_id = id[j];
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const double other = __shfl_xor(best, off, 64);
    const int other_id = __shfl_xor(best_id, off, 64);
    if (other > best || (other == best && other_id < best_id)) best = other, best_id = other_id;
  }
  if (lane == 0) token[row] = keep > 0 ? best_id : -1;
}

}  // namespace

// Parts a row is cut into for the first stage (the second size of the partial buffers).
extern "C" int sb_argmax_parts(int vocab) {
  const int parts = (vocab + 4095) / 4096;
  return parts < 1 ? 1 : (parts > 256 ? 256 : parts);
}

// part_val float [n_rows * parts], part_idx int32 [n_rows * parts] with parts = sb_argmax_parts(vocab);
// unused (may be NULL) when parts == 1.
extern "C" int sb_argmax(int32_t *ids, const float *logits, int n_rows, int vocab, float *part_val,
                         int32_t *part_idx, void *stream) {
  SB_REQUIRE(ids && logits, "sb_argmax: null pointer");
  SB_REQUIRE(n_rows >= 0 && vocab > 0, "sb_argmax: bad sizes rows=%d vocab=%d", n_rows, vocab);
  SB_SUPPORT(n_rows <= 65535, "sb_argmax: more than 65535 rows");
  if (n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  const int parts = sb_argmax_parts(vocab);
  if (parts == 1) {
    argmax_kernel<<<dim3(1, n_rows), kArgThreads, 0, s>>>(ids, nullptr, nullptr, logits, nullptr, vocab, vocab);
    return sb::check_launch("sb_argmax");
  }
  SB_REQUIRE(part_val && part_idx, "sb_argmax: no buffers for the partial results");
  const int span = (vocab + parts - 1) / parts;
  argmax_kernel<<<dim3(parts, n_rows), kArgThreads, 0, s>>>(nullptr, part_val, part_idx, logits, nullptr, vocab,
                                                            span);
  int rc = sb::check_launch("sb_argmax");
  if (rc != SB_OK) return rc;
  argmax_kernel<<<dim3(1, n_rows), kArgThreads, 0, s>>>(ids, nullptr, nullptr, part_val, part_idx, parts, parts);
  return sb::check_launch("sb_argmax (second stage)");
}

// ---- the greedy choice for callers that cannot allocate ------------------------
// The first stage's partial results go to a file-scope device array instead of
// buffers the caller brings.  In host code the array's name is only a stand-in
// for the symbol: its device address is asked for once per device and kept.
namespace {

constexpr int kNoAllocEntries = 64 * 1024;     // rows * parts of one call, at most
constexpr int kNoAllocDevices = 64;

// [0, 4 * kNoAllocEntries): float values; [4 * kNoAllocEntries, 8 * kNoAllocEntries): int32 indices
static __device__ __align__(256) unsigned char scratch[size_t(kNoAllocEntries) * 8];

std::mutex g_scratch_lock;
void *g_scratch_ptr[kNoAllocDevices] = {nullptr};

// Device address of this device's copy of the array (every GPU holds its own).
int scratch_of_current_device(void **out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return sb::fail(SB_ERR_LAUNCH, "sb_argmax_noalloc: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kNoAllocDevices)
    return sb::fail(SB_ERR_UNSUPPORTED, "sb_argmax_noalloc: device %d, at most %d devices", dev, kNoAllocDevices);
  std::lock_guard<std::mutex> hold(g_scratch_lock);
  if (!g_scratch_ptr[dev]) {
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return sb::fail(SB_ERR_LAUNCH, "sb_argmax_noalloc: hipGetSymbolAddress: %s", hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return SB_OK;
}

}  // namespace

extern "C" int sb_argmax_noalloc_max_entries(void) { return kNoAllocEntries; }

extern "C" int sb_argmax_noalloc(int32_t *ids, const float *logits, int n_rows, int vocab, void *stream) {
  SB_REQUIRE(ids && logits, "sb_argmax_noalloc: null pointer");
  SB_REQUIRE(n_rows >= 0 && vocab > 0, "sb_argmax_noalloc: bad sizes rows=%d vocab=%d", n_rows, vocab);
  SB_SUPPORT(n_rows <= 65535, "sb_argmax_noalloc: more than 65535 rows");
  const int parts = sb_argmax_parts(vocab);
  SB_SUPPORT(parts == 1 || size_t(n_rows) * parts <= size_t(kNoAllocEntries),
             "sb_argmax_noalloc: %d rows of %d parts need %zu partial results, the fixed buffer holds %d", n_rows,
             parts, size_t(n_rows) * parts, kNoAllocEntries);
  if (n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  if (parts == 1) {
    argmax_kernel<<<dim3(1, n_rows), kArgThreads, 0, s>>>(ids, nullptr, nullptr, logits, nullptr, vocab, vocab);
    return sb::check_launch("sb_argmax_noalloc");
  }
  void *base = nullptr;
  int rc = scratch_of_current_device(&base);
  if (rc != SB_OK) return rc;
  // Stage 1 writes every partial result that stage 2 reads, so nothing has to be cleared.
  float *part_val = (float *)base;
  int32_t *part_idx = (int32_t *)((unsigned char *)base + size_t(kNoAllocEntries) * 4);
  const int span = (vocab + parts - 1) / parts;
  argmax_kernel<<<dim3(parts, n_rows), kArgThreads, 0, s>>>(nullptr, part_val, part_idx, logits, nullptr, vocab,
                                                            span);
  rc = sb::check_launch("sb_argmax_noalloc");
  if (rc != SB_OK) return rc;
  argmax_kernel<<<dim3(1, n_rows), kArgThreads, 0, s>>>(ids, nullptr, nullptr, part_val, part_idx, parts, parts);
  return sb::check_launch("sb_argmax_noalloc (second stage)");
}

extern "C" int sb_penalize(float *logits, int vocab, const int32_t *item_row, const int32_t *item_token,
                           const int32_t *item_count, int n_items, float repeat_penalty,
                           float presence_penalty, float frequency_penalty, int exact, void *stream) {
  SB_REQUIRE(logits && (n_items == 0 || (item_row && item_token && item_count)), "sb_penalize: null pointer");
  SB_REQUIRE(n_items >= 0 && vocab > 0, "sb_penalize: bad sizes");
  if (n_items == 0) return SB_OK;
  penalize_kernel<<<(n_items + 255) / 256, 256, 0, (hipStream_t)stream>>>(
      logits, vocab, item_row, item_token, item_count, n_items, repeat_penalty, presence_penalty,
      frequency_penalty, exact);
  return sb::check_launch("sb_penalize");
}

// logits [n_rows, vocab] in place: -inf wherever the row's bitmap (bitmaps uint8 [n_rows, n_bytes],
// bit i & 7 of byte i >> 3 for id i; ids past it are not allowed) does not allow the id.
extern "C" int sb_mask_logits(float *logits, int n_rows, int vocab, const uint8_t *bitmaps, int n_bytes,
                              void *stream) {
  SB_REQUIRE(logits && bitmaps, "sb_mask_logits: null pointer");
  SB_REQUIRE(n_rows >= 0 && vocab > 0 && n_bytes > 0, "sb_mask_logits: bad sizes rows=%d vocab=%d bytes=%d", n_rows,
             vocab, n_bytes);
  SB_SUPPORT(n_rows <= 65535, "sb_mask_logits: more than 65535 rows");
  if (n_rows == 0) return SB_OK;
  mask_logits_kernel<<<dim3((vocab + 255) / 256, n_rows), 256, 0, (hipStream_t)stream>>>(logits, vocab, bitmaps,
                                                                                        n_bytes);
  return sb::check_launch("sb_mask_logits");
}

// 64-bit words of scratch sb_top_candidates needs for rows of this length (0: none).  Rows of
// more than two parts go through stage 1.
extern "C" size_t sb_top_candidates_scratch(int n_rows, int vocab) {
  if (n_rows <= 0 || vocab <= 2 * kPartElems) return 0;
  return size_t(n_rows) * ((vocab + kPartElems - 1) / kPartElems) * kMaxCand;
}
// The longest row sb_top_candidates takes: what its second stage can hold of the parts' keys.
extern "C" int sb_top_candidates_max_vocab(void) { return kRowKeys * kSelThreads / kMaxCand * kPartElems; }

// cand_id int32 [n_rows, k], cand_z float [n_rows, k]: the k <= 256 best of every row by
// z = logit / temperature, ordered (z descending, id ascending); entries past the row's length
// hold id -1.  scratch: sb_top_candidates_scratch(n_rows, vocab) 64-bit words (may be NULL when 0).
extern "C" int sb_top_candidates(int32_t *cand_id, float *cand_z, const float *logits, int n_rows,
                                 int vocab, int k, float temperature, uint64_t *scratch, void *stream) {
  SB_REQUIRE(cand_id && cand_z && logits, "sb_top_candidates: null pointer");
  SB_REQUIRE(n_rows >= 0 && vocab > 0, "sb_top_candidates: bad sizes rows=%d vocab=%d", n_rows, vocab);
  SB_REQUIRE(temperature > 0.0f, "sb_top_candidates: temperature must be positive");
  SB_SUPPORT(k >= 1 && k <= kMaxCand, "sb_top_candidates: %d candidates asked, at most %d", k, kMaxCand);
  SB_SUPPORT(n_rows <= 65535, "sb_top_candidates: more than 65535 rows");
  SB_SUPPORT(vocab <= sb_top_candidates_max_vocab(), "sb_top_candidates: a row of %d logits, at most %d", vocab,
             sb_top_candidates_max_vocab());
  if (n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  if (sb_top_candidates_scratch(n_rows, vocab) == 0) {
    top_candidates_kernel<false><<<n_rows, kSelThreads, 0, s>>>(cand_id, cand_z, logits, nullptr, 0, vocab, k,
                                                                temperature);
    return sb::check_launch("sb_top_candidates");
  }
  SB_REQUIRE(scratch, "sb_top_candidates: no scratch for the parts' candidates");
  const int parts = (vocab + kPartElems - 1) / kPartElems;
  top_part_kernel<<<dim3(parts, n_rows), kSelThreads, 0, s>>>(scratch, logits, vocab, temperature);
  int rc = sb::check_launch("sb_top_candidates (parts)");
  if (rc != SB_OK) return rc;
  top_candidates_kernel<true><<<n_rows, kSelThreads, 0, s>>>(cand_id, cand_z, logits, scratch, parts * kMaxCand,
                                                             vocab, k, temperature);
  return sb::check_launch("sb_top_candidates");
}

// One token per row from its candidates (what sb_top_candidates wrote: k <= 256 per row, ordered
// (z descending, id ascending), id -1 past a short row's end): window, top-k (0: off), min-p
// (log_min_p = ln of it as a float; use_min_p 0: off), top-p (use_top_p 0: off), Gumbel-max under
// (seed, position[row], id).  token int32 [n_rows]: -1 for a row that keeps no candidate.
extern "C" int sb_draw(int32_t *token, const int32_t *cand_id, const float *cand_z, const int64_t *position,
                       int n_rows, int k, int top_k, int use_min_p, float log_min_p, int use_top_p, double top_p,
                       uint64_t seed, void *stream) {
  SB_REQUIRE(token && cand_id && cand_z && position, "sb_draw: null pointer");
  SB_REQUIRE(n_rows >= 0 && top_k >= 0, "sb_draw: bad sizes rows=%d top_k=%d", n_rows, top_k);
  SB_SUPPORT(k >= 1 && k <= kMaxCand, "sb_draw: %d candidates a row, at most %d", k, kMaxCand);
  if (n_rows == 0) return SB_OK;
  draw_kernel<int64_t><<<n_rows, 64, 0, (hipStream_t)stream>>>(token, cand_id, cand_z, position, 0, k, top_k,
                                                               use_min_p, log_min_p, use_top_p, top_p, seed);
  return sb::check_launch("sb_draw");
}

// The same for a decode step whose bookkeeping lives on the device: the position of row r's new
// token is length_before[r] + 1 (the token it feeds sits at length_before[r]).
extern "C" int sb_draw_after(int32_t *token, const int32_t *cand_id, const float *cand_z,
                             const int32_t *length_before, int n_rows, int k, int top_k, int use_min_p,
                             float log_min_p, int use_top_p, double top_p, uint64_t seed, void *stream) {
  SB_REQUIRE(token && cand_id && cand_z && length_before, "sb_draw_after: null pointer");
  SB_REQUIRE(n_rows >= 0 && top_k >= 0, "sb_draw_after: bad sizes rows=%d top_k=%d", n_rows, top_k);
  SB_SUPPORT(k >= 1 && k <= kMaxCand, "sb_draw_after: %d candidates a row, at most %d", k, kMaxCand);
  if (n_rows == 0) return SB_OK;
  draw_kernel<int32_t><<<n_rows, 64, 0, (hipStream_t)stream>>>(token, cand_id, cand_z, length_before, 1, k, top_k,
                                                               use_min_p, log_min_p, use_top_p, top_p, seed);
  return sb::check_launch("sb_draw_after");
}
