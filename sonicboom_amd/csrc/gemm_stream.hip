// bf16 matrix product for up to 128 rows against a packed matrix (decode steps and
// short prompts: the gate/up product, the head; qkv, output and down with K cut
// over the grid):  Y[t,n] = sum_k X[t,k] W[n,k].
//
// Like the few-row kernel it is bound by reading W once, and every wave loads its
// W fragments straight from global memory into MFMA operands.  With this many rows
// the X fragments are the problem: a wave needs TT of them (16 rows each) for every
// W fragment, and fetched per wave from cache they take more of the memory pipeline
// than the weights do.  Here the block's waves share X through LDS: the rows' next
// 256 k are staged once per block (two buffers, one barrier per 256 k) and each wave
// reads its fragments from there, while the waves split the block's output features
// between them (a wave owns 16 * R features, or R gate/up pairs, over all of K).  W
// loads run eight k-steps ahead of the MFMAs in a ring of registers.
//
// A CU works through its blocks at a rate that co-resident blocks share, so the time
// is set by the CU with the most work: 296 blocks of four waves on 256 CUs take 1.4
// times as long as 256.  The launcher therefore picks the waves per block (4 to 8) so
// that the blocks fill a whole number of rounds over the CUs as nearly as possible
// (gate/up of 18,944 features: 237 blocks of five waves, 47 against 68 us at 64 rows).
//
// MFMA roles: A = 16 rows of W, B = 16 rows of X, D[n][t]; a lane holds four
// consecutive n of one t.
#include "mfma.h"

namespace {

constexpr int kStepK = 32;                    // k per MFMA
constexpr int kAhead = 8;                     // k-steps of W in flight per wave
constexpr int kChunkK = kAhead * kStepK;      // k staged per LDS buffer: 256
constexpr int kRowChunks = kChunkK / 8;       // 16-byte groups of a staged row: 32
constexpr int kRowStride = kRowChunks + 1;    // in 16-byte units: one of padding, so that the
                                              // 16 rows a quarter-wave reads fall into 16 banks groups

struct StreamArgs {
  void *y;
  int y_dtype;
  const void *bias;
  int bias_dtype;
  const float *resid;
  int n_rows, n_out, n_in;
  // K cut over the grid (blockIdx.y): slice s multiplies k-steps [s * steps_per_slice, ...), a
  // multiple of eight of them, and writes its raw sums to partial [slice][n_rows][n_out]; NULL:
  // one slice and the epilogues below
  float *partial;
  int steps_per_slice;
  int gate;        // the gate's activation (an sb_gate) of the gated form
};


template <int TT, int G, int R, int W>
__global__ void __launch_bounds__(64 * W)
gemm_stream_kernel(const bf16_t *__restrict__ x, const bf16_t *__restrict__ w, StreamArgs a) {
  extern __shared__ uint4 xs_lds[];            // [2][TT * 16][kRowStride]
  constexpr int F = G * R;                     // W fragments per k-step and wave
  constexpr int kRows = TT * 16;
  constexpr int kBufUnits = kRows * kRowStride;
  constexpr int kThreads = 64 * W;
  constexpr int kXUnits = kRows * kRowChunks;               // 16-byte groups of a staged chunk
  constexpr int kXLoads = (kXUnits + kThreads - 1) / kThreads;   // loads per thread and chunk
  constexpr bool kXEven = kXUnits % kThreads == 0;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, q = lane >> 4;
  const int n_steps = (a.n_in + kStepK - 1) / kStepK;
  const int tiles_out = (a.n_out + 15) / 16;
  const int tile0 = (blockIdx.x * W + wave) * R;
  const int s0 = a.partial ? int(blockIdx.y) * a.steps_per_slice : 0;
  const int s1 = a.partial ? min(s0 + a.steps_per_slice, n_steps) : n_steps;

  floatx4_t acc[F][TT];
#pragma unroll
  for (int f = 0; f < F; ++f)
#pragma unroll
    for (int j = 0; j < TT; ++j) acc[f][j] = floatx4_t{0.f, 0.f, 0.f, 0.f};

  // Every load goes through a buffer descriptor, so that what lies outside (a tile past the
  // last, a k-step past the end, a row past the last) reads as zero without a branch: a branch
  // around a load makes the compiler wait for every load in flight.
  // W: one descriptor per fragment stream (tile, half): blocks of 1 KB up to this slice's end.
  __amdgpu_buffer_rsrc_t rsrc_w[F];
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const int tile = tile0 + i;
      const bf16_t *base = w + (size_t(g * tiles_out + min(tile, tiles_out - 1)) * n_steps) * 512;
      rsrc_w[g * R + i] = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<bf16_t *>(base), 0, tile < tiles_out ? uint32_t(s1) * 1024u : 0u, 0x00020000);
    }
  const __amdgpu_buffer_rsrc_t rsrc_x = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16_t *>(x), 0, uint32_t(size_t(a.n_rows) * a.n_in * 2), 0x00020000);

  // staging of X: thread's load i covers row (id / 32), 16-byte group (id % 32), id = tid + 256 i
  uint32_t x_off[kXLoads];
  int x_dst[kXLoads], x_k[kXLoads];
#pragma unroll
  for (int i = 0; i < kXLoads; ++i) {
    const int id = tid + kThreads * i;
    const int row = id / kRowChunks, c = id - row * kRowChunks;   // a row past the last when id >= kXUnits
    x_k[i] = c * 8;
    x_off[i] = uint32_t((size_t(min(row, a.n_rows)) * a.n_in + c * 8) * 2);   // row n_rows: outside
    x_dst[i] = row * kRowStride + c;
  }
  constexpr uint32_t kOutside = 0x80000000u;
  uint4 xs[kXLoads];
  const int chunk0 = s0 / kAhead;              // slices start on whole chunks
  auto issue_x = [&](int c) {
    const int chunk = chunk0 + c;
#pragma unroll
    for (int i = 0; i < kXLoads; ++i) {
      const uint32_t off = chunk * kChunkK + x_k[i] < a.n_in ? x_off[i] + uint32_t(chunk) * (kChunkK * 2) : kOutside;
      xs[i] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_x, int(off), 0, 0));
    }
  };
  auto store_x = [&](int buf) {
#pragma unroll
    for (int i = 0; i < kXLoads; ++i)
      if (kXEven || i + 1 < kXLoads || tid + kThreads * i < kXUnits) xs_lds[buf * kBufUnits + x_dst[i]] = xs[i];
  };

  uint4 ring[kAhead][F];
  uint32_t w_off = uint32_t(lane) * 16u + uint32_t(s0) * 1024u;   // of the next k-step to ask for
#pragma unroll
  for (int u = 0; u < kAhead; ++u) {
#pragma unroll
    for (int f = 0; f < F; ++f)
      ring[u][f] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_w[f], int(w_off), 0, 0));
    w_off += 1024u;
  }
  issue_x(0);
  store_x(0);
  __syncthreads();

  const int n_chunks = (s1 - s0 + kAhead - 1) / kAhead;
  for (int c = 0; c < n_chunks; ++c) {
    const bool more = c + 1 < n_chunks;
    if (more) issue_x(c + 1);
    const uint4 *buf = xs_lds + (c & 1) * kBufUnits;
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      uint4 b[TT];
#pragma unroll
      for (int j = 0; j < TT; ++j) b[j] = buf[(j * 16 + r) * kRowStride + u * 4 + q];
#pragma unroll
      for (int f = 0; f < F; ++f) {
#pragma unroll
        for (int j = 0; j < TT; ++j) acc[f][j] = mfma16(as_bf16x8(ring[u][f]), as_bf16x8(b[j]), acc[f][j]);
        ring[u][f] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_w[f], int(w_off), 0, 0));
      }
      w_off += 1024u;
    }
    if (more) store_x((c + 1) & 1);
    __syncthreads();
  }

  // D[n][t]: lane (q, r) holds n = 16 * tile + 4 q + 0..3 of row t = 16 j + r
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int nb = (tile0 + i) * 16 + q * 4;
#pragma unroll
    for (int j = 0; j < TT; ++j) {
      const int t = j * 16 + r;
      if (t >= a.n_rows) continue;
      const size_t row_off = size_t(t) * a.n_out;
      if (G == 1 && a.partial) {
        float *dst = a.partial + size_t(blockIdx.y) * a.n_rows * a.n_out + row_off;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (nb + e < a.n_out) dst[nb + e] = acc[i][j][e];
        continue;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int n = nb + e;
        if (n >= a.n_out) continue;
        float v = acc[i][j][e];
        if (G == 2) v = gate_act(v, a.gate) * acc[R + i][j][e];
        if (a.bias) v = v + ld_dyn(a.bias, a.bias_dtype, n);
        if (a.resid) v = v + a.resid[row_off + n];
        if (a.y_dtype == SB_F32) ((float *)a.y)[row_off + n] = v;
        else ((bf16_t *)a.y)[row_off + n] = f32_to_bf16(v);
      }
    }
  }
}

template <int TT, int G, int R, int W>
void launch_w(const bf16_t *x, const bf16_t *w, const StreamArgs &a, hipStream_t s) {
  const int tiles = (a.n_out + 15) / 16;
  const int per_block = W * R;
  const size_t lds = size_t(2) * TT * 16 * kRowStride * sizeof(uint4);
  auto kern = gemm_stream_kernel<TT, G, R, W>;
  static bool raised = false;   // once per instantiation: allow more than the default dynamic LDS
  if (lds > 48 * 1024 && !raised) {
    (void)hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, int(lds));
    raised = true;
  }
  const int n_steps = (a.n_in + kStepK - 1) / kStepK;
  const unsigned slices = a.partial ? unsigned((n_steps + a.steps_per_slice - 1) / a.steps_per_slice) : 1u;
  kern<<<dim3((tiles + per_block - 1) / per_block, slices), 64 * W, lds, s>>>(x, w, a);
}

// A call's hint (for tests and measurements; 0 = the launcher chooses): bits 0..7 the waves per
// block (4..8), bits 8..15 the K slices the partial form aims at (1..8).
inline int hint_waves(int hint) { return hint & 0xff; }
inline int hint_slices(int hint) { return (hint >> 8) & 0xff; }

// Waves per block: the count whose blocks fill whole rounds over the CUs best; more waves on a tie.
int waves_for(int tiles, int r, int force_waves) {
  if (force_waves >= 4 && force_waves <= 8) return force_waves;
  const int n_cu = sb::cu_count();
  int best = 4;
  long long best_cost = -1;
  for (int w = 4; w <= 8; ++w) {
    const int blocks = (tiles + w * r - 1) / (w * r);
    const long long cost = (long long)((blocks + n_cu - 1) / n_cu) * w;
    if (best_cost < 0 || cost <= best_cost) best = w, best_cost = cost;
  }
  return best;
}

// K cut over the grid for narrow matrices: waves per block and slices such that the blocks fill
// whole rounds over the CUs, every slice a whole number of staged chunks.  The cost of a choice:
// rounds x a block's k-steps (plus what a block costs before it streams) x the bytes a step
// moves (1 KB of W per wave from memory, 1 KB of X per 16 rows from L2, counted half), plus what
// the consumer pays per slice it has to add.
struct Cut {
  int waves, slices, steps_per_slice;
};
inline int row_tiles(int n_rows) { return n_rows <= 16 ? 1 : (n_rows <= 32 ? 2 : (n_rows <= 64 ? 4 : 8)); }
Cut cut_for(int tiles, int n_steps, int tt, int hint) {
  const int force_waves = hint_waves(hint), force_slices = hint_slices(hint);
  const int n_cu = sb::cu_count();
  Cut best{4, 1, (n_steps + kAhead - 1) / kAhead * kAhead};
  long long best_cost = -1;
  for (int want = 1; want <= 8; ++want) {
    if (force_slices && want != force_slices) continue;
    const int sps = ((n_steps + want - 1) / want + kAhead - 1) / kAhead * kAhead;
    const int slices = (n_steps + sps - 1) / sps;
    for (int w = 4; w <= 8; ++w) {
      if (force_waves >= 4 && force_waves <= 8 && w != force_waves) continue;
      const long long blocks = (long long)((tiles + w - 1) / w) * slices;
      // (+ 4 per wave: between choices that this prices alike, the one with fewer waves and slices
      // measured 1 to 2 % faster in whole decode steps of the 14B and 32B sizes at up to 16 rows)
      const long long cost = (blocks + n_cu - 1) / n_cu * (sps + 24) * (2 * w + tt) + 12LL * slices + 4LL * w;
      if (best_cost < 0 || cost < best_cost) best = Cut{w, slices, sps}, best_cost = cost;
    }
  }
  return best;
}

template <int TT>
void launch_cut(const bf16_t *x, const bf16_t *w, const StreamArgs &a, int waves, hipStream_t s) {
  switch (waves) {
    case 4: return launch_w<TT, 1, 1, 4>(x, w, a, s);
    case 5: return launch_w<TT, 1, 1, 5>(x, w, a, s);
    case 6: return launch_w<TT, 1, 1, 6>(x, w, a, s);
    case 7: return launch_w<TT, 1, 1, 7>(x, w, a, s);
    default: return launch_w<TT, 1, 1, 8>(x, w, a, s);
  }
}

template <int TT, int G, int R>
void launch(const bf16_t *x, const bf16_t *w, const StreamArgs &a, int hint, hipStream_t s) {
  switch (waves_for((a.n_out + 15) / 16, R, hint_waves(hint))) {
    case 4: return launch_w<TT, G, R, 4>(x, w, a, s);
    case 5: return launch_w<TT, G, R, 5>(x, w, a, s);
    case 6: return launch_w<TT, G, R, 6>(x, w, a, s);
    case 7: return launch_w<TT, G, R, 7>(x, w, a, s);
    default: return launch_w<TT, G, R, 8>(x, w, a, s);
  }
}

}  // namespace

// Rows of X this kernel takes.
extern "C" int sb_gemm_stream_max_rows(void) { return 128; }

// Y = X W^T (+bias) (+resid), or with gated != 0: Y = silu(X Wg^T) * (X Wu^T) for the packed
// halves [Wg; Wu].  X [n_rows, n_in] bf16, n_rows <= 128, n_in a multiple of 8; W in the packed
// tile layout (16 x 32 tiles of 1 KB in fragment order, tiles of a row block consecutive in k).
extern "C" int sb_gemm_stream_bf16(void *y, int y_dtype, const void *x, const void *w, const void *bias,
                                   int bias_dtype, const float *resid, int n_rows, int n_out, int n_in,
                                   int gated, int hint, void *stream) {
  SB_REQUIRE(y && x && w, "sb_gemm_stream_bf16: null pointer");
  SB_REQUIRE(n_rows >= 0 && n_out > 0 && n_in > 0, "sb_gemm_stream_bf16: bad sizes rows=%d out=%d in=%d",
             n_rows, n_out, n_in);
  SB_REQUIRE(sb::valid_dtype(y_dtype) && (!bias || sb::valid_dtype(bias_dtype)),
             "sb_gemm_stream_bf16: unknown dtype");
  SB_SUPPORT(n_rows <= 128, "sb_gemm_stream_bf16: %d rows, at most 128", n_rows);
  SB_SUPPORT(n_in % 8 == 0, "sb_gemm_stream_bf16: inner size %d is not a multiple of 8", n_in);
  SB_SUPPORT((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) % 16 == 0,
             "sb_gemm_stream_bf16: operands must be 16-byte aligned");
  SB_REQUIRE(!(gated && (bias || resid)), "sb_gemm_stream_bf16: the gated form takes no bias or residual");
  // the kernel addresses X and each fragment stream of W with 32-bit byte offsets
  SB_SUPPORT((unsigned long long)(n_rows + 1) * n_in * 2 < (1ull << 31) && (unsigned long long)n_in * 32 < (1ull << 31),
             "sb_gemm_stream_bf16: inner size %d is too large", n_in);
  if (n_rows == 0) return SB_OK;
  hipStream_t s = (hipStream_t)stream;
  SB_SUPPORT(gated >= SB_GATE_NONE && gated <= SB_GATE_GELU_TANH, "sb_gemm_stream_bf16: unknown gate activation %d", gated);
  const StreamArgs a{y, y_dtype, bias, bias_dtype, resid, n_rows, n_out, n_in, nullptr, 0, gated};
  const bf16_t *xb = (const bf16_t *)x, *wb = (const bf16_t *)w;
  const int tt = row_tiles(n_rows);
  if (gated) {
    if (tt == 1) launch<1, 2, 1>(xb, wb, a, hint, s);
    else if (tt == 2) launch<2, 2, 1>(xb, wb, a, hint, s);
    else if (tt == 4) launch<4, 2, 1>(xb, wb, a, hint, s);
    else launch<8, 2, 1>(xb, wb, a, hint, s);
  } else {
    if (tt == 1) launch<1, 1, 2>(xb, wb, a, hint, s);
    else if (tt == 2) launch<2, 1, 2>(xb, wb, a, hint, s);
    else if (tt == 4) launch<4, 1, 2>(xb, wb, a, hint, s);
    else launch<8, 1, 2>(xb, wb, a, hint, s);
  }
  return sb::check_launch("sb_gemm_stream_bf16");
}

// K slices sb_gemm_stream_partial_bf16 will produce for these sizes.
extern "C" int sb_gemm_stream_slices(int n_rows, int n_out, int n_in, int hint) {
  if (n_rows <= 0 || n_out <= 0 || n_in <= 0) return 1;
  return cut_for((n_out + 15) / 16, (n_in + kStepK - 1) / kStepK, row_tiles(n_rows), hint).slices;
}

// The raw product in K slices, for a consumer that adds them (and bias, residual, ...) itself:
// partial float [slices][n_rows][n_out], slices = sb_gemm_stream_slices(...).  Operands as above.
extern "C" int sb_gemm_stream_partial_bf16(float *partial, const void *x, const void *w, int n_rows, int n_out,
                                           int n_in, int hint, void *stream) {
  SB_REQUIRE(partial && x && w, "sb_gemm_stream_partial_bf16: null pointer");
  SB_REQUIRE(n_rows >= 0 && n_out > 0 && n_in > 0, "sb_gemm_stream_partial_bf16: bad sizes");
  SB_SUPPORT(n_rows <= 64, "sb_gemm_stream_partial_bf16: %d rows, at most 64", n_rows);
  SB_SUPPORT(n_in % 8 == 0, "sb_gemm_stream_partial_bf16: inner size %d is not a multiple of 8", n_in);
  SB_SUPPORT((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) % 16 == 0,
             "sb_gemm_stream_partial_bf16: operands must be 16-byte aligned");
  SB_SUPPORT((unsigned long long)(n_rows + 1) * n_in * 2 < (1ull << 31) && (unsigned long long)n_in * 32 < (1ull << 31),
             "sb_gemm_stream_partial_bf16: inner size %d is too large", n_in);
  if (n_rows == 0) return SB_OK;
  const Cut c = cut_for((n_out + 15) / 16, (n_in + kStepK - 1) / kStepK, row_tiles(n_rows), hint);
  const StreamArgs a{nullptr, SB_F32, nullptr, 0, nullptr, n_rows, n_out, n_in, partial, c.steps_per_slice, 0};
  const bf16_t *xb = (const bf16_t *)x, *wb = (const bf16_t *)w;
  hipStream_t s = (hipStream_t)stream;
  if (n_rows <= 16) launch_cut<1>(xb, wb, a, c.waves, s);
  else if (n_rows <= 32) launch_cut<2>(xb, wb, a, c.waves, s);
  else launch_cut<4>(xb, wb, a, c.waves, s);
  return sb::check_launch("sb_gemm_stream_partial_bf16");
}
