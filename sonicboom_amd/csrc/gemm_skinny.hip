// bf16 matrix product for a few rows (decode):  Y[t,n] = sum_k X[t,k] W[n,k],
// t <= 64, with the epilogues the model needs (bias, residual, SiLU gate).
//
// The step is bound by reading W once from HBM.  A block owns 16*R output
// features; its four waves take a quarter each of the k-steps of the block's K
// slice, each loading W fragments straight from global
// memory into MFMA operands (16 rows x 64 bytes per load, every byte of W
// read once) and the matching X fragments from cache.  The waves' partial
// tiles are summed through shared memory in wave order, so the result does
// not depend on timing.  When the matrix has too few rows to fill the GPU, K
// is also split over the grid: slices go to a scratch buffer and a second
// kernel adds them in slice order and applies the epilogue.
//
// MFMA roles: A = 16 rows of W, B = 16 rows of X, D[n][t]; a lane then holds
// four consecutive n of one t, a 16-byte store.
#include "mfma.h"

namespace {

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;
constexpr int kStepK = 32;   // k per MFMA

struct Epilogue {
  void *y;
  int y_dtype;
  const void *bias;
  int bias_dtype;
  const float *resid;
  int n_rows, n_out;
  int gated;
};


__device__ __forceinline__ void store_out(const Epilogue &e, int t, int n, float v) {
  if (e.bias) v = v + ld_dyn(e.bias, e.bias_dtype, n);
  const size_t idx = size_t(t) * e.n_out + n;
  if (e.resid) v = v + e.resid[idx];
  if (e.y_dtype == SB_F32) ((float *)e.y)[idx] = v;
  else ((bf16_t *)e.y)[idx] = f32_to_bf16(v);
}

// G = 1: plain.  G = 2: rows n and n_out + n of W are gate and up of output n.
// PACKED: W is stored tile by tile in MFMA fragment order (ops.pack_weight lays it out): the
// fragment of row tile nb and k-step ks is the 1 KB block (nb * n_steps + ks), lane l's eight
// elements at l * 8; rows and k are padded with zeros to whole tiles.
template <int R, int TT, int G, bool PACKED>
__global__ void __launch_bounds__(kThreads)
gemm_skinny_kernel(const bf16_t *__restrict__ x, const bf16_t *__restrict__ w, Epilogue ep,
                   float *__restrict__ partial, int n_in, int steps_per_slice) {
  extern __shared__ float red[];   // [kWaves][G*R*TT][64][4]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 15, q = lane >> 4;
  const int n0 = blockIdx.x * (16 * R);
  const int n_steps = (n_in + kStepK - 1) / kStepK;
  const int s_begin = blockIdx.y * steps_per_slice;
  const int s_end = min(s_begin + steps_per_slice, n_steps);
  const int n_w_rows = ep.n_out * G;

  floatx4_t acc[G * R][TT];
#pragma unroll
  for (int i = 0; i < G * R; ++i)
#pragma unroll
    for (int j = 0; j < TT; ++j) acc[i][j] = floatx4_t{0.f, 0.f, 0.f, 0.f};

  const bf16_t *w_row[G * R];
  bool w_ok[G * R];
  const int tiles_out = (ep.n_out + 15) / 16;
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const int n = n0 + i * 16 + r;
      if (PACKED) {
        const int tile = blockIdx.x * R + i;
        w_ok[g * R + i] = tile < tiles_out;
        w_row[g * R + i] = w + (size_t(g * tiles_out + min(tile, tiles_out - 1)) * n_steps) * 512 + lane * 8;
      } else {
        w_ok[g * R + i] = n < ep.n_out;
        const int row = min(g * ep.n_out + n, n_w_rows - 1);
        w_row[g * R + i] = w + size_t(row) * n_in;
      }
    }
  const bf16_t *x_row[TT];
  bool x_ok[TT];
#pragma unroll
  for (int j = 0; j < TT; ++j) {
    const int t = j * 16 + r;
    x_ok[j] = t < ep.n_rows;
    x_row[j] = x + size_t(min(t, ep.n_rows - 1)) * n_in;
  }

  // Each wave takes a contiguous quarter of the slice's k-steps, so that it streams whole
  // cache lines of every row; U steps' fragments are requested before the first MFMA, to
  // keep loads in flight.
  constexpr int U = (G * R + TT <= 4) ? 4 : 2;
  const int per_wave = (s_end - s_begin + kWaves - 1) / kWaves;
  const int w_begin = s_begin + wave * per_wave;
  const int w_end = min(w_begin + per_wave, s_end);
  for (int s = w_begin; s < w_end; s += U) {
    uint4 a[U][G * R], b[U][TT];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int ss = s + u;
      const int k = ss * kStepK + q * 8;
      // n_in is a multiple of 8: a 16-byte group lies inside a row or outside as a whole
      const bool k_ok = ss < w_end && k < n_in;
#pragma unroll
      for (int i = 0; i < G * R; ++i)
        a[u][i] = PACKED ? ld16(w_row[i] + size_t(ss) * 512, ss < w_end && w_ok[i])
                         : ld16(w_row[i] + k, k_ok && w_ok[i]);
#pragma unroll
      for (int j = 0; j < TT; ++j) b[u][j] = ld16(x_row[j] + k, k_ok && x_ok[j]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int i = 0; i < G * R; ++i)
#pragma unroll
        for (int j = 0; j < TT; ++j)
          acc[i][j] = mfma16(as_bf16x8(a[u][i]), as_bf16x8(b[u][j]), acc[i][j]);
  }

  // Sum the waves' partial tiles in wave order.
  constexpr int kTiles = G * R * TT;
#pragma unroll
  for (int i = 0; i < G * R; ++i)
#pragma unroll
    for (int j = 0; j < TT; ++j) {
      float *dst = red + ((size_t(wave) * kTiles + (i * TT + j)) * 64 + lane) * 4;
      *reinterpret_cast<floatx4_t *>(dst) = acc[i][j];
    }
  __syncthreads();

  // Thread e owns lane-quad (tile, lane) pairs: R*TT output tiles of 64 quads.
  for (int e = threadIdx.x; e < R * TT * 64; e += kThreads) {
    const int tile = e >> 6, l = e & 63;
    const int i = tile / TT, j = tile - i * TT;
    floatx4_t v[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const int src_tile = (g * R + i) * TT + j;
      floatx4_t sum = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int wv = 0; wv < kWaves; ++wv)
        sum += *reinterpret_cast<const floatx4_t *>(red + ((size_t(wv) * kTiles + src_tile) * 64 + l) * 4);
      v[g] = sum;
    }
    const int t = j * 16 + (l & 15);
    const int nb = n0 + i * 16 + (l >> 4) * 4;
    if (t >= ep.n_rows) continue;
    if (partial != nullptr) {
      // grid split-K: raw sums of this slice, [slice][t][G*n_out]
#pragma unroll
      for (int g = 0; g < G; ++g)
#pragma unroll
        for (int c = 0; c < 4; ++c)
          if (nb + c < ep.n_out)
            partial[(size_t(blockIdx.y) * ep.n_rows + t) * n_w_rows + g * ep.n_out + nb + c] = v[g][c];
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        if (nb + c >= ep.n_out) continue;
        float val = v[0][c];
        if (G == 2) val = gate_act(val, ep.gated) * v[1][c];
        store_out(ep, t, nb + c, val);
      }
    }
  }
}

__global__ void __launch_bounds__(256)
reduce_slices_kernel(const float *__restrict__ partial, Epilogue ep, int n_slices) {
  const size_t total = size_t(ep.n_rows) * ep.n_out;
  const size_t idx = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int t = int(idx / ep.n_out), n = int(idx - size_t(t) * ep.n_out);
  const int width = ep.n_out * (ep.gated ? 2 : 1);
  float g = 0.f, u = 0.f;
  for (int s = 0; s < n_slices; ++s) {
    const float *p = partial + (size_t(s) * ep.n_rows + t) * width;
    g += p[n];
    if (ep.gated) u += p[ep.n_out + n];
  }
  store_out(ep, t, n, ep.gated ? gate_act(g, ep.gated) * u : g);
}

template <int R, int TT, int G, bool PACKED>
void launch(const bf16_t *x, const bf16_t *w, const Epilogue &ep, float *partial, int n_in,
            int n_slices, int steps_per_slice, hipStream_t s) {
  dim3 grid((ep.n_out + 16 * R - 1) / (16 * R), n_slices);
  const size_t lds = size_t(kWaves) * G * R * TT * 64 * 4 * sizeof(float);
  auto kern = gemm_skinny_kernel<R, TT, G, PACKED>;
  static bool raised = false;   // once per instantiation: allow more than the default dynamic LDS
  if (lds > 48 * 1024 && !raised) {
    (void)hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, int(lds));
    raised = true;
  }
  kern<<<grid, kThreads, lds, s>>>(x, w, ep, partial, n_in, steps_per_slice);
}

template <int G, bool PACKED>
void launch_rt(int R, int TT, const bf16_t *x, const bf16_t *w, const Epilogue &ep, float *partial,
               int n_in, int n_slices, int steps_per_slice, hipStream_t s) {
#define SB_CASE(r, tt) \
  if (R == r && TT == tt) \
  return launch<r, tt, G, PACKED>(x, w, ep, partial, n_in, n_slices, steps_per_slice, s)
  SB_CASE(1, 1); SB_CASE(1, 2); SB_CASE(1, 4);
  SB_CASE(2, 1); SB_CASE(2, 2); SB_CASE(2, 4);
  if (G == 1) { SB_CASE(4, 1); SB_CASE(4, 2); SB_CASE(4, 4); }
#undef SB_CASE
}

}  // namespace

// Rows of X this kernel takes at most.
extern "C" int sb_gemm_skinny_max_rows(void) { return 64; }

// Floats of scratch the call may need (0 when it will not split K over the grid).
extern "C" size_t sb_gemm_skinny_scratch(int n_rows, int n_out, int n_in, int gated);

namespace {
struct Plan {
  int R, TT, n_slices, steps_per_slice;
};
Plan plan_for(int n_rows, int n_out, int n_in, int gated) {
  Plan p;
  p.TT = n_rows <= 16 ? 1 : (n_rows <= 32 ? 2 : 4);
  const int tiles = (n_out + 15) / 16;
  // Measured on MI355X.  Up to 16 rows: one row tile per block streams best, and K is cut
  // into slices until about a thousand blocks exist.  More rows: every X fragment a wave loads
  // must serve several row tiles (it comes from L2, and there are TT of them per W fragment), so
  // a wave takes four row tiles (two gated pairs) and fewer, fatter blocks are better.
  const int n_steps = (n_in + kStepK - 1) / kStepK;
  int want_blocks;
  if (p.TT == 1) {
    p.R = 1;
    want_blocks = 1024;
  } else {
    p.R = gated ? 2 : 4;
    want_blocks = 224;
  }
  const int blocks = (tiles + p.R - 1) / p.R;
  int slices = 1;
  if (blocks < want_blocks) {
    slices = (want_blocks + blocks - 1) / blocks;
    const int most = n_steps / (kWaves * 4);   // every wave keeps at least four steps
    if (slices > most) slices = most;
    if (slices > 8) slices = 8;     // what the kernels that add the slices take
    if (slices < 1) slices = 1;
  }
  p.steps_per_slice = (n_steps + slices - 1) / slices;
  p.n_slices = (n_steps + p.steps_per_slice - 1) / p.steps_per_slice;
  return p;
}
}  // namespace

extern "C" size_t sb_gemm_skinny_scratch(int n_rows, int n_out, int n_in, int gated) {
  if (n_rows <= 0 || n_out <= 0 || n_in <= 0) return 0;
  const Plan p = plan_for(n_rows, n_out, n_in, gated);
  return p.n_slices > 1 ? size_t(p.n_slices) * n_rows * n_out * (gated ? 2 : 1) : 0;
}

// Y = X W^T (+bias) (+resid), or with gated != 0: Y = silu(X Wg^T) * (X Wu^T) where W = [Wg; Wu]
// is [2*n_out, n_in].  X [n_rows, n_in] and W are bf16; n_rows <= 64; n_in a multiple of 8.
// packed != 0: W is in the packed tile layout.
extern "C" int sb_gemm_skinny_bf16(void *y, int y_dtype, const void *x, const void *w, const void *bias,
                                   int bias_dtype, const float *resid, int n_rows, int n_out, int n_in,
                                   int gated, int packed, float *scratch, size_t scratch_floats,
                                   void *stream) {
  SB_REQUIRE(y && x && w, "sb_gemm_skinny_bf16: null pointer");
  SB_REQUIRE(n_rows >= 0 && n_out > 0 && n_in > 0, "sb_gemm_skinny_bf16: bad sizes rows=%d out=%d in=%d",
             n_rows, n_out, n_in);
  SB_REQUIRE(sb::valid_dtype(y_dtype) && (!bias || sb::valid_dtype(bias_dtype)),
             "sb_gemm_skinny_bf16: unknown dtype");
  SB_SUPPORT(n_rows <= 64, "sb_gemm_skinny_bf16: %d rows, at most 64", n_rows);
  SB_SUPPORT(n_in % 8 == 0, "sb_gemm_skinny_bf16: inner size %d is not a multiple of 8", n_in);
  SB_SUPPORT((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) % 16 == 0,
             "sb_gemm_skinny_bf16: operands must be 16-byte aligned");
  SB_REQUIRE(!(gated && (bias || resid)), "sb_gemm_skinny_bf16: the gated form takes no bias or residual");
  if (n_rows == 0) return SB_OK;
  const Plan p = plan_for(n_rows, n_out, n_in, gated);
  const size_t need = p.n_slices > 1 ? size_t(p.n_slices) * n_rows * n_out * (gated ? 2 : 1) : 0;
  SB_REQUIRE(need == 0 || (scratch && scratch_floats >= need),
             "sb_gemm_skinny_bf16: scratch of %zu floats needed, %zu given", need, scratch_floats);
  hipStream_t s = (hipStream_t)stream;
  SB_SUPPORT(gated >= SB_GATE_NONE && gated <= SB_GATE_GELU_TANH, "sb_gemm_skinny_bf16: unknown gate activation %d", gated);
  Epilogue ep{y, y_dtype, bias, bias_dtype, resid, n_rows, n_out, gated};
  float *partial = p.n_slices > 1 ? scratch : nullptr;
  const bf16_t *xb = (const bf16_t *)x, *wb = (const bf16_t *)w;
  if (gated && packed) launch_rt<2, true>(p.R, p.TT, xb, wb, ep, partial, n_in, p.n_slices, p.steps_per_slice, s);
  else if (gated) launch_rt<2, false>(p.R, p.TT, xb, wb, ep, partial, n_in, p.n_slices, p.steps_per_slice, s);
  else if (packed) launch_rt<1, true>(p.R, p.TT, xb, wb, ep, partial, n_in, p.n_slices, p.steps_per_slice, s);
  else launch_rt<1, false>(p.R, p.TT, xb, wb, ep, partial, n_in, p.n_slices, p.steps_per_slice, s);
  int rc = sb::check_launch("sb_gemm_skinny_bf16");
  if (rc != SB_OK) return rc;
  if (p.n_slices > 1) {
    const size_t total = size_t(n_rows) * n_out;
    reduce_slices_kernel<<<unsigned((total + 255) / 256), 256, 0, s>>>(scratch, ep, p.n_slices);
    rc = sb::check_launch("sb_gemm_skinny_bf16 (slice sum)");
  }
  return rc;
}

// K slices sb_gemm_skinny_partial_bf16 will produce for these sizes.
extern "C" int sb_gemm_skinny_slices(int n_rows, int n_out, int n_in) {
  if (n_rows <= 0 || n_out <= 0 || n_in <= 0) return 1;
  return plan_for(n_rows, n_out, n_in, 0).n_slices;
}

// The raw product in K slices, for a consumer that adds them (and bias, residual, ...) itself:
// partial float [slices][n_rows][n_out], slices = sb_gemm_skinny_slices(...), slice s holding
// sum over its k range of X[t,k] W[n,k].
extern "C" int sb_gemm_skinny_partial_bf16(float *partial, const void *x, const void *w, int n_rows,
                                           int n_out, int n_in, int packed, void *stream) {
  SB_REQUIRE(partial && x && w, "sb_gemm_skinny_partial_bf16: null pointer");
  SB_REQUIRE(n_rows >= 0 && n_out > 0 && n_in > 0, "sb_gemm_skinny_partial_bf16: bad sizes");
  SB_SUPPORT(n_rows <= 64, "sb_gemm_skinny_partial_bf16: %d rows, at most 64", n_rows);
  SB_SUPPORT(n_in % 8 == 0, "sb_gemm_skinny_partial_bf16: inner size %d is not a multiple of 8", n_in);
  SB_SUPPORT((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) % 16 == 0,
             "sb_gemm_skinny_partial_bf16: operands must be 16-byte aligned");
  if (n_rows == 0) return SB_OK;
  const Plan p = plan_for(n_rows, n_out, n_in, 0);
  Epilogue ep{nullptr, SB_F32, nullptr, 0, nullptr, n_rows, n_out, 0};
  const bf16_t *xb = (const bf16_t *)x, *wb = (const bf16_t *)w;
  hipStream_t s = (hipStream_t)stream;
  if (packed) launch_rt<1, true>(p.R, p.TT, xb, wb, ep, partial, n_in, p.n_slices, p.steps_per_slice, s);
  else launch_rt<1, false>(p.R, p.TT, xb, wb, ep, partial, n_in, p.n_slices, p.steps_per_slice, s);
  return sb::check_launch("sb_gemm_skinny_partial_bf16");
}
