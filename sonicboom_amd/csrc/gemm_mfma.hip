// bf16 matrix product for many rows (prefill):  Y[t,n] = sum_k X[t,k] W[n,k]
// on the matrix cores, with the model's epilogues fused: bias, float32
// residual, SiLU gate, float32 or bfloat16 output.
//
// A block of 256 threads (2 x 2 waves) owns a 128 x 128 tile of Y and walks K
// in steps of 64.  Both operand tiles go global -> registers -> LDS, the next
// step's loads being issued before the current step's MFMAs (two LDS buffers,
// one barrier per step).  An LDS row holds 64 k (128 bytes, eight 16-byte
// chunks); chunk c of row r is stored at chunk c ^ (r & 7), which makes the
// 16-byte fragment reads of eight consecutive lanes fall on distinct banks.
// A wave owns 64 x 64: 2 x 2 tiles of v_mfma_f32_32x32x16_bf16, A = rows of X,
// B = rows of W, so a lane holds one output column of 16 rows.
//
// Block order: consecutive block numbers go to different XCDs (each with its
// own L2).  The grid is walked so that the blocks one XCD runs at a time share
// their X rows and neighbouring W rows.
#include "mfma.cuh"

namespace {

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int kThreads = 256;
constexpr int kChunksPerRow = BK / 8;                       // 16-byte chunks in an LDS row
constexpr int kLoadsA = BM * kChunksPerRow / kThreads;      // 4
constexpr int kLoadsB = BN * kChunksPerRow / kThreads;      // 4
constexpr int kXcds = 8;

struct Args {
  void *y;
  int y_dtype;
  const bf16_t *x, *w;
  const void *bias;
  int bias_dtype;
  const float *resid;
  int n_rows, n_out, n_in;
  int gated;       // W is [2*n_out, n_in]: rows n (gate) and n_out + n (up)
  int tiles_m, tiles_n;
  int w_tiles;     // packed W: 16-row tiles of one half (ceil(n_out / 16))
  int w_steps;     // packed W: 32-wide k-steps (ceil(n_in / 32))
};

__device__ __forceinline__ int swz(int row, int chunk) { return row * kChunksPerRow + (chunk ^ (row & 7)); }

__device__ __forceinline__ float silu_f(float g) { return g / (1.0f + expf(-g)); }

// PACKED: W comes in the packed tile layout (1 KB blocks of 16 rows x 32 k in fragment order,
// zero padded), which makes its global loads contiguous and free of bounds checks.
template <int GATED, bool PACKED>
__global__ void __launch_bounds__(kThreads)
gemm_mfma_kernel(Args a) {
  __shared__ uint4 lds_a[2][BM * kChunksPerRow];
  __shared__ uint4 lds_b[2][BN * kChunksPerRow];

  // XCD-aware order: hardware sends block b to XCD b % 8.  When the count divides, XCD x
  // gets the contiguous run of tiles [x * per, (x + 1) * per), which share rows of X and W in
  // that XCD's L2.
  const int n_blocks = a.tiles_m * a.tiles_n;
  int bid = blockIdx.x;
  if (n_blocks % kXcds == 0) bid = (bid % kXcds) * (n_blocks / kXcds) + bid / kXcds;
  // tiles of one column of N (same W rows) are neighbours: m runs fastest
  const int tn = bid / a.tiles_m, tm = bid - tn * a.tiles_m;
  const int t0 = tm * BM;
  const int n0 = tn * (GATED ? BN / 2 : BN);

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wm = wave >> 1, wn = wave & 1;

  // global -> register staging: thread handles chunk ids tid + 256 * i
  const bf16_t *ga[kLoadsA];
  const bf16_t *gb[kLoadsB];
  bool oka[kLoadsA], okb[kLoadsB];
  int sa[kLoadsA], sb_[kLoadsB], ca[kLoadsA], cb[kLoadsB];
#pragma unroll
  for (int i = 0; i < kLoadsA; ++i) {
    const int id = tid + kThreads * i, row = id / kChunksPerRow, c = id % kChunksPerRow;
    const int t = t0 + row;
    oka[i] = t < a.n_rows;
    ga[i] = a.x + size_t(min(t, a.n_rows - 1)) * a.n_in + c * 8;
    sa[i] = swz(row, c);
    ca[i] = c * 8;
  }
  int step_b[kLoadsB];    // packed: which of the two k-steps of a BK stage this load takes
#pragma unroll
  for (int i = 0; i < kLoadsB; ++i) {
    if (PACKED) {
      // load id -> 1 KB block (id / 64) = (row tile of the LDS tile, k-step), lane id % 64
      const int id = tid + kThreads * i, blk = id >> 6, l = id & 63;
      const int rt = blk >> 1, j = blk & 1;      // LDS rows rt * 16 .., k-step j of the stage
      int tile;
      if (GATED) {
        const int half = rt >> 2, within = rt & 3;
        tile = (within >> 1) * a.w_tiles + min(n0 / 16 + half * 2 + (within & 1), a.w_tiles - 1);
      } else {
        tile = min(n0 / 16 + rt, a.w_tiles - 1);
      }
      okb[i] = true;
      gb[i] = a.w + size_t(tile) * a.w_steps * 512 + size_t(l) * 8;
      sb_[i] = swz(rt * 16 + (l & 15), j * 4 + (l >> 4));
      cb[i] = 0;
      step_b[i] = j;
      continue;
    }
    step_b[i] = 0;
    const int id = tid + kThreads * i, row = id / kChunksPerRow, c = id % kChunksPerRow;
    int n;       // output feature, and the row of W that feeds LDS row `row`
    int wrow;
    if (GATED) {
      // LDS rows [0,32) gate of features n0..n0+31, [32,64) up of the same, [64,96) gate of
      // n0+32.., [96,128) up of the same: a wave's two B tiles are gate and up of 32 features.
      const int half = row >> 6, within = row & 63, is_up = within >> 5;
      n = n0 + half * 32 + (within & 31);
      wrow = is_up * a.n_out + n;
    } else {
      n = n0 + row;
      wrow = n;
    }
    okb[i] = n < a.n_out;
    gb[i] = a.w + size_t(okb[i] ? wrow : 0) * a.n_in + c * 8;
    sb_[i] = swz(row, c);
    cb[i] = c * 8;
  }

  floatx16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  uint4 ra[kLoadsA], rb[kLoadsB];
  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < kLoadsA; ++i) ra[i] = ld16(ga[i] + k0, oka[i] && (k0 + ca[i]) < a.n_in);
#pragma unroll
    for (int i = 0; i < kLoadsB; ++i) {
      if (PACKED) {
        const int ks = k0 / 32 + step_b[i];
        rb[i] = ld16(gb[i] + size_t(ks) * 512, ks < a.w_steps);
      } else {
        rb[i] = ld16(gb[i] + k0, okb[i] && (k0 + cb[i]) < a.n_in);
      }
    }
  };
  auto store_lds = [&](int buf) {
#pragma unroll
    for (int i = 0; i < kLoadsA; ++i) lds_a[buf][sa[i]] = ra[i];
#pragma unroll
    for (int i = 0; i < kLoadsB; ++i) lds_b[buf][sb_[i]] = rb[i];
  };

  const int n_k = (a.n_in + BK - 1) / BK;
  load_global(0);
  store_lds(0);
  __syncthreads();

  const int frag_row = lane & 31, frag_c = lane >> 5;   // row within a 32-row tile, chunk within a k16 step
  for (int kt = 0; kt < n_k; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < n_k) load_global((kt + 1) * BK);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      const int c = ks * 2 + frag_c;
      bf16x8_t fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) fa[i] = as_bf16x8(lds_a[buf][swz(wm * 64 + i * 32 + frag_row, c)]);
#pragma unroll
      for (int j = 0; j < 2; ++j) fb[j] = as_bf16x8(lds_b[buf][swz(wn * 64 + j * 32 + frag_row, c)]);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = mfma32(fa[i], fb[j], acc[i][j]);
    }
    if (kt + 1 < n_k) store_lds(buf ^ 1);
    __syncthreads();
  }

  // Epilogue.  acc[i][j][e]: row = 8 * (e / 4) + 4 * (lane / 32) + e % 4, column = lane % 32.
  const int col = lane & 31, row_base = (lane >> 5) * 4;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int t = t0 + wm * 64 + i * 32 + 8 * (e >> 2) + row_base + (e & 3);
      if (t >= a.n_rows) continue;
      if (GATED) {
        const int n = n0 + wn * 32 + col;
        if (n < a.n_out) {
          const float v = silu_f(acc[i][0][e]) * acc[i][1][e];
          const size_t idx = size_t(t) * a.n_out + n;
          if (a.y_dtype == SB_F32) ((float *)a.y)[idx] = v;
          else ((bf16_t *)a.y)[idx] = f32_to_bf16(v);
        }
      } else {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int n = n0 + wn * 64 + j * 32 + col;
          if (n >= a.n_out) continue;
          float v = acc[i][j][e];
          if (a.bias) v = v + ld_dyn(a.bias, a.bias_dtype, n);
          const size_t idx = size_t(t) * a.n_out + n;
          if (a.resid) v = v + a.resid[idx];
          if (a.y_dtype == SB_F32) ((float *)a.y)[idx] = v;
          else ((bf16_t *)a.y)[idx] = f32_to_bf16(v);
        }
      }
    }
  }
}

}  // namespace

// Y = X W^T (+bias) (+resid), or gated: Y = silu(X Wg^T) * (X Wu^T), W = [Wg; Wu].
// X [n_rows, n_in] and W bf16, n_in a multiple of 8, operands 16-byte aligned; packed != 0: W is
// in the packed tile layout.
extern "C" int sb_gemm_mfma_bf16(void *y, int y_dtype, const void *x, const void *w, const void *bias,
                                 int bias_dtype, const float *resid, int n_rows, int n_out, int n_in,
                                 int gated, int packed, void *stream) {
  SB_REQUIRE(y && x && w, "sb_gemm_mfma_bf16: null pointer");
  SB_REQUIRE(n_rows >= 0 && n_out > 0 && n_in > 0, "sb_gemm_mfma_bf16: bad sizes rows=%d out=%d in=%d",
             n_rows, n_out, n_in);
  SB_REQUIRE(sb::valid_dtype(y_dtype) && (!bias || sb::valid_dtype(bias_dtype)),
             "sb_gemm_mfma_bf16: unknown dtype");
  SB_SUPPORT(n_in % 8 == 0, "sb_gemm_mfma_bf16: inner size %d is not a multiple of 8", n_in);
  SB_SUPPORT((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) % 16 == 0,
             "sb_gemm_mfma_bf16: operands must be 16-byte aligned");
  SB_REQUIRE(!(gated && (bias || resid)), "sb_gemm_mfma_bf16: the gated form takes no bias or residual");
  if (n_rows == 0) return SB_OK;
  Args a;
  a.y = y; a.y_dtype = y_dtype; a.x = (const bf16_t *)x; a.w = (const bf16_t *)w;
  a.bias = bias; a.bias_dtype = bias_dtype; a.resid = resid;
  a.n_rows = n_rows; a.n_out = n_out; a.n_in = n_in; a.gated = gated ? 1 : 0;
  a.tiles_m = (n_rows + BM - 1) / BM;
  const int bn = gated ? BN / 2 : BN;
  a.tiles_n = (n_out + bn - 1) / bn;
  const long long blocks = (long long)a.tiles_m * a.tiles_n;
  SB_SUPPORT(blocks <= 0x7fffffffLL, "sb_gemm_mfma_bf16: too many tiles");
  hipStream_t s = (hipStream_t)stream;
  a.w_tiles = (n_out + 15) / 16;
  a.w_steps = (n_in + 31) / 32;
  if (gated && packed) gemm_mfma_kernel<1, true><<<unsigned(blocks), kThreads, 0, s>>>(a);
  else if (gated) gemm_mfma_kernel<1, false><<<unsigned(blocks), kThreads, 0, s>>>(a);
  else if (packed) gemm_mfma_kernel<0, true><<<unsigned(blocks), kThreads, 0, s>>>(a);
  else gemm_mfma_kernel<0, false><<<unsigned(blocks), kThreads, 0, s>>>(a);
  return sb::check_launch("sb_gemm_mfma_bf16");
}
