// bf16 matrix product for many rows (prefill):  Y[t,n] = sum_k X[t,k] W[n,k]
// on the matrix cores, with the model's epilogues fused: bias, float32
// residual, gate activation, float32 or bfloat16 output.
//
// A block of 2 x NW waves owns a BM x BN tile of Y (128 x 128, 256 x 128 or
// 256 x 256) and walks K in stages of BK.  Both operand tiles go
// global -> registers -> LDS, the next stage's loads being issued before the
// current stage's MFMAs (two LDS buffers, one barrier per stage).  An LDS row
// holds BK k (BK / 8 chunks of 16 bytes); chunk c of row r is stored at chunk
// c ^ f(r), f chosen so that the 16-byte fragment reads of sixteen consecutive
// rows fall on distinct banks.  A wave owns (BM / 2) x 64: MT x 2 tiles of
// v_mfma_f32_32x32x16_bf16, A = rows of X, B = rows of W, so a lane holds one
// output column of 16 rows.  The taller tile halves the LDS reads per MFMA;
// the launcher picks the shape from the problem's sizes.
//
// Block order: consecutive block numbers go to different XCDs (each with its
// own L2).  The grid is walked so that the blocks one XCD runs at a time share
// their X rows and neighbouring W rows.
#include <type_traits>

#include "mfma.h"

namespace {

constexpr int kXcds = 8;
typedef uint16_t u16x4_t __attribute__((ext_vector_type(4)));

struct Args {
  void *y;
  int y_dtype;
  const bf16_t *x, *w;
  const void *bias;
  int bias_dtype;
  const float *resid;
  int n_rows, n_out, n_in;
  int gated;       // an sb_gate; not 0: W is [2*n_out, n_in], rows n (gate) and n_out + n (up)
  int tiles_m, tiles_n;
  int w_tiles;     // packed W: 16-row tiles of one half (ceil(n_out / 16))
  int w_steps;     // packed W: 32-wide k-steps (ceil(n_in / 32))
  // K cut over the grid (blockIdx.y): slice s multiplies stages [s * stages_per_slice, ...) and
  // writes its raw sums to partial [slice][n_rows][n_out]; NULL: one slice, the epilogues below
  float *partial;
  int stages_per_slice;
  int vec4;        // n_out % 4 == 0 and y, resid, partial 16-byte aligned: four outputs of a row at a time
};

// index (in 16-byte chunks) of chunk `chunk` of LDS row `row`, CPR chunks per row
template <class T>
constexpr int const_of() {
  if constexpr (std::is_integral<T>::value) return 0;
  else return T::value;
}

template <int CPR>
__device__ __forceinline__ int swz(int row, int chunk) {
  return row * CPR + (chunk ^ ((row / (16 / CPR)) & (CPR - 1)));
}


// Which tile of Y block number `block` of the grid owns (a block that goes on to further tiles
// asks for the numbers one grid apart).  XCD-aware order: hardware sends block b to XCD b % 8.  XCD x
// gets the contiguous run of tiles [x * per, (x + 1) * per), which share rows of X and W in that
// XCD's L2; the grid is padded to a multiple of eight blocks, and the blocks past the last tile
// get false and leave at once.  The tiles are walked in bands of kBand tiles along M: inside a
// band m runs fastest, then n, and the bands follow one another.  The thirty-odd blocks that an
// XCD runs at a time then cover a patch of kBand x 4 tiles and share their rows of X and of W in
// its L2, where one column of all M tiles would read a different piece of X for every block.
__device__ __forceinline__ bool tile_of_block(const Args &a, int block, int &tm, int &tn) {
  const int n_blocks = a.tiles_m * a.tiles_n;
  const int per_xcd = (n_blocks + kXcds - 1) / kXcds;
  const int bid = (block % kXcds) * per_xcd + block / kXcds;
  if (block / kXcds >= per_xcd || bid >= n_blocks) return false;
  constexpr int kBand = 8;
  const int band = bid / (kBand * a.tiles_n), in_band = bid - band * (kBand * a.tiles_n);
  const int band_m = min(kBand, a.tiles_m - band * kBand);       // the last band may be lower
  tn = in_band / band_m;
  tm = band * kBand + (in_band - tn * band_m);
  return true;
}

// The epilogue of a block's tile.  The matrix cores leave a lane with single elements of many
// rows (32 x 32 tiles: sixteen rows of one column), which stored as they lie would be sixty-four
// 2- or 4-byte stores a lane.  The caller has ended its last stage with a barrier, so LDS is
// free: each wave turns SLAB rows at a time through a float area of its own (`fill(i, area)` puts
// rows SLAB i .. SLAB (i + 1) - 1 of the wave's tile there, row r at area + r * PITCH, with the gate
// already applied) and takes them out again four columns a lane, whole rows side by side, for 8-
// or 16-byte loads of the residual and stores of the result.  The wave's LDS operations run in
// program order, so a fence for the compiler is all the ordering it needs.
// SLABS groups of SLAB rows (32 or 16) make a wave's rows, NW: waves along N, NC: output columns
// of a wave; `lds_f`: at least (waves of the block) * SLAB * PITCH floats.
template <int SLABS, int SLAB, int NW, int NC, int PITCH, class Fill>
__device__ __forceinline__ void store_tile(const Args &a, float *lds_f, int t0, int n0, bool raw_allowed, Fill fill) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = wave / NW, wn = wave % NW;
  constexpr int kLanesPerRow = NC / 4, kRowsPerPass = 64 / kLanesPerRow, kPasses = SLAB / kRowsPerPass;
  static_assert(SLAB % kRowsPerPass == 0, "whole passes");
  float *turn = lds_f + wave * (SLAB * PITCH);
  const int r_in = lane / kLanesPerRow, c4 = (lane % kLanesPerRow) * 4;
  const int n_first = n0 + wn * NC + c4;              // first of this lane's four columns
  const bool raw = raw_allowed && a.partial;          // K slices: raw sums to the slice's plane
  float *y_f = raw ? a.partial + size_t(blockIdx.y) * a.n_rows * a.n_out : (float *)a.y;
  bf16_t *y_h = (bf16_t *)a.y;
  const bool f32_out = raw || a.y_dtype == SB_F32;
  const void *bias = raw ? nullptr : a.bias;
  const float *resid = raw ? nullptr : a.resid;
#pragma unroll
  for (int i = 0; i < SLABS; ++i) {
    fill(i, turn);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
      const int r = p * kRowsPerPass + r_in;
      const int t = t0 + wm * (SLABS * SLAB) + i * SLAB + r;
      floatx4_t v = *reinterpret_cast<const floatx4_t *>(turn + r * PITCH + c4);
      if (t >= a.n_rows || n_first >= a.n_out) continue;
      const size_t idx = size_t(t) * a.n_out + n_first;
      if (a.vec4) {
        if (bias) {
#pragma unroll
          for (int q = 0; q < 4; ++q) v[q] = v[q] + ld_dyn(bias, a.bias_dtype, n_first + q);
        }
        if (resid) {
          const floatx4_t rv = *reinterpret_cast<const floatx4_t *>(resid + idx);
#pragma unroll
          for (int q = 0; q < 4; ++q) v[q] = v[q] + rv[q];
        }
        if (f32_out) {
          *reinterpret_cast<floatx4_t *>(y_f + idx) = v;
        } else {
          u16x4_t h;
#pragma unroll
          for (int q = 0; q < 4; ++q) h[q] = f32_to_bf16(v[q]);
          *reinterpret_cast<u16x4_t *>(y_h + idx) = h;
        }
      } else {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          if (n_first + q >= a.n_out) continue;
          float u = v[q];
          if (bias) u = u + ld_dyn(bias, a.bias_dtype, n_first + q);
          if (resid) u = u + resid[idx + q];
          if (f32_out) y_f[idx + q] = u;
          else y_h[idx + q] = f32_to_bf16(u);
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
}

// The filling of the turning area from 32 x 32 tiles: acc[i][j][e] is row 8 * (e / 4) +
// 4 * (lane / 32) + e % 4, column lane % 32 of tile (i, j).  PITCH = NC + 8: rows four apart fall on
// the other half of the banks.
template <int MT, int GATED>
__device__ __forceinline__ void fill_from_32(floatx16_t (&acc)[MT][2], int i, float *turn) {
  constexpr int kPitch = (GATED ? 32 : 64) + 8;
  const int lane = threadIdx.x & 63, col = lane & 31, row_base = (lane >> 5) * 4;
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const int row = 8 * (e >> 2) + row_base + (e & 3);
    if (GATED) {
      turn[row * kPitch + col] = gate_act(acc[i][0][e], GATED) * acc[i][1][e];   // GATED: the sb_gate, fixed at compile time
    } else {
      turn[row * kPitch + col] = acc[i][0][e];
      turn[row * kPitch + 32 + col] = acc[i][1][e];
    }
  }
}

// PACKED: W comes in the packed tile layout (1 KB blocks of 16 rows x 32 k in fragment order,
// zero padded), which makes its global loads contiguous and free of bounds checks.
// MT: 32-row tiles of a wave (the block has two waves along M), NW: waves along N (64 columns
// each), DEPTH: stages the global loads run ahead of the products.
template <int MT, int NW, int BK, int DEPTH, int GATED, bool PACKED, bool EVEN_K>
__global__ void __launch_bounds__(128 * NW)
gemm_mfma_kernel(Args a) {
  constexpr int BM = 64 * MT, BN = 64 * NW, kThreads = 128 * NW;
  constexpr int CPR = BK / 8;                       // 16-byte chunks in an LDS row
  constexpr int kLoadsA = BM * CPR / kThreads;
  constexpr int kLoadsB = BN * CPR / kThreads;
  constexpr int kLoads = kLoadsA + kLoadsB;
  constexpr int kSteps32 = BK / 32;                 // packed k-steps in a stage
  constexpr int kSteps16 = BK / 16;                 // MFMA k-steps in a stage
  constexpr int kMfmas = 2 * MT;                    // MFMAs of a wave per k-step
  // 16-byte chunks travel as first-class vectors, so the staging arrays stay in registers
  extern __shared__ bf16x8_t lds[];
  bf16x8_t *lds_a0 = lds, *lds_a1 = lds + BM * CPR;
  bf16x8_t *lds_b0 = lds + 2 * BM * CPR, *lds_b1 = lds_b0 + BN * CPR;

  int tm, tn;
  if (!tile_of_block(a, int(blockIdx.x), tm, tn)) return;
  const int t0 = tm * BM;
  const int n0 = tn * (GATED ? BN / 2 : BN);

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wm = wave / NW, wn = wave % NW;

  // Global -> register staging: load i of a thread takes chunk id tid + kThreads * i of the
  // stage.  Buffer loads: a descriptor per operand in scalar registers, one 32-bit byte offset
  // per load, the stage's offset along K as the scalar offset; what lies past the operand's end
  // reads as zero, which covers the rows past the last one.  Chunks past the end of K inside a
  // row have to be zeroed by hand (EVEN_K: there are none).  Load i + 1 lands kThreads chunks
  // after load i in LDS (its rows are a multiple of 16 further on, so the swizzle term repeats).
  static_assert((kThreads / CPR) % 16 == 0, "rows per load must keep the swizzle term");
  // Byte offset of load i at stage 0.  With packed weights the loads of an operand lie a constant
  // stride apart (nothing is clamped: what lies past an operand's end is out of the descriptor's
  // range and reads as zero), so two offsets and two strides stand for all of them; kept as an
  // array they did not fit the registers beside 128 accumulators, and the one the compiler
  // spilled came back through a scratch load whose wait (the memory counter runs in order) also
  // waited for every global load just issued, once in every two stages.
  constexpr bool kLinear = PACKED && (kThreads / 64) % kSteps32 == 0 &&
                           (!GATED || (kThreads / 64 / kSteps32) % 4 == 0);   // see the loads of W below
  constexpr int kOffsets = kLinear ? 2 : kLoads;
  uint32_t off[kOffsets];
  uint32_t stride_a = 0, stride_b = 0;
  int kpos[kLoads];           // !EVEN_K: first k of the chunk within the stage (packed: of its k-step)
  int slot_a0, slot_b0;       // LDS chunk index of loads 0 of A and of B
  const size_t w_rows_total = size_t(GATED ? 2 : 1) * (PACKED ? size_t(a.w_tiles) * 16 : size_t(a.n_out));
  const size_t w_row_bytes = PACKED ? size_t(a.w_steps) * 64 : size_t(a.n_in) * 2;
  const __amdgpu_buffer_rsrc_t rsrc_x = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16_t *>(a.x), 0, uint32_t(size_t(a.n_rows) * a.n_in * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_w = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16_t *>(a.w), 0, uint32_t(w_rows_total * w_row_bytes), 0x00020000);
#pragma unroll
  for (int i = 0; i < kLoadsA; ++i) {
    const int id = tid + kThreads * i, row = id / CPR, c = id % CPR;
    if (kLinear) {
      // rows past the last one lie past the descriptor's end (the host has checked that their
      // offsets still fit 32 bits)
      if (i == 0) off[0] = uint32_t((size_t(t0 + row) * a.n_in + c * 8) * 2);
      stride_a = uint32_t(size_t(kThreads / CPR) * a.n_in * 2);
    } else {
      const int t = min(t0 + row, a.n_rows);          // n_rows: one past the end, reads zeros
      off[i] = uint32_t((size_t(t) * a.n_in + c * 8) * 2);
    }
    if (i == 0) slot_a0 = swz<CPR>(row, c);
    kpos[i] = c * 8;
  }
#pragma unroll
  for (int i = 0; i < kLoadsB; ++i) {
    const int id = tid + kThreads * i;
    if (PACKED) {
      // load id -> 1 KB block (id / 64) = (row tile of the LDS tile, k-step), lane id % 64
      const int blk = id >> 6, l = id & 63;
      const int rt = blk / kSteps32, j = blk % kSteps32;   // LDS rows rt * 16 .., k-step j of the stage
      if constexpr (kLinear) {
        // load i + 1 takes the block kThreads / 64 further on: the same k-step, row tile
        // rt + kThreads / 64 / kSteps32, which is a constant number of tiles of W further on
        if (i == 0) {
          int tile;
          if (GATED) {
            const int half = rt >> 2, within = rt & 3;
            tile = (within >> 1) * a.w_tiles + n0 / 16 + half * 2 + (within & 1);
          } else {
            tile = n0 / 16 + rt;
          }
          // a tile past the last: past the half's (or the matrix's) end; its columns are not stored
          off[1] = uint32_t(((size_t(tile) * a.w_steps + j) * 512 + size_t(l) * 8) * 2);
          constexpr int kTilesApart = GATED ? (kThreads / 64 / kSteps32) / 2 : kThreads / 64 / kSteps32;
          stride_b = uint32_t(size_t(kTilesApart) * a.w_steps * 1024);
        }
      } else {
        int tile;
        if (GATED) {
          const int half = rt >> 2, within = rt & 3;
          tile = (within >> 1) * a.w_tiles + min(n0 / 16 + half * 2 + (within & 1), a.w_tiles - 1);
        } else {
          tile = min(n0 / 16 + rt, a.w_tiles - 1);
        }
        off[kLoadsA + i] = uint32_t(((size_t(tile) * a.w_steps + j) * 512 + size_t(l) * 8) * 2);
      }
      if (i == 0) slot_b0 = swz<CPR>(rt * 16 + (l & 15), j * 4 + (l >> 4));
      kpos[kLoadsA + i] = j * 32;
    } else {
      const int row = id / CPR, c = id % CPR;
      int wrow;       // the row of W that feeds LDS row `row`
      if (GATED) {
        // LDS rows [0,32) gate of features n0..n0+31, [32,64) up of the same, [64,96) gate of
        // n0+32.., [96,128) up of the same: a wave's two B tiles are gate and up of 32 features.
        const int half = row >> 6, within = row & 63, is_up = within >> 5;
        wrow = is_up * a.n_out + min(n0 + half * 32 + (within & 31), a.n_out - 1);
      } else {
        wrow = min(n0 + row, a.n_out - 1);
      }
      off[kLoadsA + i] = uint32_t((size_t(wrow) * a.n_in + c * 8) * 2);
      if (i == 0) slot_b0 = swz<CPR>(row, c);
      kpos[kLoadsA + i] = c * 8;
    }
  }

  floatx16_t acc[MT][2];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // DEPTH 2, two register sets: while stage kt is multiplied out of LDS, stage kt + 1 waits in
  // one set (its loads went out a stage earlier) and the loads of stage kt + 2 go out into the
  // other.  DEPTH 1, one set: the loads of stage kt + 1 go out in the first half of stage kt.
  const int n_k_all = (a.n_in + BK - 1) / BK;
  const int kt_begin = a.partial ? int(blockIdx.y) * a.stages_per_slice : 0;
  const int n_k = a.partial ? min(kt_begin + a.stages_per_slice, n_k_all) : n_k_all;   // end of this slice
  constexpr uint32_t kPastEnd = 0xfff00000u;      // the host keeps every operand below this size
  bf16x8_t staged[DEPTH][kLoads];
  auto issue_load = [&](auto SET, int i, int kt) {
    constexpr int set = decltype(SET)::value;
    const bool is_a = i < kLoadsA;
    // uniform part of the address: the stage's offset along K
    int stage_off = (PACKED && !is_a) ? kt * (kSteps32 * 1024) : kt * (BK * 2);
    uint32_t offset;
    if constexpr (kLinear) offset = is_a ? off[0] + uint32_t(i) * stride_a : off[1] + uint32_t(i - kLoadsA) * stride_b;
    else offset = off[i];
    // a stage past the end of K (of this slice): an offset past every operand, which reads as zeros
    // (with no scalar offset on top, so that the sum cannot wrap around into the operand)
    if (DEPTH == 2 && kt >= n_k) { offset |= kPastEnd; stage_off = 0; }
    bf16x8_t v = __builtin_bit_cast(
        bf16x8_t, __builtin_amdgcn_raw_buffer_load_b128(is_a ? rsrc_x : rsrc_w, int(offset), stage_off, 0));
    if (!EVEN_K) {
      const bool ok = (PACKED && !is_a) ? (kt * BK + kpos[i] < a.w_steps * 32) : (kt * BK + kpos[i] < a.n_in);
      if (!ok) v = bf16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
    }
    staged[set][i] = v;
  };
  auto store_lds = [&](auto SET, int i, int buf) {
    constexpr int set = decltype(SET)::value;
    if (i < kLoadsA) (buf ? lds_a1 : lds_a0)[slot_a0 + i * kThreads] = staged[set][i];
    else (buf ? lds_b1 : lds_b0)[slot_b0 + (i - kLoadsA) * kThreads] = staged[set][i];
  };

  using Set0 = std::integral_constant<int, 0>;
  using Set1 = std::integral_constant<int, 1>;
#pragma unroll
  for (int i = 0; i < kLoads; ++i) issue_load(Set0{}, i, kt_begin);
  if (DEPTH == 2) {
#pragma unroll
    for (int i = 0; i < kLoads; ++i) issue_load(std::integral_constant<int, DEPTH - 1>{}, i, kt_begin + 1);
  }
#pragma unroll
  for (int i = 0; i < kLoads; ++i) store_lds(Set0{}, i, 0);
  __syncthreads();

  // fragment reads: lane -> row lane % 32 of a 32-row tile, chunk 2 * ks + lane / 32 of the stage
  const int frag_row = lane & 31, frag_c = lane >> 5;
  const int frag_sw = (frag_row / (16 / CPR)) & (CPR - 1);     // swizzle term, equal for all tiles of a wave
  const int a_row0 = (wm * (32 * MT) + frag_row) * CPR, b_row0 = (wn * 64 + frag_row) * CPR;

  // One stage.  CUR: LDS buffer of this stage (and with two register sets the free one); LOAD: the
  // stage to load (kt + DEPTH) exists, STORE: stage kt + 1 exists.  The memory operations are spread between the MFMAs in the source
  // so that the matrix pipe keeps running while they issue.
  auto stage = [&](auto CUR, auto LOAD, auto STORE, int kt) {
    // CUR: a constant with two register sets (it names the set too); with one set it may be a
    // plain int, and then one copy of the stage serves both LDS buffers
    constexpr bool kFixed = !std::is_integral<decltype(CUR)>::value;
    const int cur = int(CUR);
    constexpr bool do_load = decltype(LOAD)::value, do_store = decltype(STORE)::value;
    using SetCur = std::integral_constant<int, DEPTH == 2 ? const_of<decltype(CUR)>() : 0>;          // set to load into
    using SetNext = std::integral_constant<int, DEPTH == 2 ? (const_of<decltype(CUR)>() ^ 1) : 0>;   // set to store from
    static_assert(kFixed || DEPTH == 1, "two register sets need the buffer as a constant");
    const bf16x8_t *la = cur ? lds_a1 : lds_a0, *lb = cur ? lds_b1 : lds_b0;
    bf16x8_t frag[2][MT + 2];
    auto read_frag = [&](int fs, int ks, int f) {
      const int c = (ks * 2 + frag_c) ^ frag_sw;
      frag[fs][f] = f < MT ? la[a_row0 + f * 32 * CPR + c] : lb[b_row0 + (f - MT) * 32 * CPR + c];
    };
#pragma unroll
    for (int f = 0; f < MT + 2; ++f) read_frag(0, 0, f);
    constexpr int kSlots = kSteps16 * kMfmas;           // MFMAs of the stage = places to put other work
    constexpr int kHalf = kSlots / 2;
#pragma unroll
    for (int ks = 0; ks < kSteps16; ++ks) {
#pragma unroll
      for (int m = 0; m < kMfmas; ++m) {
        const int i = m >> 1, j = m & 1, at = ks * kMfmas + m;
        acc[i][j] = mfma32(frag[ks & 1][i], frag[ks & 1][MT + j], acc[i][j]);
        // fragments of the next k-step, one read after each of the first MFMAs
        if (ks + 1 < kSteps16 && m < MT + 2) read_frag((ks + 1) & 1, ks + 1, m);
        // loads of stage kt + DEPTH over the first half of the stage
        if (do_load && at < kHalf) {
#pragma unroll
          for (int l = 0; l < kLoads; ++l)
            if (l >= at * kLoads / kHalf && l < (at + 1) * kLoads / kHalf)
              issue_load(SetCur{}, l, DEPTH == 1 ? min(kt + 1, n_k - 1) : kt + DEPTH);
        }
        // stage kt + 1 into the other LDS buffer over the second half: nobody reads that buffer
        // since the last barrier
        if (do_store && at >= kHalf) {
#pragma unroll
          for (int l = 0; l < kLoads; ++l)
            if (l >= (at - kHalf) * kLoads / kHalf && l < (at - kHalf + 1) * kLoads / kHalf)
              store_lds(SetNext{}, l, cur ^ 1);
        }
        // keep this order: left alone, the scheduler gathers the memory operations into lumps
        // and reads each fragment right before its MFMA, and the matrix pipe waits on both
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __syncthreads();
  };
  using Yes = std::true_type;
  using No = std::false_type;
  int kt = kt_begin;
  if constexpr (DEPTH == 2) {
    // Pairs of stages, one for each register set, and nothing peeled off at the end: with an odd
    // count the last pair's second stage multiplies zeros (its loads were aimed past the end).
    for (; kt < n_k; kt += 2) {
      stage(Set0{}, Yes{}, Yes{}, kt);
      stage(Set1{}, Yes{}, Yes{}, kt + 1);
    }
  } else {
    // One copy of the stage for every k, the LDS buffer as a variable: the accumulators stay in
    // their registers up to the epilogue (the peeled last stages made the compiler move them
    // through scratch memory).  The last stage loads itself once more instead of a stage past
    // the end, into the buffer that nobody reads.
    for (; kt < n_k; ++kt) stage((kt - kt_begin) & 1, Yes{}, Yes{}, kt);
  }

  static_assert(2 * (BM + BN) * CPR * 16 >= (kThreads / 64) * 32 * ((GATED ? 32 : 64) + 8) * 4,
                "the turning areas of the epilogue must fit the stage buffers");
  store_tile<MT, 32, NW, (GATED ? 32 : 64), (GATED ? 32 : 64) + 8>(
      a, reinterpret_cast<float *>(lds), t0, n0, !GATED,
      [&](int i, float *turn) { fill_from_32<MT, GATED>(acc, i, turn); });
}

// ---------------------------------------------------------------------------------------------
// The same product with the operand tiles loaded from global memory straight into LDS
// (buffer_load ... lds: the 64 lanes of a wave fill 1 KB of LDS in lane order, 16 bytes each),
// for packed weights and an inner size that is a multiple of BK.  No registers hold a stage on
// its way, so the loads run NBUF - 1 whole stages ahead of the products (the register path has
// half a stage), and the LDS stores are gone.  X keeps the row-major swizzled layout of the
// register path in LDS: a lane's place in LDS is fixed by its number, so the swizzle goes into
// the source address instead: the lane that fills chunk place c' of row r loads chunk c' ^ f(r)
// of that row.  W is copied block by block as the packed layout has it (lanes that follow one
// another read memory that follows one another; aimed at swizzled rows instead, the four lanes
// that the address unit takes at a time fell on four cache lines, and the kernel was slower than
// the register path).
//
// It multiplies with v_mfma_f32_16x16x32_bf16.  With real data the chip runs at the clock its
// power allows, and for the same count of flops this instruction lets it run faster than
// 32 x 32 x 16 (measured: 2.13 against 1.88 PFLOP/s on registers alone, 2.49 with zeros).  The
// operand traffic is the same: a wave owns (16 * MT16) x 64 outputs as MT16 x 4 tiles and reads
// MT16 + 4 fragments for every 32 k.  W's 1 KB blocks are fragments of this instruction as they
// lie (lane 16 g + r: row r, k = 8 g ..), so a B fragment is one linear read of a block, free of
// bank conflicts without a swizzle.  Fragments: B for a whole k-step in two sets of registers, A
// in a ring of four tiles that runs two tiles ahead of the MFMAs.
//
// PERSIST: the grid is one round of blocks, and a block goes on to the tile one grid further
// until the tiles end.  The last stage of a tile then loads the first stage of the next tile (not
// itself once more), so the next tile's loop starts right after the epilogue with its operands in
// LDS, the epilogue's stores drain behind the next tile's products instead of holding the CU
// until the block has left, and no block has to be started for a tile.
template <int MT16, int NW, int BK, int NBUF, int GATED, bool PERSIST>
__global__ void __launch_bounds__(128 * NW)
gemm_direct16_kernel(Args a) {
  constexpr int BM = 32 * MT16, BN = 64 * NW, kThreads = 128 * NW, kWaves = kThreads / 64;
  constexpr int CPR = BK / 8;                       // 16-byte chunks in an LDS row of A
  constexpr int kRowsPerLoad = 64 / CPR;            // rows of A that one load of a wave (1 KB) fills
  constexpr int kSteps32 = BK / 32;
  constexpr int kLoadsA = BM / kRowsPerLoad / kWaves, kLoadsB = BN / 16 * kSteps32 / kWaves;
  constexpr int kLoads = kLoadsA + kLoadsB;
  constexpr int kBufChunks = (BM + BN) * CPR;       // 16-byte chunks of a stage buffer: A, then B
  constexpr int kTiles = kSteps32 * MT16;           // A tiles of a stage, in the order they are used
  static_assert((NBUF & (NBUF - 1)) == 0 && NBUF >= 2, "the buffers are counted modulo a power of two");
  static_assert(!PERSIST || NBUF == 2, "going on to the next tile is written for two buffers");
  static_assert(BM % (kRowsPerLoad * kWaves) == 0 && (BN / 16 * kSteps32) % kWaves == 0, "whole loads");
  static_assert((NBUF - 2) * kLoads < 64, "the memory counter has six bits");
  static_assert(CPR == 8 || CPR == 4, "stages of 64 or 32 k");
  static_assert(kTiles * 2 >= kLoads, "two loads go out with each A tile");
  extern __shared__ bf16x8_t lds[];
  typedef __attribute__((address_space(3))) bf16x8_t *lds_ptr_t;

  int vblock = blockIdx.x, tm, tn;
  if (!tile_of_block(a, vblock, tm, tn)) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / NW, wn = wave % NW;

  const size_t w_rows_total = size_t(GATED ? 2 : 1) * size_t(a.w_tiles) * 16;
  const __amdgpu_buffer_rsrc_t rsrc_x = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16_t *>(a.x), 0, uint32_t(size_t(a.n_rows) * a.n_in * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_w = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16_t *>(a.w), 0, uint32_t(w_rows_total * size_t(a.w_steps) * 64), 0x00020000);
  // Byte offset of each load's source at stage 0 of tile (m, n) (the stage's offset along K is
  // added as the scalar offset).  Rows and row tiles past an operand's end are past its
  // descriptor's range and read as zeros; the host has checked that their offsets fit 32 bits.
  // W's row tiles in LDS: [0,2) gate of features n0.., [2,4) up of the same, [4,6) gate of n0 + 32..,
  // and so on: a wave's four B tiles are gate and up of 32 features.
  uint32_t off[kLoads];
  auto aim_at = [&](int m, int n) {
    const int t0 = m * BM, n0 = n * (GATED ? BN / 2 : BN);
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      if (i < kLoadsA) {
        const int place = (i * kWaves + wave) * 64 + lane;
        const int row = place / CPR;
        const int c = (place % CPR) ^ ((row / (16 / CPR)) & (CPR - 1));
        off[i] = uint32_t((size_t(t0 + row) * a.n_in + c * 8) * 2);
      } else {
        const int blk = (i - kLoadsA) * kWaves + wave, rt = blk / kSteps32, j = blk % kSteps32;
        const int tile = GATED ? ((rt & 3) >> 1) * a.w_tiles + n0 / 16 + (rt >> 2) * 2 + (rt & 1) : n0 / 16 + rt;
        off[i] = uint32_t(((size_t(tile) * a.w_steps + j) * 512 + size_t(lane) * 8) * 2);
      }
    }
  };
  auto issue_load = [&](int i, int kt, int buf) {
    const bool is_a = i < kLoadsA;
    const int stage_off = is_a ? kt * (BK * 2) : kt * (kSteps32 * 1024);
    const int chunk = buf * kBufChunks + (is_a ? (i * kWaves + wave) * 64 : BM * CPR + ((i - kLoadsA) * kWaves + wave) * 64);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(is_a ? rsrc_x : rsrc_w, (lds_ptr_t)(lds) + chunk, 16, int(off[i]),
                                             stage_off, 0, 0);
  };
  // The next stage's tiles: this wave's share has landed (the loads of the NBUF - 2 stages after
  // it may still be on their way), and after the barrier everybody's.  A bare barrier between
  // two fences for the compiler: __syncthreads() carries a release fence, which for loads into
  // LDS means waiting for all of them.
  auto wait_and_meet = [&]() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NBUF - 2) * kLoads) : "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };

  const int n_k_all = a.n_in / BK;
  const int kt_begin = a.partial ? int(blockIdx.y) * a.stages_per_slice : 0;
  const int n_k = a.partial ? min(kt_begin + a.stages_per_slice, n_k_all) : n_k_all;   // end of this slice
  // A stage past the end (of the last tile, when the block goes on) is the last stage once more,
  // into a buffer that nobody reads again: the count of loads in flight stays the same in every
  // stage, which the waits rely on.
  aim_at(tm, tn);
#pragma unroll
  for (int s = 0; s < NBUF - 1; ++s)
#pragma unroll
    for (int i = 0; i < kLoads; ++i) issue_load(i, min(kt_begin + s, n_k - 1), s);
  wait_and_meet();

  // A fragment of tile i, k-step j: lane 16 g + r reads row 16 i + r, chunk 4 j + g of the stage,
  // swizzled by the row (the term depends on r alone).  B fragment of tile f, k-step j: block
  // (4 wn + f, j), lane by lane.
  const int fr = lane & 15, fg = lane >> 4;
  const int frag_sw = (fr / (16 / CPR)) & (CPR - 1);
  int a_lane[kSteps32];
#pragma unroll
  for (int j = 0; j < kSteps32; ++j) a_lane[j] = (wm * (16 * MT16) + fr) * CPR + ((4 * j + fg) ^ frag_sw);
  const int b_lane = BM * CPR + (wn * 4 * kSteps32) * 64 + lane;

  floatx4_t acc[MT16][4];
  // One stage: buffer `buf` is multiplied, the loads of stage kt_load go out (two with each of the
  // first A tiles) into buffer buf_load, which the stage before has read.
  auto stage = [&](int buf, int kt_load, int buf_load) {
    const bf16x8_t *ls = lds + buf * kBufChunks;
    bf16x8_t fa[4], fb[2][4];
    auto read_a = [&](int tile) {       // tile = j * MT16 + i, in the order of use
      const int j = tile / MT16, i = tile % MT16;
      fa[tile & 3] = ls[a_lane[j] + i * 16 * CPR];
    };
    auto read_b = [&](int j, int f) { fb[j & 1][f] = ls[b_lane + (f * kSteps32 + j) * 64]; };
#pragma unroll
    for (int f = 0; f < 4; ++f) read_b(0, f);
    read_a(0);
    read_a(1);
#pragma unroll
    for (int tile = 0; tile < kTiles; ++tile) {
      const int j = tile / MT16, i = tile % MT16;
#pragma unroll
      for (int f = 0; f < 4; ++f) {
        acc[i][f] = mfma16(fa[tile & 3], fb[j & 1][f], acc[i][f]);
        if (f == 0 && tile + 2 < kTiles) read_a(tile + 2);
        // the next k-step's B fragments, one with each of the first A tiles of this one
        if (f == 1 && i < 4 && j + 1 < kSteps32) read_b(j + 1, i);
        if (f >= 2 && tile * 2 + (f - 2) < kLoads) issue_load(tile * 2 + (f - 2), kt_load, buf_load);
        // keep this order: left alone, the scheduler gathers the memory operations into lumps
        // and reads each fragment right before its MFMA, and the matrix pipe waits on both
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    wait_and_meet();
  };

  // Epilogue.  acc[i][f][e]: row 4 * (lane / 16) + e, column lane % 16 of tile (i, f); gated: tiles
  // 0, 1 are the gate and 2, 3 the up projection of the same 32 features.  PITCH = NC + 4: the
  // four row groups of a store fall on four different quarters of the banks.
  constexpr int NC = GATED ? 32 : 64, kPitch = NC + 4;
  static_assert((NBUF == 2 ? 1 : NBUF) * kBufChunks * 16 >= kWaves * 16 * kPitch * 4,
                "the turning areas must fit a stage buffer (two buffers: the other one may hold the next tile)");
  auto epilogue = [&](int m, int n, int buf_free) {
    store_tile<MT16, 16, NW, NC, kPitch>(
        a, reinterpret_cast<float *>(lds + buf_free * kBufChunks), m * BM, n * (GATED ? BN / 2 : BN), !GATED,
        [&](int i, float *turn) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int row = 4 * fg + e;
            if (GATED) {
#pragma unroll
              for (int f = 0; f < 2; ++f)
                turn[row * kPitch + f * 16 + fr] = gate_act(acc[i][f][e], GATED) * acc[i][f + 2][e];
            } else {
#pragma unroll
              for (int f = 0; f < 4; ++f) turn[row * kPitch + f * 16 + fr] = acc[i][f][e];
            }
          }
        });
  };

  int buf = 0;
  for (;;) {
#pragma unroll
    for (int i = 0; i < MT16; ++i)
#pragma unroll
      for (int f = 0; f < 4; ++f) acc[i][f] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    int tm_next = 0, tn_next = 0;
    const bool more = PERSIST && tile_of_block(a, vblock + int(gridDim.x), tm_next, tn_next);
    for (int kt = kt_begin; kt < n_k; ++kt) {
      int kt_load = kt + NBUF - 1;
      if (kt_load >= n_k) {
        if (PERSIST && more) {
          // (two buffers: this is the tile's last stage) from here on the loads are the next tile's
          aim_at(tm_next, tn_next);
          kt_load = kt_begin;
        } else {
          kt_load = n_k - 1;
        }
      }
      stage(buf, kt_load, (buf + NBUF - 1) & (NBUF - 1));
      buf = (buf + 1) & (NBUF - 1);
    }
    if (NBUF > 2) {
      // the last stages' loads (of the last stage again) are still writing LDS
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
    }
    // two buffers: `buf` holds the next tile's first stage (or the last stage once more), the
    // other one is free for the epilogue
    epilogue(tm, tn, NBUF == 2 ? (buf ^ 1) : 0);
    if (!PERSIST || !more) break;
    // the next stage's loads go into the buffer that the epilogue has turned its rows through
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    vblock += int(gridDim.x);
    tm = tm_next;
    tn = tn_next;
  }
}


template <int MT, int NW, int BK, int DEPTH, int GATED, bool PACKED, bool EVEN_K>
int launch_one(const Args &a, long long blocks, hipStream_t s) {
  constexpr int lds_bytes = 2 * (64 * MT + 64 * NW) * (BK / 8) * 16;
  static bool raised = false;     // per instantiation; harmless if repeated
  if (lds_bytes > 48 * 1024 && !raised) {
    const hipError_t e =
        hipFuncSetAttribute((const void *)gemm_mfma_kernel<MT, NW, BK, DEPTH, GATED, PACKED, EVEN_K>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    SB_REQUIRE(e == hipSuccess, "sb_gemm_mfma_bf16: cannot reserve %d bytes of LDS: %s", lds_bytes,
               hipGetErrorString(e));
    raised = true;
  }
  const int n_k = (a.n_in + BK - 1) / BK;
  const unsigned slices = a.partial ? unsigned((n_k + a.stages_per_slice - 1) / a.stages_per_slice) : 1u;
  gemm_mfma_kernel<MT, NW, BK, DEPTH, GATED, PACKED, EVEN_K>
      <<<dim3(unsigned((blocks + kXcds - 1) / kXcds * kXcds), slices), 128 * NW, lds_bytes, s>>>(a);
  return SB_OK;
}

template <int MT, int NW, int BK, int DEPTH, bool PLAIN_TOO>
int launch(const Args &a, long long blocks, int packed, hipStream_t s) {
  // the gate's activation is a template argument: the SiLU kernels hold no code of the others
  const int which = a.gated * 4 + (packed ? 2 : 0) + (a.n_in % BK == 0 ? 1 : 0);
  switch (which) {
    case 11: return launch_one<MT, NW, BK, DEPTH, 2, true, true>(a, blocks, s);
    case 10: return launch_one<MT, NW, BK, DEPTH, 2, true, false>(a, blocks, s);
    case 7: return launch_one<MT, NW, BK, DEPTH, 1, true, true>(a, blocks, s);
    case 6: return launch_one<MT, NW, BK, DEPTH, 1, true, false>(a, blocks, s);
    case 3: return launch_one<MT, NW, BK, DEPTH, 0, true, true>(a, blocks, s);
    case 2: return launch_one<MT, NW, BK, DEPTH, 0, true, false>(a, blocks, s);
    default: break;
  }
  if constexpr (PLAIN_TOO) {
    switch (which) {
      case 9: return launch_one<MT, NW, BK, DEPTH, 2, false, true>(a, blocks, s);
      case 8: return launch_one<MT, NW, BK, DEPTH, 2, false, false>(a, blocks, s);
      case 5: return launch_one<MT, NW, BK, DEPTH, 1, false, true>(a, blocks, s);
      case 4: return launch_one<MT, NW, BK, DEPTH, 1, false, false>(a, blocks, s);
      case 1: return launch_one<MT, NW, BK, DEPTH, 0, false, true>(a, blocks, s);
      default: return launch_one<MT, NW, BK, DEPTH, 0, false, false>(a, blocks, s);
    }
  }
  return sb::fail(SB_ERR_UNSUPPORTED, "sb_gemm_mfma_bf16: this tile shape takes packed weights only");
}

// PERSIST: one round of blocks (`round_blocks`: what the GPU runs at a time), each going from
// tile to tile
template <int MT16, int NW, int BK, int NBUF, int GATED, bool PERSIST>
int launch_direct_one(const Args &a, long long blocks, int round_blocks, hipStream_t s) {
  constexpr int lds_bytes = NBUF * (32 * MT16 + 64 * NW) * (BK / 8) * 16;
  static bool raised = false;     // per instantiation; harmless if repeated
  if (lds_bytes > 48 * 1024 && !raised) {
    const hipError_t e = hipFuncSetAttribute((const void *)gemm_direct16_kernel<MT16, NW, BK, NBUF, GATED, PERSIST>,
                                             hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    SB_REQUIRE(e == hipSuccess, "sb_gemm_mfma_bf16: cannot reserve %d bytes of LDS: %s", lds_bytes,
               hipGetErrorString(e));
    raised = true;
  }
  const int n_k = a.n_in / BK;
  const unsigned slices = a.partial ? unsigned((n_k + a.stages_per_slice - 1) / a.stages_per_slice) : 1u;
  long long grid = (blocks + kXcds - 1) / kXcds * kXcds;
  if (PERSIST && grid > round_blocks) grid = round_blocks;
  gemm_direct16_kernel<MT16, NW, BK, NBUF, GATED, PERSIST><<<dim3(unsigned(grid), slices), 128 * NW, lds_bytes, s>>>(a);
  return SB_OK;
}

// packed weights, n_in a multiple of BK
template <int MT16, int NW, int BK, int NBUF, bool PERSIST>
int launch_direct(const Args &a, long long blocks, int round_blocks, hipStream_t s) {
  switch (a.gated) {
    case 2: return launch_direct_one<MT16, NW, BK, NBUF, 2, PERSIST>(a, blocks, round_blocks, s);
    case 1: return launch_direct_one<MT16, NW, BK, NBUF, 1, PERSIST>(a, blocks, round_blocks, s);
    default: return launch_direct_one<MT16, NW, BK, NBUF, 0, PERSIST>(a, blocks, round_blocks, s);
  }
}

// Tile shapes the launcher chooses from: rows x columns of Y per block.
struct Shape { int bm, bn; };
constexpr Shape kShapes[5] = {{128, 128}, {256, 128}, {256, 256}, {128, 256}, {192, 256}};

// The tile shape for a problem: the one with the best product of three factors.  How fast the
// shape's kernel runs on a full grid, relative to 128 x 128 (measured on MI355X at 2,048 to 16,384
// rows of Qwen2.5-7B's four products: the 256 x 256 kernel, which loads straight into LDS, reaches
// 1.19 to 1.31 PFLOP/s where the 128 x 128 one reaches 0.73 to 0.98; the same kernel with tiles of
// 192 rows takes 0.84 of the time for 0.75 of the outputs); the share of the tiles' rows
// that are rows of Y; and the share of the last round of tiles over the CUs that is filled.
// Some of what this decides at 2,048 rows: the output product (3,584 x 3,584) takes 256 x 128
// (224 tiles, one round: 65 us against 92 with 112 tiles of 256 x 256), the QKV product 192 x 256
// (198 tiles: 63 us against 73 with 144 of 256 x 256), the down product 256 x 128 (274 against 403 us);
// from 4,096 rows on nearly everything takes 256 x 256.  `direct_ok`: the kernel that loads
// straight into LDS takes these operands (the 192 x 256 shape has no other).
int pick_shape(int n_rows, int n_out, int n_in, int gated, bool direct_ok, double *score_out = nullptr) {
  (void)n_in;
  const double speed[5] = {1.0, gated ? 1.0 : 1.05, gated ? 1.25 : 1.35, 0.0, (gated ? 1.25 : 1.35) * 0.89};
  double best = 0;
  int pick = 0;
  for (int v = 0; v < 5; ++v) {
    if (v == 3 || (v == 4 && !direct_ok)) continue;
    const int bm = kShapes[v].bm, bn = gated ? kShapes[v].bn / 2 : kShapes[v].bn;
    const long long tiles_m = (n_rows + bm - 1) / bm, tiles_n = (n_out + bn - 1) / bn;
    const long long tiles = tiles_m * tiles_n, rounds = (tiles + sb::cu_count() - 1) / sb::cu_count();
    const double score = speed[v] * (double(n_rows) / double(tiles_m * bm)) * (double(tiles) / double(rounds * sb::cu_count()));
    if (score > best) { best = score; pick = v; }
  }
  if (score_out) *score_out = best;
  return pick;
}

}  // namespace

// Y = X W^T (+bias) (+resid), or gated: Y = silu(X Wg^T) * (X Wu^T), W = [Wg; Wu].
// X [n_rows, n_in] and W bf16, n_in a multiple of 8, operands 16-byte aligned; packed != 0: W is
// in the packed tile layout.
extern "C" int sb_gemm_mfma_bf16(void *y, int y_dtype, const void *x, const void *w, const void *bias,
                                 int bias_dtype, const float *resid, int n_rows, int n_out, int n_in,
                                 int gated, int packed, int tile_shape, void *stream) {
  SB_REQUIRE(y && x && w, "sb_gemm_mfma_bf16: null pointer");
  SB_REQUIRE(n_rows >= 0 && n_out > 0 && n_in > 0, "sb_gemm_mfma_bf16: bad sizes rows=%d out=%d in=%d",
             n_rows, n_out, n_in);
  SB_REQUIRE(sb::valid_dtype(y_dtype) && (!bias || sb::valid_dtype(bias_dtype)),
             "sb_gemm_mfma_bf16: unknown dtype");
  SB_SUPPORT(n_in % 8 == 0, "sb_gemm_mfma_bf16: inner size %d is not a multiple of 8", n_in);
  SB_SUPPORT((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) % 16 == 0,
             "sb_gemm_mfma_bf16: operands must be 16-byte aligned");
  SB_REQUIRE(!(gated && (bias || resid)), "sb_gemm_mfma_bf16: the gated form takes no bias or residual");
  SB_SUPPORT(gated >= SB_GATE_NONE && gated <= SB_GATE_GELU_TANH, "sb_gemm_mfma_bf16: unknown gate activation %d", gated);
  if (n_rows == 0) return SB_OK;
  Args a;
  a.y = y; a.y_dtype = y_dtype; a.x = (const bf16_t *)x; a.w = (const bf16_t *)w;
  a.bias = bias; a.bias_dtype = bias_dtype; a.resid = resid;
  a.n_rows = n_rows; a.n_out = n_out; a.n_in = n_in; a.gated = gated;
  a.partial = nullptr; a.stages_per_slice = 0;
  a.vec4 = n_out % 4 == 0 && (reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(resid)) % 16 == 0;
  const bool direct_ok = packed && n_in % 64 == 0;
  int variant = pick_shape(n_rows, n_out, n_in, a.gated, direct_ok);
  // a test's or a measurement's choice: the shape (0..3) + 16 * the path (0: the launcher's, 1:
  // through registers, 2: straight into LDS)
  int path = 0;
  if (tile_shape >= 0) {
    SB_REQUIRE((tile_shape & 15) < 5 && (tile_shape >> 4) < 4, "sb_gemm_mfma_bf16: unknown tile shape %d", tile_shape);
    variant = tile_shape & 15;
    path = tile_shape >> 4;
  }
  if (!packed) variant = 0;       // the bigger tiles are built for packed weights only
  const int bm = kShapes[variant].bm, bn = gated ? kShapes[variant].bn / 2 : kShapes[variant].bn;
  a.tiles_m = (n_rows + bm - 1) / bm;
  a.tiles_n = (n_out + bn - 1) / bn;
  const long long blocks = (long long)a.tiles_m * a.tiles_n;
  SB_SUPPORT(blocks <= 0x7fffffffLL, "sb_gemm_mfma_bf16: too many tiles");
  // the kernel addresses both operands with 32-bit byte offsets
  const unsigned long long w_rows = (unsigned long long)((n_out + 15) / 16 * 16) * (gated ? 2 : 1);
  const unsigned long long k_padded = (unsigned long long)((n_in + 31) / 32 * 32);
  // ... also for the rows and row tiles past an operand's end that a block at the edge asks for
  // (they lie past the descriptor's end and read as zero, but must not wrap around)
  SB_SUPPORT(((unsigned long long)n_rows + 257) * n_in * 2 < (1ull << 32) - (1ull << 20) &&
                 (w_rows + 512) * k_padded * 2 < (1ull << 32) - (1ull << 20),
             "sb_gemm_mfma_bf16: an operand of 4 GiB or more (rows=%d out=%d in=%d)", n_rows, n_out, n_in);
  hipStream_t s = (hipStream_t)stream;
  a.w_tiles = (n_out + 15) / 16;
  a.w_steps = (n_in + 31) / 32;
  int rc;
  SB_SUPPORT(path < 2 || direct_ok, "sb_gemm_mfma_bf16: the direct path takes packed weights and an inner size in 64s");
  // left to itself only the 256 x 256 shape goes straight into LDS: the smaller tiles' stages are too
  // short for loads that run one stage ahead, and the register path, which runs two ahead, is
  // faster there (128 x 128, QKV product at 2,048 rows: 92 against 128 us)
  const bool direct = path >= 2 || (path == 0 && direct_ok && (variant == 2 || variant == 4));
  SB_SUPPORT(variant < 3 || direct, "sb_gemm_mfma_bf16: the shapes 128 x 256 and 192 x 256 exist on the direct path only");
  if (direct) {
    // path 3 (a measurement's): the 256 x 256 shape with a block for every tile
    if (variant == 0) rc = launch_direct<4, 2, 64, 2, false>(a, blocks, 0, s);
    else if (variant == 1) rc = launch_direct<8, 2, 64, 2, false>(a, blocks, 0, s);
    else if (variant == 2 && path == 3) rc = launch_direct<8, 4, 64, 2, false>(a, blocks, 0, s);
    else if (variant == 2) rc = launch_direct<8, 4, 64, 2, true>(a, blocks, sb::cu_count(), s);     // 128 KB of LDS: a block a CU
    else if (variant == 3) rc = launch_direct<4, 4, 64, 2, false>(a, blocks, 0, s);
    else rc = launch_direct<6, 4, 64, 2, true>(a, blocks, sb::cu_count(), s);
  } else {
    if (variant == 0) rc = launch<2, 2, 64, 2, true>(a, blocks, packed, s);
    else if (variant == 1) rc = launch<4, 2, 64, 2, false>(a, blocks, packed, s);
    else rc = launch<4, 4, 64, 1, false>(a, blocks, packed, s);
  }
  if (rc != SB_OK) return rc;
  return sb::check_launch("sb_gemm_mfma_bf16");
}

namespace {
// K slices of the partial form, and the tiles that multiply them.  Few rows: enough blocks for
// the GPU (one 128 x 128 tile per CU and slice), every slice at least four stages of 64 long, at
// most the eight that the consumers add.  Where that gives one slice, a problem with few tiles
// of 256 x 256 (a prompt of one or two thousand rows against a matrix a few thousand wide) may
// still be faster with those tiles, loaded straight into LDS, and K cut so that the tiles and
// slices together make one round over the CUs.  Both ways are priced in microseconds from
// what was measured on MI355X with the 7B products at 768 to 2,304 rows: a shape's tile takes
// 2 bm bn K flops at its kernel's rate on a full GPU (pick_shape's speeds, 1 standing for 0.93
// PFLOP/s over 256 CUs); a round that leaves CUs idle runs faster (0.72 of the time with up to 170
// blocks, rising to 1 at 256: the chip's clock follows its load); either kernel costs 14 us
// beside its tiles; the consumer's pass over the additional slices moves (2 slices - 2) x the
// result's bytes at 4 TB/s.  The cut is taken when it comes out under 0.9 of the best whole
// product (at the 3B and 1.5B products of 2,048 rows, whose 128 x 128 tiles fill the GPU in one
// round as it is, a cut priced at 0.9 to 0.97 measured 0.99 to 1.04).  Measured, whole + norm against cut + the pass that adds the slices, the
// residual and the norm: down (3,584 x 18,944) at 1,280 rows 237 against 152 us, at 2,048 rows 272
// against 247; output (3,584 x 3,584) at 1,280 rows 69 against 52.
struct PartialPlan { int slices; bool big; };
double load_factor(long long blocks) { return blocks <= 170 ? 0.72 : 0.72 + 0.28 * double(blocks - 170) / 86.0; }
PartialPlan partial_plan(int n_rows, int n_out, int n_in, bool direct_ok) {
  const long long tiles = (long long)((n_rows + 127) / 128) * ((n_out + 127) / 128);
  const int n_k = (n_in + 63) / 64;
  long long s = (224 + tiles - 1) / tiles;
  if (s > n_k / 4) s = n_k / 4;
  if (s > 8) s = 8;
  if (s < 1) s = 1;
  const long long big = (long long)((n_rows + 255) / 256) * ((n_out + 255) / 256);
  const long long big_grid = (big + kXcds - 1) / kXcds * kXcds;       // the grid is padded to whole eights
  if (s == 1 && direct_ok && 2 * big_grid <= sb::cu_count()) {
    const double per_cu = 0.93e9 / 256.0;                                        // a CU's flops per microsecond at speed 1
    const double speed[5] = {1.0, 1.05, 1.35, 0.0, 1.35 * 0.89};
    double t_whole = 0;
    for (int v = 0; v < 5; ++v) {
      if (v == 3) continue;
      const int bm = kShapes[v].bm, bn = kShapes[v].bn;
      const long long n_tiles = (long long)((n_rows + bm - 1) / bm) * ((n_out + bn - 1) / bn);
      const long long rounds = (n_tiles + sb::cu_count() - 1) / sb::cu_count(), last = n_tiles - (rounds - 1) * sb::cu_count();
      const double t = 2.0 * bm * bn * double(n_in) / (speed[v] * per_cu) * (double(rounds - 1) + load_factor(last)) + 14.0;
      if (v == 0 || t < t_whole) t_whole = t;
    }
    double t_best = 0;
    long long s_best = 0;
    for (long long s2 = 2; s2 <= 8 && s2 * big_grid <= sb::cu_count() && s2 <= n_k / 4; ++s2) {
      const int per = int((n_k + s2 - 1) / s2);
      const double t = 2.0 * 256 * 256 * (64.0 * per) / (speed[2] * per_cu) * load_factor(s2 * big_grid) + 14.0 +
                       (2.0 * s2 - 2.0) * n_rows * double(n_out) * 4.0 / 4e6;
      if (s_best == 0 || t < t_best) t_best = t, s_best = s2;
    }
    if (s_best && t_best < 0.9 * t_whole) {
      const int per = int((n_k + s_best - 1) / s_best);
      return {(n_k + per - 1) / per, true};
    }
  }
  const int per = int((n_k + s - 1) / s);
  return {(n_k + per - 1) / per, false};
}
}  // namespace

// Slices sb_gemm_mfma_partial_bf16 writes for these sizes.
extern "C" int sb_gemm_mfma_slices(int n_rows, int n_out, int n_in, int packed) {
  return partial_plan(n_rows, n_out, n_in, packed && n_in % 64 == 0).slices;
}

// The raw product X W^T in K slices: partial float [slices][n_rows][n_out], for a consumer that
// adds the slices itself.  For few rows against a narrow, long matrix, where one slice would not
// give the GPU enough tiles.  128 x 128 tiles, or 256 x 256 (see partial_plan).
extern "C" int sb_gemm_mfma_partial_bf16(float *partial, const void *x, const void *w, int n_rows, int n_out,
                                         int n_in, int packed, void *stream) {
  SB_REQUIRE(partial && x && w, "sb_gemm_mfma_partial_bf16: null pointer");
  SB_REQUIRE(n_rows >= 0 && n_out > 0 && n_in > 0, "sb_gemm_mfma_partial_bf16: bad sizes rows=%d out=%d in=%d",
             n_rows, n_out, n_in);
  SB_SUPPORT(n_in % 8 == 0, "sb_gemm_mfma_partial_bf16: inner size %d is not a multiple of 8", n_in);
  SB_SUPPORT((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) % 16 == 0,
             "sb_gemm_mfma_partial_bf16: operands must be 16-byte aligned");
  if (n_rows == 0) return SB_OK;
  Args a;
  a.y = nullptr; a.y_dtype = SB_F32; a.x = (const bf16_t *)x; a.w = (const bf16_t *)w;
  a.bias = nullptr; a.bias_dtype = 0; a.resid = nullptr;
  a.n_rows = n_rows; a.n_out = n_out; a.n_in = n_in; a.gated = 0;
  const PartialPlan plan = partial_plan(n_rows, n_out, n_in, packed && n_in % 64 == 0);
  const int tile = plan.big ? 256 : 128;
  a.tiles_m = (n_rows + tile - 1) / tile;
  a.tiles_n = (n_out + tile - 1) / tile;
  const long long blocks = (long long)a.tiles_m * a.tiles_n;
  SB_SUPPORT(blocks <= 0x7fffffffLL, "sb_gemm_mfma_partial_bf16: too many tiles");
  const unsigned long long w_rows = (unsigned long long)((n_out + 15) / 16 * 16);
  const unsigned long long k_padded = (unsigned long long)((n_in + 31) / 32 * 32);
  // with room for the rows and row tiles past an operand's end that a block at the edge asks for
  SB_SUPPORT(((unsigned long long)n_rows + 257) * n_in * 2 < (1ull << 32) - (1ull << 20) &&
                 (w_rows + 512) * k_padded * 2 < (1ull << 32) - (1ull << 20),
             "sb_gemm_mfma_partial_bf16: an operand of 4 GiB or more");
  a.w_tiles = (n_out + 15) / 16;
  a.w_steps = (n_in + 31) / 32;
  const int slices = plan.slices;
  const int n_k = (n_in + 63) / 64;
  a.partial = partial;
  a.vec4 = n_out % 4 == 0 && reinterpret_cast<uintptr_t>(partial) % 16 == 0;
  a.stages_per_slice = (n_k + slices - 1) / slices;
  const int rc = plan.big ? launch_direct_one<8, 4, 64, 2, 0, false>(a, blocks, 0, (hipStream_t)stream)
                          : launch<2, 2, 64, 2, true>(a, blocks, packed, (hipStream_t)stream);
  if (rc != SB_OK) return rc;
  return sb::check_launch("sb_gemm_mfma_partial_bf16");
}

