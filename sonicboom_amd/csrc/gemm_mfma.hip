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
};

// index (in 16-byte chunks) of chunk `chunk` of LDS row `row`, CPR chunks per row
template <int CPR>
__device__ __forceinline__ int swz(int row, int chunk) {
  return row * CPR + (chunk ^ ((row / (16 / CPR)) & (CPR - 1)));
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

  // XCD-aware order: hardware sends block b to XCD b % 8.  XCD x gets the contiguous run of
  // tiles [x * per, (x + 1) * per), which share rows of X and W in that XCD's L2; the grid is
  // padded to a multiple of eight blocks, and the blocks past the last tile leave at once.
  const int n_blocks = a.tiles_m * a.tiles_n;
  const int per_xcd = (n_blocks + kXcds - 1) / kXcds;
  const int bid = (int(blockIdx.x) % kXcds) * per_xcd + int(blockIdx.x) / kXcds;
  if (bid >= n_blocks) return;
  // tiles of one column of N (same W rows) are neighbours: m runs fastest
  const int tn = bid / a.tiles_m, tm = bid - tn * a.tiles_m;
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
  bf16x8_t staged[DEPTH][kLoads];
  typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
  auto issue_load = [&](auto SET, int i, int kt) {
    constexpr int set = decltype(SET)::value;
    const bool is_a = i < kLoadsA;
    // uniform part of the address: the stage's offset along K
    const int stage_off = (PACKED && !is_a) ? kt * (kSteps32 * 1024) : kt * (BK * 2);
    uint32_t offset;
    if constexpr (kLinear) offset = is_a ? off[0] + uint32_t(i) * stride_a : off[1] + uint32_t(i - kLoadsA) * stride_b;
    else offset = off[i];
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

  const int n_k_all = (a.n_in + BK - 1) / BK;
  const int kt_begin = a.partial ? int(blockIdx.y) * a.stages_per_slice : 0;
  const int n_k = a.partial ? min(kt_begin + a.stages_per_slice, n_k_all) : n_k_all;   // end of this slice
  using Set0 = std::integral_constant<int, 0>;
  using Set1 = std::integral_constant<int, 1>;
#pragma unroll
  for (int i = 0; i < kLoads; ++i) issue_load(Set0{}, i, kt_begin);
  if (DEPTH == 2 && kt_begin + 1 < n_k) {
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
    constexpr int cur = decltype(CUR)::value;
    constexpr bool do_load = decltype(LOAD)::value, do_store = decltype(STORE)::value;
    using SetCur = std::integral_constant<int, DEPTH == 2 ? cur : 0>;          // set to load into
    using SetNext = std::integral_constant<int, DEPTH == 2 ? (cur ^ 1) : 0>;   // set to store from
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
            if (l >= at * kLoads / kHalf && l < (at + 1) * kLoads / kHalf) issue_load(SetCur{}, l, kt + DEPTH);
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
  if (DEPTH == 2) {
    for (; kt + 3 < n_k; kt += 2) {
      stage(Set0{}, Yes{}, Yes{}, kt);
      stage(Set1{}, Yes{}, Yes{}, kt + 1);
    }
    const int rest = n_k - kt;
    if (rest == 3) {
      stage(Set0{}, Yes{}, Yes{}, kt);
      stage(Set1{}, No{}, Yes{}, kt + 1);
      stage(Set0{}, No{}, No{}, kt + 2);
    } else if (rest == 2) {
      stage(Set0{}, No{}, Yes{}, kt);
      stage(Set1{}, No{}, No{}, kt + 1);
    } else if (rest == 1) {
      stage(Set0{}, No{}, No{}, kt);
    }
  } else {
    for (; kt + 2 < n_k; kt += 2) {
      stage(Set0{}, Yes{}, Yes{}, kt);
      stage(Set1{}, Yes{}, Yes{}, kt + 1);
    }
    if (n_k - kt == 2) {
      stage(Set0{}, Yes{}, Yes{}, kt);
      stage(Set1{}, No{}, No{}, kt + 1);
    } else {
      stage(Set0{}, No{}, No{}, kt);
    }
  }

  // Epilogue.  acc[i][j][e]: row = 8 * (e / 4) + 4 * (lane / 32) + e % 4, column = lane % 32.
  const int col = lane & 31, row_base = (lane >> 5) * 4;
#pragma unroll
  for (int i = 0; i < MT; ++i) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int t = t0 + wm * (32 * MT) + i * 32 + 8 * (e >> 2) + row_base + (e & 3);
      if (t >= a.n_rows) continue;
      if (!GATED && a.partial) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int n = n0 + wn * 64 + j * 32 + col;
          if (n < a.n_out) a.partial[(size_t(blockIdx.y) * a.n_rows + t) * a.n_out + n] = acc[i][j][e];
        }
        continue;
      }
      if (GATED) {
        const int n = n0 + wn * 32 + col;
        if (n < a.n_out) {
          const float v = gate_act(acc[i][0][e], GATED) * acc[i][1][e];     // GATED: the sb_gate, fixed at compile time
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

constexpr int kCus = 256;

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

// Tile shapes the launcher chooses from: rows x columns of Y per block.
struct Shape { int bm, bn; };
constexpr Shape kShapes[3] = {{128, 128}, {256, 128}, {256, 256}};

// The tile shape for a problem, from what was measured on MI355X (cold weights, 2,048 to 16,384
// rows).  The gated product (a wide matrix, SiLU epilogue): rounds of the grid over the CUs times
// the work of a block, the bigger tiles getting credit for the operand traffic they save; that
// ends at 256 x 256 for every size tried.  Plain products against narrower matrices: two blocks
// of 128 x 128 share a CU (64 KB of LDS and 128 registers each), one block's first loads and
// epilogue hide behind the other's loop, and with an inner size of a few thousand that beats the
// lone 256 x 128 block by 7 to 47 % (output product of 3,584 x 3,584 at 16,384 rows: 618 against
// 910 us); only a long inner size with few blocks (the down product up to 4,096 rows) is better
// off with 256 x 128, by 10 %.
int pick_shape(int n_rows, int n_out, int n_in, int gated) {
  if (!gated) {
    const long long blocks_1 = (long long)((n_rows + 255) / 256) * ((n_out + 127) / 128);
    return (n_in >= 8192 && blocks_1 <= 2 * kCus) ? 1 : 0;
  }
  double best = 0;
  int pick = 0;
  const double speed[3] = {1.0, 1.2, 1.3};    // measured rate of a full grid, relative
  for (int v = 0; v < 3; ++v) {
    const int bn = kShapes[v].bn / 2;
    const long long blocks = (long long)((n_rows + kShapes[v].bm - 1) / kShapes[v].bm) * ((n_out + bn - 1) / bn);
    const long long rounds = (blocks + kCus - 1) / kCus;
    const double cost = double(rounds) * kShapes[v].bm * kShapes[v].bn / speed[v];
    if (v == 0 || cost < best) { best = cost; pick = v; }
  }
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
  int variant = pick_shape(n_rows, n_out, n_in, a.gated);
  if (tile_shape >= 0 && tile_shape < 3) variant = tile_shape;      // a test's or a measurement's choice
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
  if (variant == 0) rc = launch<2, 2, 64, 2, true>(a, blocks, packed, s);
  else if (variant == 1) rc = launch<4, 2, 64, 2, false>(a, blocks, packed, s);
  else rc = launch<4, 4, 64, 1, false>(a, blocks, packed, s);
  if (rc != SB_OK) return rc;
  return sb::check_launch("sb_gemm_mfma_bf16");
}

namespace {
// K slices of the partial form: enough blocks for the GPU (one 128 x 128 tile per CU and slice),
// every slice at least four stages of 64 long, at most the eight that the consumers add.
int partial_slices(int n_rows, int n_out, int n_in) {
  const long long tiles = (long long)((n_rows + 127) / 128) * ((n_out + 127) / 128);
  const int n_k = (n_in + 63) / 64;
  long long s = (224 + tiles - 1) / tiles;
  if (s > n_k / 4) s = n_k / 4;
  if (s > 8) s = 8;
  if (s < 1) s = 1;
  const int per = int((n_k + s - 1) / s);
  return (n_k + per - 1) / per;
}
}  // namespace

// Slices sb_gemm_mfma_partial_bf16 writes for these sizes.
extern "C" int sb_gemm_mfma_slices(int n_rows, int n_out, int n_in) { return partial_slices(n_rows, n_out, n_in); }

// The raw product X W^T in K slices: partial float [slices][n_rows][n_out], for a consumer that
// adds the slices itself.  For few rows against a narrow, long matrix, where one slice would not
// give the GPU enough tiles.  128 x 128 tiles.
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
  a.tiles_m = (n_rows + 127) / 128;
  a.tiles_n = (n_out + 127) / 128;
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
  const int slices = partial_slices(n_rows, n_out, n_in);
  const int n_k = (n_in + 63) / 64;
  a.partial = partial;
  a.stages_per_slice = (n_k + slices - 1) / slices;
  const int rc = launch<2, 2, 64, 2, true>(a, blocks, packed, (hipStream_t)stream);
  if (rc != SB_OK) return rc;
  return sb::check_launch("sb_gemm_mfma_partial_bf16");
}

