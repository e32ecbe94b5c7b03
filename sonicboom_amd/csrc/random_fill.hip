// Seeded normal weights on the device: element e of tensor number i under a 64-bit seed.
//
// Philox4x32-10 with the seed as key and counter (e / 4 low, e / 4 high, i, 0) gives four words;
// words 0 and 1 make the standard normals of elements 4c and 4c + 1, words 2 and 3 those of
// 4c + 2 and 4c + 3 (Box and Muller: radius sqrt(-2 ln u) from the first word's u = (w + 0.5) /
// 2^32, angle 2 pi (w' + 0.5) / 2^32 from the second, cosine then sine).  The value stored is
// float32(mean + std z), rounded once more for bfloat16.
//
// The host computes the same function to the bit (sonicboom_amd/weights/random_stream.py), which
// is why no library logarithm, sine or cosine appears here: the logarithm is 2 s (1 + s^2/3 + ...
// + s^20/21) with s = (m - 1) / (m + 1) on the mantissa in [sqrt(1/2), sqrt(2)) plus the exponent
// times ln 2; sine and cosine are their series on an angle reduced in integers to at most pi / 4.
// Every float64 operation below is an addition, multiplication, division or square root rounded
// once; the pragma keeps the compiler from fusing a product with a sum, which the host cannot do.
#pragma clang fp contract(off)

#include "common.h"

namespace {

__device__ __forceinline__ void philox4(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint64_t key,
                                        uint32_t (&w)[4]) {
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
  w[0] = c0, w[1] = c1, w[2] = c2, w[3] = c3;
}

// -2 ln((w + 0.5) / 2^32)
__device__ __forceinline__ double neg2_log_u(uint32_t w) {
  const double x = double(w) * 2.0 + 1.0;                 // an odd integer below 2^33: exact
  const uint64_t bits = (uint64_t)__double_as_longlong(x);
  int e = int((bits >> 52) & 0x7ff) - 1022;               // x = m 2^e with 0.5 <= m < 1
  double m = __longlong_as_double((long long)((bits & 0x000fffffffffffffull) | 0x3fe0000000000000ull));
  if (m < 0x1.6a09e667f3bcdp-1) {
    m = m * 2.0;
    e -= 1;
  }
  const double s = (m - 1.0) / (m + 1.0);
  const double s2 = s * s;
  const double c[11] = {0x1.0000000000000p+0, 0x1.5555555555555p-2, 0x1.999999999999ap-3, 0x1.2492492492492p-3,
                        0x1.c71c71c71c71cp-4, 0x1.745d1745d1746p-4, 0x1.3b13b13b13b14p-4, 0x1.1111111111111p-4,
                        0x1.e1e1e1e1e1e1ep-5, 0x1.af286bca1af28p-5, 0x1.8618618618618p-5};
  double p = c[10];
#pragma unroll
  for (int k = 9; k >= 0; --k) p = p * s2 + c[k];
  const double ln = double(e - 33) * 0x1.62e42fefa39efp-1 + (2.0 * s) * p;
  return -2.0 * ln;
}

// cos and sin of 2 pi (w + 0.5) / 2^32
__device__ __forceinline__ void cos_sin(uint32_t w, double &cos_out, double &sin_out) {
  const uint64_t y = uint64_t(w) * 2 + 1;                  // the angle is 2 pi y / 2^33
  const int octant = int(y >> 30);
  int64_t r = int64_t(y & ((1ull << 30) - 1));
  if (octant & 1) r = (int64_t(1) << 30) - r;
  const double phi = double(r) * 0x1.921fb54442d18p-31;    // (pi / 4) / 2^30
  const double p2 = phi * phi;
  const double sc[8] = {0x1.0000000000000p+0,  -0x1.5555555555555p-3, 0x1.1111111111111p-7,  -0x1.a01a01a01a01ap-13,
                        0x1.71de3a556c734p-19, -0x1.ae64567f544e4p-26, 0x1.6124613a86d09p-33, -0x1.ae7f3e733b81fp-41};
  const double cc[9] = {0x1.0000000000000p+0,  -0x1.0000000000000p-1, 0x1.5555555555555p-5,
                        -0x1.6c16c16c16c17p-10, 0x1.a01a01a01a01ap-16, -0x1.27e4fb7789f5cp-22,
                        0x1.1eed8eff8d898p-29, -0x1.93974a8c07c9dp-37, 0x1.ae7f3e733b81fp-45};
  double sp = sc[7];
#pragma unroll
  for (int k = 6; k >= 0; --k) sp = sp * p2 + sc[k];
  sp = sp * phi;
  double cp = cc[8];
#pragma unroll
  for (int k = 7; k >= 0; --k) cp = cp * p2 + cc[k];
  const bool swap = octant == 1 || octant == 2 || octant == 5 || octant == 6;
  double c = swap ? sp : cp, s = swap ? cp : sp;
  if (octant >= 2 && octant <= 5) c = -c;
  if (octant >= 4) s = -s;
  cos_out = c;
  sin_out = s;
}

// One thread per counter: four elements.  OUT: 0 float32, 1 bfloat16, 2 the float64 standard
// normals themselves (what the tests compare with the host's).
template <int OUT>
__global__ void __launch_bounds__(256)
random_normal_kernel(void *__restrict__ out, uint64_t n, uint64_t first_counter, uint64_t seed, uint32_t tensor_index,
                     double mean, double std) {
  const uint64_t local = uint64_t(blockIdx.x) * 256 + threadIdx.x;
  if (local * 4 >= n) return;
  const uint64_t counter = first_counter + local;
  uint32_t w[4];
  philox4(uint32_t(counter), uint32_t(counter >> 32), tensor_index, 0u, seed, w);
  double z[4];
#pragma unroll
  for (int pair = 0; pair < 2; ++pair) {
    const double radius = __dsqrt_rn(neg2_log_u(w[2 * pair]));
    double c, s;
    cos_sin(w[2 * pair + 1], c, s);
    z[2 * pair] = radius * c;
    z[2 * pair + 1] = radius * s;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint64_t e = local * 4 + i;
    if (e >= n) break;
    if (OUT == 2) {
      ((double *)out)[e] = z[i];
    } else {
      const float v = float(z[i] * std + mean);
      if (OUT == 0) ((float *)out)[e] = v;
      else ((bf16_t *)out)[e] = f32_to_bf16(v);
    }
  }
}

}  // namespace

extern "C" int sb_random_normal(void *out, int out_kind, uint64_t n, uint64_t first, uint64_t seed, int tensor_index,
                                double mean, double std, void *stream) {
  SB_REQUIRE(out != nullptr || n == 0, "sb_random_normal: no output buffer");
  SB_REQUIRE(out_kind >= 0 && out_kind <= 2, "sb_random_normal: output kind %d (0 float32, 1 bfloat16, 2 float64)", out_kind);
  SB_REQUIRE(tensor_index >= 0, "sb_random_normal: negative tensor number");
  SB_REQUIRE(first % 4 == 0, "sb_random_normal: the first element must be a multiple of four (a whole counter)");
  if (n == 0) return SB_OK;
  const uint64_t counters = (n + 3) / 4, blocks = (counters + 255) / 256;
  SB_SUPPORT(blocks <= 0x7fffffffull, "sb_random_normal: %llu elements are more than one launch takes",
             (unsigned long long)n);
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid{(unsigned)blocks}, block{256};
  if (out_kind == 0)
    hipLaunchKernelGGL(random_normal_kernel<0>, grid, block, 0, s, out, n, first / 4, seed, uint32_t(tensor_index), mean, std);
  else if (out_kind == 1)
    hipLaunchKernelGGL(random_normal_kernel<1>, grid, block, 0, s, out, n, first / 4, seed, uint32_t(tensor_index), mean, std);
  else
    hipLaunchKernelGGL(random_normal_kernel<2>, grid, block, 0, s, out, n, first / 4, seed, uint32_t(tensor_index), mean, std);
  return sb::check_launch("sb_random_normal");
}
