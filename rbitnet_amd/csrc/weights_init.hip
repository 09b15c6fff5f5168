// Load-time kernels: random normal values that are the same on every device, and the copy that
// casts and places the rows of a stored matrix inside a packed one.
//
// rb_fill_normal.  The idea of the reference's toy model, every value fixed by a seed
// (crates/bitnet-core/src/model/toy.rs:16-30), for tensors of any size: element i of a tensor is a
// function of (key, i) alone, where the caller derives `key` from the seed and the tensor's name.
//   pair p = i / 2;  h = mix(key + (p + 1) * 0x9E3779B97F4A7C15)  (64-bit, wrapping)
//   m = (h >> 32) + 1 in [1, 2^32],  n = h & 0xffffffff
//   radius = sqrt(-2 ln(m / 2^32)),  angle = 2 pi n / 2^32
//   z = radius * cos(angle) for even i, radius * sin(angle) for odd i      (Box-Muller)
//   value = float32(mean + std * z), rounded once more to bfloat16 when that is the storage
// The logarithm, sine and cosine are spelled out below with double additions, multiplications,
// divisions and a square root only, none of them contracted into fused operations: all of these
// round the same way on every IEEE machine, so that weights/random_init.py, which repeats the same
// operations with numpy on the host, gives the same bits.
#include <math.h>

#include "api.h"
#include "common.h"

#pragma clang fp contract(off)

namespace {

__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z ^= z >> 30;
  z *= 0xBF58476D1CE4E5B9ull;
  z ^= z >> 27;
  z *= 0x94D049BB133111EBull;
  z ^= z >> 31;
  return z;
}

// ln(m / 2^32) for an integer m in [1, 2^32]:  m = f * 2^e with f in [sqrt(1/2), sqrt(2)),
// s = (f - 1) / (f + 1), ln f = 2 s (1 + s^2/3 + s^4/5 + ... + s^22/23)   (|s| < 0.172)
__device__ __forceinline__ double log_unit(uint32_t m_minus_1) {
  const double m = (double)m_minus_1 + 1.0;
  int e;
  double f = frexp(m, &e);            // f in [0.5, 1)
  if (f < 0.70710678118654752440) {
    f = f * 2.0;
    e -= 1;
  }
  const double s = (f - 1.0) / (f + 1.0);
  const double s2 = s * s;
  double p = 1.0 / 23.0;
  p = p * s2 + 1.0 / 21.0;
  p = p * s2 + 1.0 / 19.0;
  p = p * s2 + 1.0 / 17.0;
  p = p * s2 + 1.0 / 15.0;
  p = p * s2 + 1.0 / 13.0;
  p = p * s2 + 1.0 / 11.0;
  p = p * s2 + 1.0 / 9.0;
  p = p * s2 + 1.0 / 7.0;
  p = p * s2 + 1.0 / 5.0;
  p = p * s2 + 1.0 / 3.0;
  p = p * s2 + 1.0;
  return (double)(e - 32) * 0.69314718055994530942 + 2.0 * s * p;
}

// sine and cosine of x in [0, pi/4]: the power series to x^17 and x^18
__device__ __forceinline__ void sincos_octant(double x, double& s, double& c) {
  const double x2 = x * x;
  double p = 1.0 / 355687428096000.0;             // 1/17!
  p = p * x2 - 1.0 / 1307674368000.0;             // 1/15!
  p = p * x2 + 1.0 / 6227020800.0;                // 1/13!
  p = p * x2 - 1.0 / 39916800.0;                  // 1/11!
  p = p * x2 + 1.0 / 362880.0;                    // 1/9!
  p = p * x2 - 1.0 / 5040.0;                      // 1/7!
  p = p * x2 + 1.0 / 120.0;                       // 1/5!
  p = p * x2 - 1.0 / 6.0;                         // 1/3!
  p = p * x2 + 1.0;
  s = x * p;
  double q = -1.0 / 6402373705728000.0;           // 1/18!
  q = q * x2 + 1.0 / 20922789888000.0;            // 1/16!
  q = q * x2 - 1.0 / 87178291200.0;               // 1/14!
  q = q * x2 + 1.0 / 479001600.0;                 // 1/12!
  q = q * x2 - 1.0 / 3628800.0;                   // 1/10!
  q = q * x2 + 1.0 / 40320.0;                     // 1/8!
  q = q * x2 - 1.0 / 720.0;                       // 1/6!
  q = q * x2 + 1.0 / 24.0;                        // 1/4!
  q = q * x2 - 1.0 / 2.0;
  q = q * x2 + 1.0;
  c = q;
}

// The two normal numbers of pair p.
__device__ __forceinline__ void normal_pair(uint64_t key, uint64_t p, double& z0, double& z1) {
  const uint64_t h = mix64(key + (p + 1) * 0x9E3779B97F4A7C15ull);
  const uint32_t hi = (uint32_t)(h >> 32), lo = (uint32_t)h;
  const double radius = sqrt(-2.0 * log_unit(hi));
  // angle = (octant + r / 2^29) * pi/4; odd octants are walked backwards from their end
  const uint32_t octant = lo >> 29, r = lo & 0x1fffffffu;
  const uint32_t t = (octant & 1u) ? 0x20000000u - r : r;
  const double x = (double)t * (3.14159265358979323846 / 2147483648.0);        // t * (pi/4) / 2^29
  double s, c;
  sincos_octant(x, s, c);
  const bool swap = ((octant + 1u) >> 1) & 1u;              // octants 1, 2, 5, 6
  double cosv = swap ? s : c, sinv = swap ? c : s;
  if (((octant + 2u) >> 2) & 1u) cosv = -cosv;              // octants 2..5
  if (octant >> 2) sinv = -sinv;                            // octants 4..7
  z0 = radius * cosv;
  z1 = radius * sinv;
}

template <typename T>
__global__ __launch_bounds__(256) void fill_normal_kernel(T* __restrict__ out, long long n, uint64_t key, double mean,
                                                          double std) {
  const long long n_pairs = (n + 1) / 2;
  for (long long p = (long long)blockIdx.x * blockDim.x + threadIdx.x; p < n_pairs;
       p += (long long)gridDim.x * blockDim.x) {
    double z0, z1;
    normal_pair(key, (uint64_t)p, z0, z1);
    const float v0 = (float)(mean + std * z0), v1 = (float)(mean + std * z1);
    Num<T>::store(out + 2 * p, v0);
    if (2 * p + 1 < n) Num<T>::store(out + 2 * p + 1, v1);
  }
}

// dst row (row0 + (r / block) * period + r % block) = src row r, cast
template <typename S, typename T>
__global__ __launch_bounds__(256) void place_rows_kernel(const S* __restrict__ src, T* __restrict__ dst,
                                                         long long n_rows, long long width, long long row0,
                                                         long long block, long long period, int frag) {
  const long long total = n_rows * width;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (long long)gridDim.x * blockDim.x) {
    const long long r = i / width, c = i - r * width;
    const long long d = row0 + (r / block) * period + r % block;
    // fragment-major: blocks of 16 rows x 4 E columns (1 KB; E = the values of the destination's type
    // in 16 bytes: 8 bfloat16, 4 float32) in the order [rows / 16][width / (4 E)]; inside a block the
    // value of row r, column q lies at E * (16 * (q / E) + r) + q % E
    constexpr long long E = 16 / sizeof(T);
    const long long at = frag ? ((d / 16) * (width / (4 * E)) + c / (4 * E)) * (64 * E) +
                                    (16 * ((c % (4 * E)) / E) + d % 16) * E + c % E
                              : d * width + c;
    Num<T>::store(dst + at, Num<S>::load(src + i));
  }
}

int grid_for(long long work) {
  long long blocks = (work + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  return (int)(blocks < 1 ? 1 : blocks);
}

}  // namespace

extern "C" int rb_fill_normal(void* out, int dtype, long long n, unsigned long long key, double mean, double std,
                              void* stream) {
  RB_REQUIRE(n >= 0, "rb_fill_normal: negative count");
  RB_REQUIRE(dtype == RB_F32 || dtype == RB_BF16, "rb_fill_normal: dtype %d", dtype);
  if (n == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int grid = grid_for((n + 1) / 2);
  if (dtype == RB_F32)
    fill_normal_kernel<float><<<grid, 256, 0, s>>>((float*)out, n, (uint64_t)key, mean, std);
  else
    fill_normal_kernel<bf16_t><<<grid, 256, 0, s>>>((bf16_t*)out, n, (uint64_t)key, mean, std);
  RB_LAUNCH_CHECK();
  return 0;
}

extern "C" int rb_place_rows(const void* src, int src_dtype, void* dst, int dst_dtype, int dst_layout,
                             long long n_rows, long long width, long long dst_rows, long long row0, long long block,
                             long long period, void* stream) {
  RB_REQUIRE(dst_layout == 0 || (dst_layout == 1 && dst_rows % 16 == 0 && width % (dst_dtype == RB_F32 ? 16 : 32) == 0),
             "rb_place_rows: layout %d of a destination of %lld rows of %lld", dst_layout, dst_rows, width);
  RB_REQUIRE(n_rows >= 0 && width > 0 && block > 0 && period >= block && row0 >= 0,
             "rb_place_rows: bad sizes (rows %lld, width %lld, block %lld, period %lld, first row %lld)", n_rows, width,
             block, period, row0);
  RB_REQUIRE((src_dtype == RB_F32 || src_dtype == RB_BF16) && (dst_dtype == RB_F32 || dst_dtype == RB_BF16),
             "rb_place_rows: dtypes %d -> %d", src_dtype, dst_dtype);
  if (n_rows == 0) return 0;
  const long long last = row0 + ((n_rows - 1) / block) * period + (n_rows - 1) % block;
  RB_REQUIRE(last < dst_rows, "rb_place_rows: row %lld lies beyond the %lld rows of the destination", last, dst_rows);
  hipStream_t s = (hipStream_t)stream;
  const int grid = grid_for(n_rows * width);
#define RB_PLACE(S, T) \
  place_rows_kernel<S, T><<<grid, 256, 0, s>>>((const S*)src, (T*)dst, n_rows, width, row0, block, period, dst_layout)
  if (src_dtype == RB_F32 && dst_dtype == RB_F32)
    RB_PLACE(float, float);
  else if (src_dtype == RB_F32)
    RB_PLACE(float, bf16_t);
  else if (dst_dtype == RB_F32)
    RB_PLACE(bf16_t, float);
  else
    RB_PLACE(bf16_t, bf16_t);
#undef RB_PLACE
  RB_LAUNCH_CHECK();
  return 0;
}
