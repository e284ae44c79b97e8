// The arithmetic of the seeded random stream, apart from the kernels so that a host
// compiler can build it too (a CPU test compares it with the numpy twin bit for bit).
// Every function is __host__ __device__ and uses nothing but integer operations and
// float64 additions, multiplications, divisions and one square root.
#pragma once

#include <stdint.h>
#include <math.h>

namespace hfee_random {

#pragma clang fp contract(off)

__host__ __device__ inline uint64_t mix(uint64_t key, uint64_t counter) {
  uint64_t z = key + (counter + 1) * 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// -2 ln(p) for p = n / 2^33, n odd, 0 < n < 2^33.
// n = m 2^e with m in [sqrt(1/2), sqrt(2)); ln m = 2 atanh(t), t = (m - 1) / (m + 1),
// |t| <= 0.1716, by the series t (1 + t^2/3 + t^4/5 + ...) to t^22.
__host__ __device__ inline double minus_two_log(uint64_t n) {
  const int lead = 63 - __builtin_clzll(n);          // n in [2^lead, 2^(lead+1))
  double m = (double)n * __builtin_bit_cast(double, (int64_t)(1023 - lead - 1) << 52);     // exact: in [0.5, 1)
  int e = lead + 1;
  if (m < 0.7071067811865476) {
    m = m * 2.0;
    e -= 1;
  }
  const double t = (m - 1.0) / (m + 1.0);
  const double t2 = t * t;
  double s = 1.0 / 23.0;
  for (int k = 21; k >= 1; k -= 2) s = s * t2 + 1.0 / (double)k;
  const double log_m = 2.0 * (t * s);
  return 2.0 * ((double)(33 - e) * 0.6931471805599453 - log_m);
}

// cos and sin of 2 pi k / 2^32: the octant by integer arithmetic, then Taylor series on
// [0, pi/4] to x^18 and x^19.
__host__ __device__ inline void cos_sin_turn(uint32_t k, double& c_out, double& s_out) {
  const uint32_t octant = k >> 29;
  uint32_t r = k & 0x1FFFFFFFu;
  if (octant & 1) r = 0x20000000u - r;
  const double x = (double)r * (0.7853981633974483 / 536870912.0);
  const double x2 = x * x;
  double c = 1.0, s = 1.0;
  for (int j = 9; j >= 1; --j) {
    c = 1.0 - x2 * c * (1.0 / (double)((2 * j - 1) * (2 * j)));
    s = 1.0 - x2 * s * (1.0 / (double)((2 * j) * (2 * j + 1)));
  }
  s = s * x;
  double co, si;
  switch (octant) {
    case 0: co = c; si = s; break;
    case 1: co = s; si = c; break;
    case 2: co = -s; si = c; break;
    case 3: co = -c; si = s; break;
    case 4: co = -c; si = -s; break;
    case 5: co = -s; si = -c; break;
    case 6: co = s; si = -c; break;
    default: co = c; si = -s; break;
  }
  c_out = co;
  s_out = si;
}

// Elements 2j and 2j + 1 of the stream: std * z (plus_one: 1 + std * z) with z standard
// normal, float64 rounded once to float32.
__host__ __device__ inline void normal_pair(uint64_t key, uint64_t j, bool plus_one, double std, float& f0, float& f1) {
  const uint64_t h = mix(key, j);
  const double radius = sqrt(minus_two_log(2 * (h >> 32) + 1));
  double c, s;
  cos_sin_turn((uint32_t)h, c, s);
  double z0 = std * (radius * c), z1 = std * (radius * s);
  if (plus_one) {
    z0 = 1.0 + z0;
    z1 = 1.0 + z1;
  }
  f0 = (float)z0;
  f1 = (float)z1;
}

// Element i of the integer stream, in [0, bound).
__host__ __device__ inline int32_t integer(uint64_t key, uint64_t i, uint32_t bound) {
  return (int32_t)((mix(key, i) >> 11) % bound);
}

}  // namespace hfee_random
