// A normal deviate addressed by (seed, element index), the same bits wherever it is computed.
//
// Random weights are made in device memory by a kernel (large models) or on the host (model folders); a
// tensor made one way must be the tensor made the other way, so that a host-side implementation can
// regenerate any tensor of a model that was made on the device.  Library logarithms, cosines and square
// roots differ between the two in their last bit, so the deviate is built from operations that IEEE 754
// rounds correctly everywhere (add, multiply and divide in float64, integer arithmetic, bit casts) in a
// fixed order; this file is compiled without contraction into fused multiply-adds on both sides.
//
//   h  = splitmix64(seed ^ splitmix64(i))
//   u  = ((h >> 40) + 1) / 2^24 in (0, 1],   v = ((h >> 16) & 0xffffff) / 2^24 in [0, 1)
//   z  = sqrt(-2 ln u) * cos(2 pi v)                                        (Box-Muller)
//   ln u  = (e - 24) ln 2 + ln m, u = m 2^(e-24), m in [sqrt(1/2), sqrt 2): ln m = 2 s (1 + s^2/3 + ... + s^12/13),
//           s = (m - 1) / (m + 1)                                           (truncation below 2e-12)
//   sqrt  : four Newton steps from a guess made of the argument's bits
//   cos   : quadrant from the top two bits of v, the rest x in [0, pi/2) through the nested Taylor forms of
//           cosine and sine up to x^22 and x^23
//   element = float32(mean + std * z), then rounded to the stored type.
//
// The reference's fixture is a seeded generator per test model (/root/reference/engine/src/model.rs:11335-11409).
#pragma once
#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define CN_HD __host__ __device__
#else
#define CN_HD
#endif

CN_HD inline uint64_t cn_splitmix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

CN_HD inline uint64_t cn_bits(double d) {
  uint64_t u;
  memcpy(&u, &d, 8);
  return u;
}

CN_HD inline double cn_from_bits(uint64_t u) {
  double d;
  memcpy(&d, &u, 8);
  return d;
}

CN_HD inline double cn_normal(uint64_t seed, uint64_t i) {
  const uint64_t h = cn_splitmix64(seed ^ cn_splitmix64(i));
  const uint32_t a = (uint32_t)(h >> 40);
  const uint32_t b = (uint32_t)(h >> 16) & 0xffffffu;

  // L = -2 ln((a + 1) / 2^24)
  const uint64_t kb = cn_bits((double)(a + 1u));                 // 1 .. 2^24, exact
  int e = (int)((kb >> 52) & 0x7ffu) - 1022;                      // a + 1 = m 2^e, m in [0.5, 1)
  double m = cn_from_bits((kb & 0x800fffffffffffffull) | (1022ull << 52));
  if (m < 0.70710678118654752) {
    m = m * 2.0;
    e -= 1;
  }
  const double s = (m - 1.0) / (m + 1.0);
  const double t = s * s;
  double p = 1.0 / 13.0;
  p = p * t + 1.0 / 11.0;
  p = p * t + 1.0 / 9.0;
  p = p * t + 1.0 / 7.0;
  p = p * t + 1.0 / 5.0;
  p = p * t + 1.0 / 3.0;
  p = p * t + 1.0;
  const double ln_m = 2.0 * s * p;
  const double L = 2.0 * ((double)(24 - e) * 0.6931471805599453 - ln_m);

  // r = sqrt(L)
  double r = 0.0;
  if (L > 0.0) {
    r = cn_from_bits((cn_bits(L) >> 1) + 0x1ff8000000000000ull);
    r = 0.5 * (r + L / r);
    r = 0.5 * (r + L / r);
    r = 0.5 * (r + L / r);
    r = 0.5 * (r + L / r);
  }

  // cos(2 pi b / 2^24)
  const uint32_t quadrant = b >> 22;
  const double x = (double)(b & 0x3fffffu) * (1.5707963267948966 / 4194304.0);
  const double x2 = x * x;
  double c = 1.0, sn = 1.0;
  for (int j = 11; j >= 1; --j) {
    c = 1.0 - x2 / (double)((2 * j - 1) * (2 * j)) * c;
    sn = 1.0 - x2 / (double)((2 * j) * (2 * j + 1)) * sn;
  }
  sn = sn * x;
  const double cs = quadrant == 0 ? c : quadrant == 1 ? -sn : quadrant == 2 ? -c : sn;
  return r * cs;
}

// element i of a tensor filled with mean + std * N(0, 1), as float32
CN_HD inline float cn_element(uint64_t seed, uint64_t i, double mean, double std) {
  return (float)(mean + std * cn_normal(seed, i));
}
