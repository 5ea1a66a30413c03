// Counter-based normal numbers that come out bit for bit the same on the host and on the GPU.
//
// value(seed, i) for element i of a tensor: elements come in pairs (2j, 2j + 1) from one 64-bit
// hash h = mix64(seed ^ mix64(j)) through Box-Muller,
//   u = ((h >> 32) + 1) / 2^32 in (0, 1],  f = (h & 0xffffffff) / 2^32 in [0, 1),
//   r = sqrt(-2 ln u),  z(2j) = r cos(2 pi f),  z(2j + 1) = r sin(2 pi f),
// then rounded once to float, multiplied by the standard deviation in float, and (for bfloat16
// storage) rounded to nearest even.
//
// The logarithm, sine and cosine are written out here as fixed sequences of IEEE double
// additions and multiplications (no library call, no fused multiply-add: contraction is switched
// off for these functions), and division and square root are correctly rounded on both sides, so
// the host compiler and hipcc's device pass produce the same bits.  Accuracy is that of double
// arithmetic (about 1e-16 relative), far beyond the float the value is rounded to.
//
// The reference has no random-weights mode (its model tests need a model file,
// src/models/qwen2/graph.rs:455-462 of yusiwen/minfer); this is the library's own.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define MF_HD __host__ __device__ inline
#else
#define MF_HD inline
#endif

MF_HD uint64_t mf_mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// ln(m / 2^32) for an integer m in [1, 2^32]
MF_HD double mf_ln_u32(uint64_t m) {
#pragma clang fp contract(off)
  // m = t * 2^e with t in [1, 2): shift the leading one to bit 32
  const int shift = m >> 32 ? 0 : __builtin_clzll(m) - 31;
  const uint64_t v = m << shift;
  int e = -shift;
  double t = (double)v * (1.0 / 4294967296.0);          // exact: v < 2^33
  if (t > 1.4142135623730951) { t = t * 0.5; ++e; }      // t in (0.707, 1.4143]
  const double s = (t - 1.0) / (t + 1.0);                // |s| <= 0.1716
  const double s2 = s * s;
  // 2 atanh(s) = 2 s (1 + s^2/3 + s^4/5 + ... + s^24/25), Horner from the far end
  double p = 1.0 / 25.0;
  p = p * s2 + 1.0 / 23.0;
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
  const double ln_t = 2.0 * s * p;
  return (double)e * 0.6931471805599453 + ln_t;
}

// cos and sin of 2 pi n / 2^32 for a 32-bit n
MF_HD void mf_sincos_turn(uint32_t n, double* c_out, double* s_out) {
#pragma clang fp contract(off)
  const uint32_t oct = n >> 29, rem = n & 0x1FFFFFFFu;
  const uint32_t frac = (oct & 1u) ? (0x20000000u - rem) : rem;     // distance to the octant's even end
  const double x = (double)frac * (0.7853981633974483 / 536870912.0);   // in [0, pi/4]
  const double x2 = x * x;
  // sin x = x (1 - x^2/3! + ... + x^16/17!), cos x = 1 - x^2/2! + ... + x^16/16!
  double sp = 1.0 / 355687428096000.0;
  sp = sp * x2 - 1.0 / 1307674368000.0;
  sp = sp * x2 + 1.0 / 6227020800.0;
  sp = sp * x2 - 1.0 / 39916800.0;
  sp = sp * x2 + 1.0 / 362880.0;
  sp = sp * x2 - 1.0 / 5040.0;
  sp = sp * x2 + 1.0 / 120.0;
  sp = sp * x2 - 1.0 / 6.0;
  sp = sp * x2 + 1.0;
  const double S = x * sp;
  double cp = 1.0 / 20922789888000.0;
  cp = cp * x2 - 1.0 / 87178291200.0;
  cp = cp * x2 + 1.0 / 479001600.0;
  cp = cp * x2 - 1.0 / 3628800.0;
  cp = cp * x2 + 1.0 / 40320.0;
  cp = cp * x2 - 1.0 / 720.0;
  cp = cp * x2 + 1.0 / 24.0;
  cp = cp * x2 - 1.0 / 2.0;
  cp = cp * x2 + 1.0;
  const double C = cp;
  double c, s;
  switch (oct) {
    case 0: c = C; s = S; break;        // x
    case 1: c = S; s = C; break;        // pi/2 - x
    case 2: c = -S; s = C; break;       // pi/2 + x
    case 3: c = -C; s = S; break;       // pi - x
    case 4: c = -C; s = -S; break;      // pi + x
    case 5: c = -S; s = -C; break;      // 3 pi/2 - x
    case 6: c = S; s = -C; break;       // 3 pi/2 + x
    default: c = C; s = -S; break;      // 2 pi - x
  }
  *c_out = c;
  *s_out = s;
}

// correctly rounded square root of a double: the host's IEEE instruction, the device's
// round-to-nearest routine
MF_HD double mf_sqrt(double a) {
#pragma clang fp contract(off)
#if defined(__HIP_DEVICE_COMPILE__)
  return __dsqrt_rn(a);
#else
  return __builtin_sqrt(a);
#endif
}

// the two standard normals of pair j under `seed`
MF_HD void mf_normal_pair(uint64_t seed, uint64_t j, double* z0, double* z1) {
#pragma clang fp contract(off)
  const uint64_t h = mf_mix64(seed ^ mf_mix64(j));
  const double ln_u = mf_ln_u32((h >> 32) + 1ull);
  const double r = mf_sqrt(-2.0 * ln_u);
  double c, s;
  mf_sincos_turn((uint32_t)(h & 0xFFFFFFFFull), &c, &s);
  *z0 = r * c;
  *z1 = r * s;
}

// float -> bfloat16 bits, round to nearest even (finite inputs)
MF_HD uint16_t mf_bf16_bits(float v) {
  union { float f; uint32_t u; } b;
  b.f = v;
  const uint32_t lsb = (b.u >> 16) & 1u;
  return (uint16_t)((b.u + 0x7FFFu + lsb) >> 16);
}

MF_HD float mf_bf16_value(uint16_t bits) {
  union { float f; uint32_t u; } b;
  b.u = (uint32_t)bits << 16;
  return b.f;
}

// element i of a tensor: N(0, std) as float; `round_bf16`: rounded to a bfloat16 value
MF_HD float mf_normal_value(uint64_t seed, uint64_t i, float std, int round_bf16) {
#pragma clang fp contract(off)
  double z0, z1;
  mf_normal_pair(seed, i >> 1, &z0, &z1);
  const float v = (float)((i & 1ull) ? z1 : z0) * std;
  return round_bf16 ? mf_bf16_value(mf_bf16_bits(v)) : v;
}
