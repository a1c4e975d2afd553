/* Seeded synthetic payloads; see include/tp_datagen.h. */
#include "tp_datagen.h"

#include <math.h>
#include <string.h>

static const uint64_t kGamma = 0x9E3779B97F4A7C15ull;

uint64_t tpdg_u64(uint64_t seed, uint64_t i) {
  uint64_t z = seed + (i + 1) * kGamma;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

void tpdg_fill_u8(uint64_t seed, uint8_t* out, uint64_t n) {
  uint64_t words = n / 8;
  for (uint64_t w = 0; w < words; ++w) {
    uint64_t v = tpdg_u64(seed, w);
    memcpy(out + w * 8, &v, 8); /* little-endian host */
  }
  if (n % 8) {
    uint64_t v = tpdg_u64(seed, words);
    memcpy(out + words * 8, &v, n % 8);
  }
}

static void normal_pair(uint64_t seed, uint64_t p, double sigma, double* z0, double* z1) {
  const double kTwoPi = 6.283185307179586476925286766559;
  const double kScale = 1.0 / 9007199254740992.0; /* 2^-53 */
  double u1 = (double)((tpdg_u64(seed, 2 * p) >> 11) + 1) * kScale; /* (0, 1] */
  double u2 = (double)(tpdg_u64(seed, 2 * p + 1) >> 11) * kScale;   /* [0, 1) */
  double r = sqrt(-2.0 * log(u1)) * sigma;
  *z0 = r * cos(kTwoPi * u2);
  *z1 = r * sin(kTwoPi * u2);
}

static uint16_t f32_to_bf16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  if ((x & 0x7fffffffu) > 0x7f800000u) {
    return (uint16_t)((x >> 16) | 0x40u); /* quiet NaN */
  }
  uint32_t lsb = (x >> 16) & 1u;
  x += 0x7fffu + lsb;
  return (uint16_t)(x >> 16);
}

static uint16_t f32_to_f16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t mant = x & 0x007fffffu;
  int32_t exp = (int32_t)((x >> 23) & 0xffu);
  if (exp == 0xff) {
    return (uint16_t)(sign | 0x7c00u | (mant ? 0x200u : 0u));
  }
  int32_t e = exp - 127 + 15;
  if (e >= 0x1f) {
    return (uint16_t)(sign | 0x7c00u);
  }
  if (e <= 0) {
    if (e < -10) {
      return (uint16_t)sign;
    }
    mant |= 0x00800000u;
    uint32_t shift = (uint32_t)(14 - e);
    uint32_t half = mant >> shift;
    uint32_t rem = mant & ((1u << shift) - 1u);
    uint32_t mid = 1u << (shift - 1);
    if (rem > mid || (rem == mid && (half & 1u))) {
      ++half;
    }
    return (uint16_t)(sign | half);
  }
  uint32_t half = ((uint32_t)e << 10) | (mant >> 13);
  uint32_t rem = mant & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) {
    ++half; /* may carry into the exponent, which is the correct rounding */
  }
  return (uint16_t)(sign | half);
}

void tpdg_fill_normal_f32(uint64_t seed, double sigma, float* out, uint64_t n) {
  for (uint64_t p = 0; 2 * p < n; ++p) {
    double z0, z1;
    normal_pair(seed, p, sigma, &z0, &z1);
    out[2 * p] = (float)z0;
    if (2 * p + 1 < n) {
      out[2 * p + 1] = (float)z1;
    }
  }
}

void tpdg_fill_normal_bf16(uint64_t seed, double sigma, uint16_t* out, uint64_t n) {
  for (uint64_t p = 0; 2 * p < n; ++p) {
    double z0, z1;
    normal_pair(seed, p, sigma, &z0, &z1);
    out[2 * p] = f32_to_bf16((float)z0);
    if (2 * p + 1 < n) {
      out[2 * p + 1] = f32_to_bf16((float)z1);
    }
  }
}

void tpdg_fill_normal_f16(uint64_t seed, double sigma, uint16_t* out, uint64_t n) {
  for (uint64_t p = 0; 2 * p < n; ++p) {
    double z0, z1;
    normal_pair(seed, p, sigma, &z0, &z1);
    out[2 * p] = f32_to_f16((float)z0);
    if (2 * p + 1 < n) {
      out[2 * p + 1] = f32_to_f16((float)z1);
    }
  }
}

void tpdg_loguniform_sizes(uint64_t seed, uint64_t lo, uint64_t hi, uint64_t* out, uint32_t n) {
  const double kScale = 1.0 / 9007199254740992.0;
  const double a = log((double)lo), b = log((double)hi);
  for (uint32_t i = 0; i < n; ++i) {
    double u = (double)(tpdg_u64(seed, i) >> 11) * kScale;
    double v = exp(a + (b - a) * u);
    uint64_t s = (uint64_t)llround(v / 2.0) * 2;
    if (s < lo) {
      s = lo;
    }
    if (s > hi) {
      s = hi;
    }
    out[i] = s;
  }
}

void tpdg_bench_pattern(uint8_t* out, uint64_t n) {
  for (uint64_t i = 0; i < n; ++i) {
    out[i] = (uint8_t)((i >> 8) ^ (i & 0xff));
  }
}

uint64_t tpdg_fnv1a64(const uint8_t* data, uint64_t n) {
  uint64_t h = 0xcbf29ce484222325ull;
  for (uint64_t i = 0; i < n; ++i) {
    h ^= data[i];
    h *= 0x100000001b3ull;
  }
  return h;
}
