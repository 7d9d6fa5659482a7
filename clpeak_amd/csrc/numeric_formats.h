// Narrow floating-point encoders used by the backend (host and device).
// All conversions are round-to-nearest-even done in integer arithmetic, so the
// host and the GPU produce the same bits.
#pragma once
#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define MI355_HD __host__ __device__ inline
#else
#define MI355_HD inline
#endif

MI355_HD uint32_t mi355_f32_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
MI355_HD float mi355_bits_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}

// fp32 -> bf16, RNE; NaN stays NaN.
MI355_HD uint16_t mi355_f32_to_bf16(float f) {
  uint32_t u = mi355_f32_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
MI355_HD float mi355_bf16_to_f32(uint16_t h) { return mi355_bits_f32((uint32_t)h << 16); }

// Generic fp32 -> small float (1 sign, E exponent bits, M mantissa bits, bias B),
// RNE with gradual underflow.  `max_code` is the largest finite magnitude code
// (without sign); values that round above it saturate to it.  No Inf/NaN produced
// (NaN input maps to max_code as well; callers never pass NaN).
MI355_HD uint32_t mi355_f32_to_small(float f, int E, int M, int B, uint32_t max_code) {
  const uint32_t u = mi355_f32_bits(f);
  const uint32_t sign = (u >> 31) << (E + M);
  const uint32_t abs = u & 0x7fffffffu;
  if (abs >= 0x7f800000u) return sign | max_code;
  const int exp32 = (int)(abs >> 23);            // biased fp32 exponent, 0 for subnormals
  if (exp32 == 0) return sign;                   // fp32 subnormals are far below every small format
  uint32_t mant = (abs & 0x7fffffu) | 0x800000u; // 24-bit significand
  int e = exp32 - 127 + B;                       // exponent in the target bias
  int shift = 23 - M;                            // bits to drop for a normal result
  if (e <= 0) {                                  // subnormal in the target: shift further
    shift += 1 - e;
    e = 0;
    if (shift > 25) return sign;                 // below half of the smallest subnormal
  }
  const uint32_t lsb = 1u << shift;
  const uint32_t rem = mant & (lsb - 1);
  uint32_t q = mant >> shift;
  if (rem > (lsb >> 1) || (rem == (lsb >> 1) && (q & 1u))) q++;
  // q now holds (implicit bit | mantissa) for normals or the subnormal mantissa.
  uint32_t code;
  if (e == 0) code = q;                          // q == 1<<M becomes the smallest normal: same bits
  else code = ((uint32_t)(e - 1) << M) + q;      // carry out of the mantissa bumps the exponent
  if (code > max_code) code = max_code;
  return sign | code;
}

// OCP formats on gfx950.
MI355_HD uint8_t mi355_f32_to_e4m3(float f) { return (uint8_t)mi355_f32_to_small(f, 4, 3, 7, 0x7e); }   // max 448
MI355_HD uint8_t mi355_f32_to_e5m2(float f) { return (uint8_t)mi355_f32_to_small(f, 5, 2, 15, 0x7b); }  // max 57344
MI355_HD uint8_t mi355_f32_to_e2m3(float f) { return (uint8_t)mi355_f32_to_small(f, 2, 3, 1, 0x1f); }   // max 7.5
MI355_HD uint8_t mi355_f32_to_e3m2(float f) { return (uint8_t)mi355_f32_to_small(f, 3, 2, 3, 0x1f); }   // max 28
MI355_HD uint8_t mi355_f32_to_e2m1(float f) { return (uint8_t)mi355_f32_to_small(f, 2, 1, 1, 0x7); }    // max 6
MI355_HD uint16_t mi355_f32_to_f16(float f) {
  const uint32_t u = mi355_f32_bits(f);
  const uint32_t abs = u & 0x7fffffffu;
  if (abs > 0x7f800000u) return (uint16_t)(((u >> 16) & 0x8000u) | 0x7e00u);
  if (abs >= 0x477ff000u) return (uint16_t)(((u >> 16) & 0x8000u) | 0x7c00u);  // rounds to inf
  return (uint16_t)mi355_f32_to_small(f, 5, 10, 15, 0x7bff);
}
