#include "seeded_inputs.h"
#include <cmath>
#include <cstring>
#include "../csrc/seeded_rng.h"

namespace {
struct Layout { int E, M, bias; uint32_t maxCode; bool ieeeOverflow; };

Layout layout_of(OperandFormat f) {
  switch (f) {
    case OperandFormat::F16: return {5, 10, 15, 0x7bff, true};
    case OperandFormat::BF16: return {8, 7, 127, 0x7f7f, true};
    case OperandFormat::E4M3: return {4, 3, 7, 0x7e, false};
    case OperandFormat::E5M2: return {5, 2, 15, 0x7b, false};
    case OperandFormat::E2M3: return {2, 3, 1, 0x1f, false};
    case OperandFormat::E3M2: return {3, 2, 3, 0x1f, false};
    default: return {2, 1, 1, 0x7, false};   // E2M1
  }
}
}  // namespace

int operand_bits(OperandFormat f) {
  switch (f) {
    case OperandFormat::F16: case OperandFormat::BF16: return 16;
    case OperandFormat::E2M3: case OperandFormat::E3M2: return 6;
    case OperandFormat::E2M1: return 4;
    default: return 8;
  }
}

// One rounding, nearest even, from the double's own bits: the 53-bit significand is cut at the
// target's precision (or deeper for a subnormal result) and the dropped part decides.
uint32_t encode_operand(OperandFormat f, double x) {
  const Layout L = layout_of(f);
  uint64_t u;
  memcpy(&u, &x, 8);
  const uint32_t sign = (uint32_t)(u >> 63) << (L.E + L.M);
  const uint64_t mag = u & 0x7fffffffffffffffull;
  if (mag == 0) return sign;
  if (mag >= 0x7ff0000000000000ull) return sign | (L.ieeeOverflow && mag == 0x7ff0000000000000ull ? L.maxCode + 1 : L.maxCode);
  const int exp64 = (int)(mag >> 52);
  if (exp64 == 0) return sign;                       // double subnormal: far below every target
  const uint64_t sig = (mag & 0xfffffffffffffull) | (1ull << 52);
  int e = exp64 - 1023 + L.bias;                     // biased exponent in the target
  int drop = 52 - L.M;                               // bits to drop for a normal result
  if (e <= 0) { drop += 1 - e; e = 0; }
  if (drop > 62) return sign;                        // less than half of the smallest subnormal
  const uint64_t unit = 1ull << drop, rem = sig & (unit - 1);
  uint64_t q = sig >> drop;
  if (rem > unit / 2 || (rem == unit / 2 && (q & 1))) q++;
  // for a normal result q carries the implicit bit: (e-1)<<M + q = e<<M | mantissa, and a carry out
  // of the mantissa lands in the exponent; for a subnormal result q is the mantissa itself.
  uint64_t code = e == 0 ? q : ((uint64_t)(e - 1) << L.M) + q;
  if (code > L.maxCode) code = L.ieeeOverflow ? (uint64_t)L.maxCode + 1 : L.maxCode;   // infinity or saturate
  return sign | (uint32_t)code;
}

double seeded_normal(uint64_t seed, uint32_t stream, uint64_t i) {
  const uint64_t z1 = mi355_rng_word(seed, stream, 2 * i), z2 = mi355_rng_word(seed, stream, 2 * i + 1);
  const double u1 = ((double)(z1 >> 11) + 1.0) * 0x1.0p-53;   // (0, 1]
  const double u2 = (double)(z2 >> 11) * 0x1.0p-53;           // [0, 1)
  return std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586476925286766559 * u2);
}

void seeded_uniform_f32(float *dst, uint64_t n, uint64_t seed, uint32_t stream) {
  for (uint64_t i = 0; i < n; i++) dst[i] = mi355_rng_u01(mi355_rng_word(seed, stream, i));
}

std::vector<uint8_t> seeded_operand(OperandFormat f, double sigma, uint64_t seed, uint32_t stream, uint64_t n) {
  const int bits = operand_bits(f);
  std::vector<uint8_t> out((n * bits + 7) / 8, 0);
  for (uint64_t i = 0; i < n; i++) {
    uint32_t code;
    if (f == OperandFormat::I8) code = (uint32_t)(uint8_t)(int8_t)((int)(mi355_rng_word(seed, stream, i) >> 60) - 8);
    else code = encode_operand(f, sigma * seeded_normal(seed, stream, i));
    const uint64_t bit = i * bits;
    const uint32_t shifted = code << (bit & 7);
    out[bit >> 3] |= (uint8_t)shifted;
    if ((bit & 7) + bits > 8) out[(bit >> 3) + 1] |= (uint8_t)(shifted >> 8);
    if ((bit & 7) + bits > 16) out[(bit >> 3) + 2] |= (uint8_t)(shifted >> 16);
  }
  return out;
}

std::vector<uint8_t> reference_operand(OperandFormat f, uint64_t n) {
  uint32_t code = 0;
  switch (f) {
    case OperandFormat::F16: code = 0x3C00; break;
    case OperandFormat::BF16: code = 0x3F80; break;
    case OperandFormat::E4M3: case OperandFormat::E5M2: code = 0x38; break;
    case OperandFormat::E2M3: code = 0x08; break;
    case OperandFormat::E3M2: code = 0x0C; break;
    case OperandFormat::E2M1: code = 0x4; break;
    case OperandFormat::I8: code = 0x01; break;
  }
  const int bits = operand_bits(f);
  std::vector<uint8_t> out((n * bits + 7) / 8, 0);
  for (uint64_t i = 0; i < n; i++) {
    const uint64_t bit = i * bits;
    const uint32_t shifted = code << (bit & 7);
    out[bit >> 3] |= (uint8_t)shifted;
    if ((bit & 7) + bits > 8) out[(bit >> 3) + 1] |= (uint8_t)(shifted >> 8);
    if ((bit & 7) + bits > 16) out[(bit >> 3) + 2] |= (uint8_t)(shifted >> 16);
  }
  return out;
}

std::vector<uint8_t> seeded_e8m0(uint64_t seed, uint32_t stream, uint64_t n) {
  std::vector<uint8_t> out(n);
  for (uint64_t i = 0; i < n; i++) out[i] = (uint8_t)(123 + mi355_rng_below(mi355_rng_word(seed, stream, i), 9));
  return out;
}

std::vector<uint8_t> seeded_sparse_meta(uint64_t seed, uint32_t stream, uint64_t n) {
  static const uint8_t pairs[6][2] = {{0, 1}, {0, 2}, {0, 3}, {1, 2}, {1, 3}, {2, 3}};
  std::vector<uint8_t> out(n);
  for (uint64_t i = 0; i < n; i++) {
    const uint8_t *p = pairs[mi355_rng_below(mi355_rng_word(seed, stream, i), 6)];
    out[i] = (uint8_t)(p[0] | (p[1] << 2));
  }
  return out;
}
