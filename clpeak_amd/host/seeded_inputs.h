// Seeded operands of the matrix tests, generated on the host (they are a few MiB).
// Values: element i of a stream is a pure function of (seed, stream, i), see
// ../csrc/seeded_rng.h.  Normal deviates are Box-Muller on two consecutive words,
// N(0,1) * sigma, rounded once (nearest even, saturating for the 8/6/4-bit formats) to the
// operand format.
#pragma once
#include <cstdint>
#include <vector>

enum class OperandFormat { F16, BF16, E4M3, E5M2, E2M3, E3M2, E2M1, I8 };

int operand_bits(OperandFormat f);   // bits per element: 16, 8, 6 or 4

// n elements of `stream`, packed K-contiguously (little-endian bit order for 6/4-bit codes).
// I8 ignores sigma: uniform integers in [-8, 7].
std::vector<uint8_t> seeded_operand(OperandFormat f, double sigma, uint64_t seed, uint32_t stream, uint64_t n);
// E8M0 block scales 2^e, e uniform in {-4..4} (byte 127 + e).
std::vector<uint8_t> seeded_e8m0(uint64_t seed, uint32_t stream, uint64_t n);
// 2:4 keep patterns: one byte per group of four, first kept position | second << 2, first < second.
std::vector<uint8_t> seeded_sparse_meta(uint64_t seed, uint32_t stream, uint64_t n);

// dst[i] = uniform [0,1) element i of `stream` (the values the device fill of the bandwidth buffer writes).
void seeded_uniform_f32(float *dst, uint64_t n, uint64_t seed, uint32_t stream);

// Round a double once to the narrow format; exported for tests.
uint32_t encode_operand(OperandFormat f, double x);
double seeded_normal(uint64_t seed, uint32_t stream, uint64_t i);
