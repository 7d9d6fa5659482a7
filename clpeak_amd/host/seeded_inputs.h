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

// The constants of the reference's matrix kernels, in the packing of seeded_operand: 1.0 in the 16-bit
// formats (src/rocm/rocm_kernels/mfma_fp16.hip:24-25, mfma_bf16.hip:16-17), byte 0x38 in the 8-bit floating
// formats (mfma_fp8.hip:17-18), byte 0x01 for int8 (mfma_int8.hip:17-18), nibble 4 for e2m1
// (mfma_mxfp4.hip:23-26); the fp6 formats, which the reference lacks, take their code of 1.0.  Its block
// scales are bytes of 0x3f (mfma_mxfp4.hip:28-29), its sparsity index register is 0 (smfmac_fp16.hip:26).
std::vector<uint8_t> reference_operand(OperandFormat f, uint64_t n);
constexpr uint8_t kReferenceScale = 0x3f, kReferenceSparseMeta = 0x00;

// dst[i] = uniform [0,1) element i of `stream` (the values the device fill of the bandwidth buffer writes).
void seeded_uniform_f32(float *dst, uint64_t n, uint64_t seed, uint32_t stream);

// Round a double once to the narrow format; exported for tests.
uint32_t encode_operand(OperandFormat f, double x);
double seeded_normal(uint64_t seed, uint32_t stream, uint64_t i);
