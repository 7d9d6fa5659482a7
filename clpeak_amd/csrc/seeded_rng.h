// Counter-based seeded generator shared by host and device code of the backend.
// Element i of stream s under seed S is a pure function of (S, s, i), so a GPU
// thread can produce exactly the value the host would, with no upload.
// For s == 0 the 64-bit word is the (i+1)-th output of SplitMix64 started at S.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define MI355_HD __host__ __device__ inline
#else
#define MI355_HD inline
#endif

// Stream ids: one per kind of seeded input, so no two inputs share values.
enum : uint32_t {
  MI355_STREAM_BW     = 0,   // global-bandwidth buffer, uniform [0,1)
  MI355_STREAM_MAD    = 1,   // vector MAD accumulator seeds
  MI355_STREAM_MFMA_A = 2,
  MI355_STREAM_MFMA_B = 3,
  MI355_STREAM_SCALE_A = 4,
  MI355_STREAM_SCALE_B = 5,
  MI355_STREAM_SPARSE = 6,   // 2:4 keep patterns
  MI355_STREAM_GEMM_A = 7,
  MI355_STREAM_GEMM_B = 8,
  MI355_STREAM_MAD_Y  = 9,   // second operand of the int8 dot-product chain
};

MI355_HD uint64_t mi355_rng_word(uint64_t seed, uint32_t stream, uint64_t i) {
  uint64_t z = seed + 0x9E3779B97F4A7C15ull * (i + 1) + 0xD6E8FEB86659FD93ull * (uint64_t)stream;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// [0,1): 24 top bits, exact in fp32.
MI355_HD float mi355_rng_u01(uint64_t z) { return (float)(uint32_t)(z >> 40) * 0x1.0p-24f; }
// [-1,1): exact in fp32.
MI355_HD float mi355_rng_upm1(uint64_t z) {
  return (float)((int32_t)(uint32_t)(z >> 40) - (1 << 23)) * 0x1.0p-23f;
}
// Integer uniform in [0, m) from the high 32 bits (m <= 2^16 keeps the bias < 2^-16).
MI355_HD uint32_t mi355_rng_below(uint64_t z, uint32_t m) {
  return (uint32_t)(((z >> 32) * (uint64_t)m) >> 32);
}
