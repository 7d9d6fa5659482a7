// 2:4 structured-sparse SMFMAC throughput kernels, register resident.
//
// Same launch and chain scheme as the dense kernels: 4 waves per workgroup, 4
// independent accumulator chains per wave, acc[c] = SMFMAC(a[c], b[c], acc[c], idx[c])
// `iters` times, final tiles written row-major.  A arrives compressed (the two kept
// values of every group of four along K) with one metadata byte per group; each lane
// packs the metadata of its own K range into the index register once, before the loop.
// Work is counted with the dense-equivalent K.  MI355_MFMA_ONE_OPERAND_SET: the four chains take
// chain 0's A, B and index registers, as the reference's kernels do (src/rocm/rocm_kernels/smfmac_fp16.hip:22-40).
#include "internal.h"
#include "mfma_common.h"

namespace {

constexpr int kChains = 4;

// The hot loop is inline assembly for the reasons given in mfma_dense.hip: accumulate in place, no
// copies between matrix instructions, and every chain advanced by a run of 32 instructions before the
// next one takes over (an instruction naming its predecessor's registers costs less power).  SMFMAC
// takes its accumulator from the destination registers: D = A*B + D.
constexpr int kBlock = 32;
#define MI355_REP8(x) x x x x x x x x
#define MI355_REP32(x) MI355_REP8(x) MI355_REP8(x) MI355_REP8(x) MI355_REP8(x)
#define MI355_ONCE(x) x
// %0-%3 accumulators, %4-%7 compressed A, %8-%11 B, %12-%15 index registers
#define MI355_SP_CHAINS(REP, INSN)      \
  REP(INSN " %0, %4, %8, %12\n")        \
  REP(INSN " %1, %5, %9, %13\n")        \
  REP(INSN " %2, %6, %10, %14\n")       \
  REP(INSN " %3, %7, %11, %15\n")
#define MI355_SP_OPERANDS                                                                          \
  : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3])                                         \
  : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(b[0]), "v"(b[1]), "v"(b[2]), "v"(b[3]),        \
    "v"(idx[0]), "v"(idx[1]), "v"(idx[2]), "v"(idx[3])

// 16-bit data, 16x16x64: A 8 kept values per lane (16 B), B 16 values per lane (32 B),
// 4 groups per lane -> 16 index bits.  8-bit data, 16x16x128: A 16 kept values per lane
// (16 B), B 32 values per lane (32 B), 8 groups per lane -> 32 index bits.
#define MI355_SPARSE_TRAIT(NAME, K_, ELEM, FRAGA, FRAGB, ACC, OUT, INSN)                           \
  struct NAME {                                                                                    \
    static constexpr int K = K_, elem = ELEM;                                                      \
    using FragA = FRAGA; using FragB = FRAGB; using Acc = ACC; using Out = OUT;                    \
    __device__ static void block(Acc (&acc)[4], const FragA (&a)[4], const FragB (&b)[4], const int (&idx)[4]) { \
      asm volatile(MI355_SP_CHAINS(MI355_REP32, INSN) MI355_SP_OPERANDS);                            \
    }                                                                                              \
    __device__ static void single(Acc (&acc)[4], const FragA (&a)[4], const FragB (&b)[4], const int (&idx)[4]) { \
      asm volatile(MI355_SP_CHAINS(MI355_ONCE, INSN) MI355_SP_OPERANDS);                                        \
    }                                                                                              \
  };

MI355_SPARSE_TRAIT(SP_F16, 64, 2, half8v, half16v, f32x4v, float, "v_smfmac_f32_16x16x64_f16")
MI355_SPARSE_TRAIT(SP_BF16, 64, 2, bf16x8v, bf16x16v, f32x4v, float, "v_smfmac_f32_16x16x64_bf16")
MI355_SPARSE_TRAIT(SP_FP8, 128, 1, i32x4v, i32x8v, f32x4v, float, "v_smfmac_f32_16x16x128_fp8_fp8")
MI355_SPARSE_TRAIT(SP_BF8, 128, 1, i32x4v, i32x8v, f32x4v, float, "v_smfmac_f32_16x16x128_bf8_bf8")
MI355_SPARSE_TRAIT(SP_I8, 128, 1, i32x4v, i32x8v, i32x4v, int32_t, "v_smfmac_i32_16x16x128_i8")

template <typename Tr, bool ONE_SET>
__global__ void __launch_bounds__(256)
smfmac_kernel(const uint8_t *__restrict__ Ac, const uint8_t *__restrict__ meta, const uint8_t *__restrict__ B,
              typename Tr::Out *__restrict__ out, uint32_t iters, uint64_t *__restrict__ clocks, uint32_t active) {
  // diagnosis: only the workgroups of some XCDs (index mod 8) or of half the CUs of every XCD take part
  if (!((active >> (blockIdx.x % 8u)) & 1u) || ((active & 0x100u) && (blockIdx.x / 8u) % 32u >= 16u)) return;
  const int lane = threadIdx.x % 64;
  const uint64_t wave = (uint64_t)blockIdx.x * (blockDim.x / 64) + threadIdx.x / 64;
  constexpr int K = Tr::K;
  constexpr size_t ac_row = (size_t)(K / 2) * Tr::elem, b_row = (size_t)K * Tr::elem, m_row = K / 4;
  constexpr int groups = K / 16;  // groups of four in one lane's quarter of K

  typename Tr::FragA a[kChains];
  typename Tr::FragB b[kChains];
  typename Tr::Acc acc[kChains];
  int idx[kChains];
#pragma unroll
  for (int c = 0; c < kChains; c++) {
#pragma unroll
    for (int r = 0; r < 4; r++) acc[c][r] = 0;
    if (ONE_SET && c > 0) {   // the very registers of chain 0
      a[c] = a[0]; b[c] = b[0]; idx[c] = idx[0];
      continue;
    }
    const uint64_t u = wave * kChains + c;
    a[c] = load_bytes<typename Tr::FragA>(Ac + u * 16 * ac_row + (lane % 16) * ac_row + (lane / 16) * (ac_row / 4));
    {  // B: 16 bytes of the first K half and 16 bytes of the second (b_row is 128 for every kind)
      const uint8_t *brow = B + u * 16 * b_row + (lane % 16) * b_row + (lane / 16) * 16;
      const i32x4v lo = load_bytes<i32x4v>(brow), hi = load_bytes<i32x4v>(brow + b_row / 2);
      const i32x8v both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      __builtin_memcpy(&b[c], &both, sizeof(both));
    }
    const uint8_t *m = meta + u * 16 * m_row + (lane % 16) * m_row + (lane / 16) * groups;
    uint32_t packed = 0;
#pragma unroll
    for (int g = 0; g < groups; g++) packed |= (uint32_t)(m[g] & 0xf) << (4 * g);
    idx[c] = (int)packed;
  }

  const uint32_t blocks = iters / kBlock, rest = iters % kBlock;
  const uint64_t t0 = clock64(), r0 = wall_clock64();
#pragma unroll 1
  for (uint32_t it = 0; it < blocks; it++) Tr::block(acc, a, b, idx);
#pragma unroll 1
  for (uint32_t it = 0; it < rest; it++) Tr::single(acc, a, b, idx);
  // Wait states the compiler cannot know are needed before the results are read.
  asm volatile("s_nop 15\n s_nop 15" ::: "memory");
  if (clocks != nullptr && wave == 0 && lane == 0) {
    clocks[0] = clock64() - t0;
    clocks[1] = wall_clock64() - r0;
  }

#pragma unroll
  for (int c = 0; c < kChains; c++) {
    typename Tr::Out *tile = out + (wave * kChains + c) * 256u;
#pragma unroll
    for (int r = 0; r < 4; r++) tile[(4 * (lane / 16) + r) * 16 + lane % 16] = acc[c][r];
  }
}

template <typename Tr>
int launch(mi355_dev *dev, bool one_set, const void *Ac, const uint8_t *meta, const void *B, void *out, uint32_t waves,
           uint32_t iters, uint64_t *clocks, uint32_t active) {
  if (one_set)
    smfmac_kernel<Tr, true><<<waves / 4, 256, 0, dev->stream>>>((const uint8_t *)Ac, meta, (const uint8_t *)B,
                                                               (typename Tr::Out *)out, iters, clocks, active);
  else
    smfmac_kernel<Tr, false><<<waves / 4, 256, 0, dev->stream>>>((const uint8_t *)Ac, meta, (const uint8_t *)B,
                                                                (typename Tr::Out *)out, iters, clocks, active);
  MI355_LAUNCH_CHECK(dev, "smfmac");
  return MI355_OK;
}

}  // namespace

extern "C" int mi355_smfmac(mi355_dev *dev, int kind, const void *Ac, const uint8_t *meta, const void *B,
                            void *out, uint32_t waves, uint32_t iters, uint64_t *clocks) {
  MI355_ENTER(dev);
  MI355_REQUIRE(dev, Ac && meta && B && out, "smfmac: null buffer");
  MI355_REQUIRE(dev, waves > 0 && waves % 4 == 0, "smfmac: waves (%u) must be a positive multiple of 4", waves);
  MI355_REQUIRE(dev, (((uintptr_t)Ac | (uintptr_t)B | (uintptr_t)out) & 15u) == 0, "smfmac: buffers must be 16-byte aligned");
  const bool one_set = (kind & MI355_MFMA_ONE_OPERAND_SET) != 0;
  uint32_t active = ((uint32_t)kind >> 16) & 0xffu;   // MI355_MATRIX_ON_XCDS: 0 = every XCD
  if (active == 0u) active = 0xffu;
  MI355_REQUIRE(dev, (active & 1u) != 0u, "smfmac: XCD 0 must be among the XCDs that take part (its first wave reads the clocks)");
  if (kind & MI355_MATRIX_ON_HALF_THE_CUS) active |= 0x100u;
  kind &= 0xff;
  switch (kind) {
    case MI355_SMFMAC_F16_16x16x64:  return launch<SP_F16>(dev, one_set, Ac, meta, B, out, waves, iters, clocks, active);
    case MI355_SMFMAC_BF16_16x16x64: return launch<SP_BF16>(dev, one_set, Ac, meta, B, out, waves, iters, clocks, active);
    case MI355_SMFMAC_FP8_16x16x128: return launch<SP_FP8>(dev, one_set, Ac, meta, B, out, waves, iters, clocks, active);
    case MI355_SMFMAC_BF8_16x16x128: return launch<SP_BF8>(dev, one_set, Ac, meta, B, out, waves, iters, clocks, active);
    case MI355_SMFMAC_I8_16x16x128:  return launch<SP_I8>(dev, one_set, Ac, meta, B, out, waves, iters, clocks, active);
    default: return mi355_fail(dev, MI355_ERR_ARG, "smfmac: unknown kind %d", kind);
  }
}
