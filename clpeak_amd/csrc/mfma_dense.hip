// Dense MFMA throughput kernels, register resident.
//
// One workgroup = 4 wavefronts (one per SIMD of a CU); the default launch of 2048
// waves puts 2 waves on every SIMD of a 256-CU part.  Each wave loads the fragments
// of its 4 chains from the logical A/B matrices once, then issues
//     acc[c] = MFMA(a[c], b[c], acc[c])        c = 0..3, `iters` times
// so that 4 independent accumulator tiles are always in flight and a dependent
// MFMA ever waits on a result it cannot have yet.  With MI355_MFMA_ONE_OPERAND_SET the four chains
// take the fragments of chain 0, from the SAME registers, as the reference's kernels do with
// their one a and one b (src/rocm/rocm_kernels/mfma_bf16.hip:16-30): an instruction whose
// sources are the registers its predecessor read costs the part less power than one that reads
// other registers holding the same values, and the clock it holds is 9 % higher.  The final accumulator tiles are written
// to memory in row-major order.  MFMA-bound: 2*M*N*K flops per instruction, no
// memory traffic inside the loop.
#include "internal.h"
#include "mfma_common.h"

namespace {

constexpr int kChains = 4;

// The hot loop is written as inline assembly: with the builtins the register
// allocator rotates the accumulator tiles through copies on every trip, and each
// copy next to an MFMA costs wait states.  One block = kBlock iterations of every chain,
// accumulating in place (vDst == SrcC), ONE CHAIN AFTER THE OTHER: 32 instructions on
// accumulator 0, then 32 on accumulator 1, and so on.  The matrix pipe forwards an
// accumulator to the next instruction that names it, so a run of dependent instructions
// issues back to back exactly like independent ones (97 % pipe utilisation either way), and
// an instruction that names the registers its predecessor named costs the part less power
// than one that switches: with the chains interleaved one instruction at a time the same
// seeded launch holds 1.96 GHz (bf16, 1.95 PFLOP/s), in runs of 2 / 4 / 8 / 16 / 32 it holds
// 2.14 / 2.26 / 2.29 / 2.33 / 2.33-2.36 GHz (2.17 / 2.29 / 2.35 / 2.39 / 2.42 PFLOP/s).
// Every chain still performs its `iters` dependent instructions in order, so results do
// not depend on the run length.  A block is 128 instructions because the loop branch costs
// the issuing wave about 20 cycles in which the pipe idles (waves of one SIMD run one after
// the other here: the oldest always has an MFMA ready and wins arbitration), 4 % at 32
// instructions per trip and 1 % at 128.
constexpr int kBlock = 32;

#define MI355_REP8(x) x x x x x x x x
#define MI355_REP32(x) MI355_REP8(x) MI355_REP8(x) MI355_REP8(x) MI355_REP8(x)
// %0-%3 accumulators, %4-%7 A fragments, %8-%11 B fragments
#define MI355_CHAINS(REP, INSN, TAIL)          \
  REP(INSN " %0, %4, %8, %0" TAIL "\n")        \
  REP(INSN " %1, %5, %9, %1" TAIL "\n")        \
  REP(INSN " %2, %6, %10, %2" TAIL "\n")       \
  REP(INSN " %3, %7, %11, %3" TAIL "\n")
// scaled: %12-%15 scale A, %16-%19 scale B
#define MI355_CHAINS_SCALED(REP, INSN, TAIL)                       \
  REP(INSN " %0, %4, %8, %0, %12, %16 op_sel_hi:[0,0,0]" TAIL "\n")   \
  REP(INSN " %1, %5, %9, %1, %13, %17 op_sel_hi:[0,0,0]" TAIL "\n")   \
  REP(INSN " %2, %6, %10, %2, %14, %18 op_sel_hi:[0,0,0]" TAIL "\n")  \
  REP(INSN " %3, %7, %11, %3, %15, %19 op_sel_hi:[0,0,0]" TAIL "\n")
#define MI355_ONCE(x) x

#define MI355_DEFINE_STEPS(INSN, TAIL)                                                             \
  __device__ static void block(Acc (&acc)[4], const Frag (&a)[4], const Frag (&b)[4], const int (&)[4], \
                               const int (&)[4]) {                                                 \
    asm volatile(MI355_CHAINS(MI355_REP32, INSN, TAIL)                                              \
                 : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3])                          \
                 : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(b[0]), "v"(b[1]), "v"(b[2]), "v"(b[3])); \
  }                                                                                                \
  __device__ static void single(Acc (&acc)[4], const Frag (&a)[4], const Frag (&b)[4], const int (&)[4], \
                                const int (&)[4]) {                                                \
    asm volatile(MI355_CHAINS(MI355_ONCE, INSN, TAIL)                                              \
                 : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3])                          \
                 : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(b[0]), "v"(b[1]), "v"(b[2]), "v"(b[3])); \
  }

#define MI355_DEFINE_STEPS_SCALED(INSN, TAIL)                                                      \
  __device__ static void block(Acc (&acc)[4], const Frag (&a)[4], const Frag (&b)[4], const int (&sa)[4], \
                               const int (&sb)[4]) {                                               \
    asm volatile(MI355_CHAINS_SCALED(MI355_REP32, INSN, TAIL)                                       \
                 : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3])                          \
                 : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(b[0]), "v"(b[1]), "v"(b[2]), "v"(b[3]), \
                   "v"(sa[0]), "v"(sa[1]), "v"(sa[2]), "v"(sa[3]), "v"(sb[0]), "v"(sb[1]), "v"(sb[2]), "v"(sb[3])); \
  }                                                                                                \
  __device__ static void single(Acc (&acc)[4], const Frag (&a)[4], const Frag (&b)[4], const int (&sa)[4], \
                                const int (&sb)[4]) {                                              \
    asm volatile(MI355_CHAINS_SCALED(MI355_ONCE, INSN, TAIL)                                       \
                 : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3])                          \
                 : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(b[0]), "v"(b[1]), "v"(b[2]), "v"(b[3]), \
                   "v"(sa[0]), "v"(sa[1]), "v"(sa[2]), "v"(sa[3]), "v"(sb[0]), "v"(sb[1]), "v"(sb[2]), "v"(sb[3])); \
  }

// ---- per-kind traits ---------------------------------------------------------
// Each trait supplies: tile shape, bytes per K-contiguous row, register types, how a
// lane loads its fragment from a logical row, and the instruction blocks.

typedef int i32x6v __attribute__((ext_vector_type(6)));

// A lane's fragment is `bytes` contiguous bytes of its row, starting at chunk * bytes.
template <typename Frag, int ROWS_MOD, int ROW_BYTES, int BYTES>
__device__ inline Frag load_fragment(const uint8_t *rows, int lane) {
  return load_bytes<Frag>(rows + (lane % ROWS_MOD) * ROW_BYTES + (lane / ROWS_MOD) * BYTES);
}

#define MI355_DENSE_TRAIT(NAME, M_, N_, K_, ROW_BYTES, FRAG, ACC, OUT, INSN)                       \
  struct NAME {                                                                                    \
    static constexpr int M = M_, N = N_, K = K_, row_bytes = ROW_BYTES, acc_regs = M_ * N_ / 64;   \
    static constexpr bool scaled = false;                                                          \
    using Frag = FRAG; using Acc = ACC; using Out = OUT;                                           \
    __device__ static Frag load(const uint8_t *rows, int lane) {                                   \
      return load_fragment<Frag, M_, ROW_BYTES, 16>(rows, lane);                                   \
    }                                                                                              \
    MI355_DEFINE_STEPS(INSN, "")                                                                   \
  };

MI355_DENSE_TRAIT(F16_16x16x32, 16, 16, 32, 64, half8v, f32x4v, float, "v_mfma_f32_16x16x32_f16")
MI355_DENSE_TRAIT(BF16_16x16x32, 16, 16, 32, 64, bf16x8v, f32x4v, float, "v_mfma_f32_16x16x32_bf16")
MI355_DENSE_TRAIT(F16_32x32x16, 32, 32, 16, 32, half8v, f32x16v, float, "v_mfma_f32_32x32x16_f16")
MI355_DENSE_TRAIT(BF16_32x32x16, 32, 32, 16, 32, bf16x8v, f32x16v, float, "v_mfma_f32_32x32x16_bf16")
MI355_DENSE_TRAIT(I8_16x16x64, 16, 16, 64, 64, i32x4v, i32x4v, int32_t, "v_mfma_i32_16x16x64_i8")

// f8f6f4, 16x16x128: a lane's 32 elements are BITS*4 bytes in BITS/... registers
// (8 for 8-bit, 6 for 6-bit, 4 for 4-bit codes); cbsz / blgp name the A / B format.
#define MI355_F8F6F4_TRAIT(NAME, BITS, FRAG, SCALED, TAIL)                                         \
  struct NAME {                                                                                    \
    static constexpr int M = 16, N = 16, K = 128, row_bytes = 128 * BITS / 8, acc_regs = 4;        \
    static constexpr bool scaled = SCALED;                                                         \
    using Frag = FRAG; using Acc = f32x4v; using Out = float;                                      \
    __device__ static Frag load(const uint8_t *rows, int lane) {                                   \
      if constexpr (BITS == 8) { /* K elements [16g,+16) then [64+16g,+16), g = lane/16 */         \
        const uint8_t *p = rows + (lane % 16) * row_bytes + (lane / 16) * 16;                      \
        const i32x4v lo = load_bytes<i32x4v>(p), hi = load_bytes<i32x4v>(p + 64);                  \
        const i32x8v both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};              \
        Frag f;                                                                                    \
        __builtin_memcpy(&f, &both, sizeof(f)); /* Frag is i32x8v on this branch */                \
        return f;                                                                                  \
      } else {                                                                                     \
        return load_fragment<Frag, 16, row_bytes, BITS * 4>(rows, lane);                           \
      }                                                                                            \
    }                                                                                              \
    MI355_DEFINE_STEPS_SCALED("v_mfma_scale_f32_16x16x128_f8f6f4", TAIL)                           \
  };

MI355_F8F6F4_TRAIT(FP8_16x16x128, 8, i32x8v, false, "")
MI355_F8F6F4_TRAIT(BF8_16x16x128, 8, i32x8v, false, " cbsz:1 blgp:1")
MI355_F8F6F4_TRAIT(FP6_E2M3_16x16x128, 6, i32x6v, true, " cbsz:2 blgp:2")
MI355_F8F6F4_TRAIT(FP6_E3M2_16x16x128, 6, i32x6v, true, " cbsz:3 blgp:3")
MI355_F8F6F4_TRAIT(FP4_E2M1_16x16x128, 4, i32x4v, true, " cbsz:4 blgp:4")

template <typename Tr, bool ONE_SET>
__global__ void __launch_bounds__(256)
mfma_dense_kernel(const uint8_t *__restrict__ A, const uint8_t *__restrict__ B,
                  const uint8_t *__restrict__ sA, const uint8_t *__restrict__ sB,
                  typename Tr::Out *__restrict__ out, uint32_t iters, uint64_t *__restrict__ clocks, uint32_t active) {
  // diagnosis: only the workgroups of some XCDs (index mod 8) or of half the CUs of every XCD take part
  if (!((active >> (blockIdx.x % 8u)) & 1u) || ((active & 0x100u) && (blockIdx.x / 8u) % 32u >= 16u)) return;
  const int lane = threadIdx.x % 64;
  const uint64_t wave = (uint64_t)blockIdx.x * (blockDim.x / 64) + threadIdx.x / 64;
  constexpr size_t a_bytes = (size_t)Tr::M * Tr::row_bytes, b_bytes = (size_t)Tr::N * Tr::row_bytes;

  typename Tr::Frag a[kChains], b[kChains];
  typename Tr::Acc acc[kChains];
  int sa[kChains], sb[kChains];
#pragma unroll
  for (int c = 0; c < kChains; c++) {
#pragma unroll
    for (int r = 0; r < Tr::acc_regs; r++) acc[c][r] = 0;
    if (ONE_SET && c > 0) {   // the very registers of chain 0, not copies of their contents
      a[c] = a[0]; b[c] = b[0]; sa[c] = sa[0]; sb[c] = sb[0];
      continue;
    }
    const uint64_t u = wave * kChains + c;
    a[c] = Tr::load(A + u * a_bytes, lane);
    b[c] = Tr::load(B + u * b_bytes, lane);
    if constexpr (Tr::scaled) {
      // scale[wave][chain][row][K/32]: this lane's row (lane%16) and K block (lane/16).
      sa[c] = sA[(u * Tr::M + lane % 16) * (Tr::K / 32) + lane / 16];
      sb[c] = sB[(u * Tr::N + lane % 16) * (Tr::K / 32) + lane / 16];
    } else {
      sa[c] = 0x7f;  // E8M0 1.0
      sb[c] = 0x7f;
    }
  }

  const uint32_t blocks = iters / kBlock, rest = iters % kBlock;
  const uint64_t t0 = clock64(), r0 = wall_clock64();
#pragma unroll 1
  for (uint32_t it = 0; it < blocks; it++) Tr::block(acc, a, b, sa, sb);
#pragma unroll 1
  for (uint32_t it = 0; it < rest; it++) Tr::single(acc, a, b, sa, sb);
  // The compiler cannot see the matrix instructions inside the asm blocks, so it will
  // not insert the wait states a VALU/VMEM read of their results needs: cover the
  // longest case (a 16-pass MFMA result read by a store) by hand.
  asm volatile("s_nop 15\n s_nop 15" ::: "memory");
  if (clocks != nullptr && wave == 0 && lane == 0) {
    clocks[0] = clock64() - t0;
    clocks[1] = wall_clock64() - r0;
  }

#pragma unroll
  for (int c = 0; c < kChains; c++) {
    typename Tr::Out *tile = out + (wave * kChains + c) * (uint64_t)(Tr::M * Tr::N);
    if constexpr (Tr::M == 16) {
#pragma unroll
      for (int r = 0; r < 4; r++) tile[(4 * (lane / 16) + r) * 16 + lane % 16] = acc[c][r];
    } else {
#pragma unroll
      for (int r = 0; r < 16; r++) tile[(8 * (r / 4) + 4 * (lane / 32) + r % 4) * 32 + lane % 32] = acc[c][r];
    }
  }
}

template <typename Tr>
int launch(mi355_dev *dev, bool one_set, const void *A, const void *B, const uint8_t *sA, const uint8_t *sB, void *out,
           uint32_t waves, uint32_t iters, uint64_t *clocks, uint32_t active) {
  if (Tr::scaled && (!sA || !sB)) return mi355_fail(dev, MI355_ERR_ARG, "mfma_dense: scaled kind needs scaleA and scaleB");
  if (one_set)
    mfma_dense_kernel<Tr, true><<<waves / 4, 256, 0, dev->stream>>>((const uint8_t *)A, (const uint8_t *)B, sA, sB,
                                                                   (typename Tr::Out *)out, iters, clocks, active);
  else
    mfma_dense_kernel<Tr, false><<<waves / 4, 256, 0, dev->stream>>>((const uint8_t *)A, (const uint8_t *)B, sA, sB,
                                                                    (typename Tr::Out *)out, iters, clocks, active);
  MI355_LAUNCH_CHECK(dev, "mfma_dense");
  return MI355_OK;
}

}  // namespace

extern "C" int mi355_mfma_dense(mi355_dev *dev, int kind, const void *A, const void *B, const uint8_t *scaleA,
                                const uint8_t *scaleB, void *out, uint32_t waves, uint32_t iters, uint64_t *clocks) {
  MI355_ENTER(dev);
  MI355_REQUIRE(dev, A && B && out, "mfma_dense: null buffer");
  MI355_REQUIRE(dev, waves > 0 && waves % 4 == 0, "mfma_dense: waves (%u) must be a positive multiple of 4", waves);
  MI355_REQUIRE(dev, (((uintptr_t)A | (uintptr_t)B | (uintptr_t)out) & 15u) == 0, "mfma_dense: buffers must be 16-byte aligned");
  const bool one_set = (kind & MI355_MFMA_ONE_OPERAND_SET) != 0;
  uint32_t active = ((uint32_t)kind >> 16) & 0xffu;   // MI355_MATRIX_ON_XCDS: 0 = every XCD
  if (active == 0u) active = 0xffu;
  MI355_REQUIRE(dev, (active & 1u) != 0u, "mfma_dense: XCD 0 must be among the XCDs that take part (its first wave reads the clocks)");
  if (kind & MI355_MATRIX_ON_HALF_THE_CUS) active |= 0x100u;
  kind &= 0xff;
  switch (kind) {
    case MI355_MFMA_F16_16x16x32:  return launch<F16_16x16x32>(dev, one_set, A, B, scaleA, scaleB, out, waves, iters, clocks, active);
    case MI355_MFMA_BF16_16x16x32: return launch<BF16_16x16x32>(dev, one_set, A, B, scaleA, scaleB, out, waves, iters, clocks, active);
    case MI355_MFMA_F16_32x32x16:  return launch<F16_32x32x16>(dev, one_set, A, B, scaleA, scaleB, out, waves, iters, clocks, active);
    case MI355_MFMA_BF16_32x32x16: return launch<BF16_32x32x16>(dev, one_set, A, B, scaleA, scaleB, out, waves, iters, clocks, active);
    case MI355_MFMA_I8_16x16x64:   return launch<I8_16x16x64>(dev, one_set, A, B, scaleA, scaleB, out, waves, iters, clocks, active);
    case MI355_MFMA_FP8_16x16x128: return launch<FP8_16x16x128>(dev, one_set, A, B, scaleA, scaleB, out, waves, iters, clocks, active);
    case MI355_MFMA_BF8_16x16x128: return launch<BF8_16x16x128>(dev, one_set, A, B, scaleA, scaleB, out, waves, iters, clocks, active);
    case MI355_MFMA_MXFP6_E2M3:    return launch<FP6_E2M3_16x16x128>(dev, one_set, A, B, scaleA, scaleB, out, waves, iters, clocks, active);
    case MI355_MFMA_MXFP6_E3M2:    return launch<FP6_E3M2_16x16x128>(dev, one_set, A, B, scaleA, scaleB, out, waves, iters, clocks, active);
    case MI355_MFMA_MXFP4_E2M1:    return launch<FP4_E2M1_16x16x128>(dev, one_set, A, B, scaleA, scaleB, out, waves, iters, clocks, active);
    default: return mi355_fail(dev, MI355_ERR_ARG, "mfma_dense: unknown kind %d", kind);
  }
}
