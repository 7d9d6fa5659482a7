// Vector multiply-add throughput kernels (VALU, register resident).
//
// Every work-item holds 16 independent accumulators and advances each of them by
// `steps` dependent multiply-adds, so a lane always has 16 FMAs in flight and the
// chain latency is hidden without relying on occupancy.  Seeds come from the
// counter generator (stream MI355_STREAM_MAD, element item*16 + j), nothing is read
// from memory, and the only store is the per-item sum of the 16 accumulators.
//
// The `width` variants (x, x2, x4) group the same 16 accumulators into vectors of
// 1, 2 or 4 lanes; the arithmetic per accumulator is identical, so all widths of
// one kind produce identical results.
#include "internal.h"
#include "seeded_rng.h"
#include "numeric_formats.h"

namespace {

constexpr int kAcc = 16;

typedef _Float16 half2v __attribute__((ext_vector_type(2)));

__device__ inline _Float16 bits_to_half(uint16_t h) {
  _Float16 r;
  __builtin_memcpy(&r, &h, 2);
  return r;
}

// ---- fp32 / fp64 -----------------------------------------------------------
template <typename T, int W>
__global__ void __launch_bounds__(256)
mad_fp_kernel(uint64_t seed, uint32_t steps, uint64_t n_items, T *__restrict__ out) {
  const uint64_t item = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (item >= n_items) return;
  // W accumulators form one vector of the reference's source (float2, double4, ...).  A lane of this machine
  // holds a vector as W separate registers, so the vectors are written as what they are: element l of vector v
  // is accumulator v*W + l.  (As ext_vector_type values the double2 / double4 chains picked up two register
  // copies per 32 multiply-adds from the allocator and ran 6 % below the scalar ones.)
  constexpr int NV = kAcc / W;
  // The multiplier of the workload is a compile-time constant because what a 32-bit vector instruction reads
  // decides its rate.  As a kernel argument it sat in a scalar register (uniform over the lanes) and v_fma_f32
  // ran at the 4-cycle rate, 75.7 TFLOP/s; from a vector register (three vector reads) 119; as the literal of
  // v_fmamk_f32 (two vector reads) 127-130.  fp64 is the other way round: the constant lands in a scalar
  // register pair, 72.9 TFLOP/s, against 66.9 from vector registers.
  constexpr T a = (T)1.0001;
  T x0[kAcc], x[kAcc];
#pragma unroll
  for (int i = 0; i < kAcc; i++) {
    x0[i] = (T)mi355_rng_upm1(mi355_rng_word(seed, MI355_STREAM_MAD, item * kAcc + i));
    x[i] = x0[i];
  }
#pragma unroll 8   // at one instruction per two cycles the counter and branch of a short trip show: +4 % over 2
  for (uint32_t s = 0; s < steps; s++) {
#pragma unroll
    for (int v = 0; v < NV; v++)
#pragma unroll
      for (int l = 0; l < W; l++)
        x[v * W + l] = __builtin_elementwise_fma(x[v * W + l], a, x0[v * W + l]);   // typed by its operands
  }
  T sum = (T)0;
#pragma unroll
  for (int i = 0; i < kAcc; i++) sum += x[i];
  out[item] = sum;
}

// ---- fp16: width 1 scalar half FMA, width 2 packed half2 FMA ---------------------
template <int W>
__global__ void __launch_bounds__(256)
mad_f16_kernel(uint64_t seed, uint16_t a_bits, uint32_t steps, uint64_t n_items, uint16_t *__restrict__ out) {
  const uint64_t item = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (item >= n_items) return;
  const _Float16 a = bits_to_half(a_bits);   // 0x3bfe (the scalar form below carries it as a literal)
  _Float16 sum = (_Float16)0;
  if constexpr (W == 1) {
    // One scalar half multiply-add per step and accumulator, as the reference's scalar row (its __hfma chains,
    // src/rocm/rocm_kernels/compute_hp.hip:12-30).  Written as the instruction itself, on 32-bit registers
    // that hold a half in their low 16 bits: from the plain expression the compiler pairs neighbouring chains
    // into v_pk_fma_f16 and the row becomes the half2 row.  The arithmetic is the same correctly rounded half
    // FMA either way.
    uint32_t x0[kAcc], x[kAcc];
#pragma unroll
    for (int j = 0; j < kAcc; j++) {
      x0[j] = mi355_f32_to_f16(mi355_rng_upm1(mi355_rng_word(seed, MI355_STREAM_MAD, item * kAcc + j)));
      x[j] = x0[j];
    }
    // (v_fma_f16 issues once per 8 cycles and SIMD on this part, with the multiplier in a vector or in a scalar register
    // alike: 38.5 TFLOP/s where the packed form, two lanes per instruction every 4 cycles, reaches 147.)
    uint32_t a32 = a_bits;
    asm volatile("" : "+v"(a32));
#define MI355_HALF_STEP(j) asm volatile("v_fma_f16 %0, %0, %1, %2" : "+v"(x[j]) : "v"(a32), "v"(x0[j]))
    for (uint32_t b = 0; b < steps / 8; b++) {   // 128 instructions per trip: the branch of a shorter one shows
#pragma unroll
      for (int t = 0; t < 8; t++)
#pragma unroll
        for (int j = 0; j < kAcc; j++) MI355_HALF_STEP(j);
    }
    for (uint32_t r = 0; r < steps % 8; r++)
#pragma unroll
      for (int j = 0; j < kAcc; j++) MI355_HALF_STEP(j);
#undef MI355_HALF_STEP
#pragma unroll
    for (int j = 0; j < kAcc; j++) sum += bits_to_half((uint16_t)x[j]);
  } else {
    half2v x0[kAcc / 2], x[kAcc / 2];
    const half2v av = {a, a};
#pragma unroll
    for (int v = 0; v < kAcc / 2; v++) {
#pragma unroll
      for (int l = 0; l < 2; l++)
        x0[v][l] = bits_to_half(mi355_f32_to_f16(mi355_rng_upm1(mi355_rng_word(seed, MI355_STREAM_MAD, item * kAcc + v * 2 + l))));
      x[v] = x0[v];
    }
#pragma unroll 2
    for (uint32_t s = 0; s < steps; s++) {
#pragma unroll
      for (int v = 0; v < kAcc / 2; v++) x[v] = __builtin_elementwise_fma(x[v], av, x0[v]);
    }
#pragma unroll
    for (int v = 0; v < kAcc / 2; v++) {
      sum += x[v][0];
      sum += x[v][1];
    }
  }
  uint16_t bits;
  __builtin_memcpy(&bits, &sum, 2);
  out[item] = bits;
}

// ---- narrow operands, fp32 accumulator ---------------------------------------------------------------------
// Both kernels keep the narrow operands live inside the chain and run on the instruction the hardware has for
// "narrow x narrow + fp32": the reference's kernels are fp32 chains that pass the running value through the
// narrow type once per block (src/rocm/rocm_kernels/compute_mp.hip:18-23, compute_bf16.hip:26-31), and so are
// these, with the narrow sources read by the multiply-add itself.
//
// mp (half):  x <- fma(x, a, x0), x in fp32, a and x0 IEEE half in registers, widened by v_fma_mix_f32 on every
//             step (exact), one fused rounding to fp32; after every 16th step x <- float(half(x)) (round to
//             nearest even) and the next step reads that half directly.  a = 1 - 2^-10 (0x3bfe), x0 = half(u),
//             x starts at x0.  2 flop per step.
// bf16:       acc <- acc + xb * ab + x0b * 1, one v_dot2_f32_bf16 per step (packed sources (xb, x0b) and
//             (ab, 1.0), fp32 accumulator; 4 flop); after every 128th step xb <- bf16(acc) (round to nearest
//             even).  ab = -2^-8 (0xbb80), x0b = bf16(u), xb and acc start at x0b.
#define MI355_FMA_MIX_F32(x, a_h, x0_h) \
  asm volatile("v_fma_mix_f32 %0, %0, %1, %2 op_sel_hi:[0,1,1]" : "+v"(x) : "v"(a_h), "v"(x0_h))
// first step after a round trip: the chain value itself is the half in the low 16 bits of xh
#define MI355_FMA_MIX_F32_FROM_HALF(x, xh, a_h, x0_h) \
  asm volatile("v_fma_mix_f32 %0, %1, %2, %3 op_sel_hi:[1,1,1]" : "=v"(x) : "v"(xh), "v"(a_h), "v"(x0_h))
#define MI355_DOT2_F32_BF16(acc, a_pair, b_pair) \
  asm volatile("v_dot2_f32_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a_pair), "v"(b_pair))

constexpr uint32_t kMpBlock = 16, kBf16Block = 128;

__global__ void __launch_bounds__(256)
mad_mp_kernel(uint64_t seed, uint32_t steps, uint64_t n_items, float *__restrict__ out) {
  const uint64_t item = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (item >= n_items) return;
  uint32_t x0h[kAcc];   // half bits in the low 16
  float x[kAcc];
  uint32_t a_h = 0x3bfeu;
  asm volatile("" : "+v"(a_h));   // a vector register, not a literal: the mixed form takes no 16-bit literal
#pragma unroll
  for (int j = 0; j < kAcc; j++) {
    x0h[j] = mi355_f32_to_f16(mi355_rng_upm1(mi355_rng_word(seed, MI355_STREAM_MAD, item * kAcc + j)));
    x[j] = (float)bits_to_half((uint16_t)x0h[j]);
  }
  const uint32_t blocks = steps / kMpBlock, rem = steps % kMpBlock;
  uint32_t xh[kAcc];
  bool from_half = false;
  for (uint32_t b = 0; b < blocks; b++) {
    if (from_half) {
#pragma unroll
      for (int j = 0; j < kAcc; j++) MI355_FMA_MIX_F32_FROM_HALF(x[j], xh[j], a_h, x0h[j]);
    } else {
#pragma unroll
      for (int j = 0; j < kAcc; j++) MI355_FMA_MIX_F32(x[j], a_h, x0h[j]);
    }
#pragma unroll
    for (uint32_t t = 1; t < kMpBlock; t++)
#pragma unroll
      for (int j = 0; j < kAcc; j++) MI355_FMA_MIX_F32(x[j], a_h, x0h[j]);
#pragma unroll
    for (int j = 0; j < kAcc; j++) {
      const _Float16 h = (_Float16)x[j];   // v_cvt_f16_f32, round to nearest even
      uint16_t bits;
      __builtin_memcpy(&bits, &h, 2);
      xh[j] = bits;
      x[j] = (float)h;                     // what the chain holds if no further step follows
    }
    from_half = true;
  }
  for (uint32_t r = 0; r < rem; r++)
#pragma unroll
    for (int j = 0; j < kAcc; j++) MI355_FMA_MIX_F32(x[j], a_h, x0h[j]);
  float sum = 0.0f;
#pragma unroll
  for (int j = 0; j < kAcc; j++) sum += x[j];
  out[item] = sum;
}

__global__ void __launch_bounds__(256)
mad_bf16_kernel(uint64_t seed, uint32_t steps, uint64_t n_items, float *__restrict__ out) {
  const uint64_t item = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (item >= n_items) return;
  uint32_t pair[kAcc];   // low half: xb, high half: x0b
  float acc[kAcc];
  uint32_t b_pair = 0x3f80bb80u;   // low half ab = -2^-8, high half 1.0
  asm volatile("" : "+v"(b_pair));
#pragma unroll
  for (int j = 0; j < kAcc; j++) {
    const uint32_t x0b = mi355_f32_to_bf16(mi355_rng_upm1(mi355_rng_word(seed, MI355_STREAM_MAD, item * kAcc + j)));
    pair[j] = x0b | (x0b << 16);
    acc[j] = mi355_bf16_to_f32((uint16_t)x0b);
  }
  const uint32_t blocks = steps / kBf16Block, rem = steps % kBf16Block;
  for (uint32_t b = 0; b < blocks; b++) {
    for (uint32_t t8 = 0; t8 < kBf16Block / 16; t8++) {
#pragma unroll
      for (uint32_t t = 0; t < 16; t++)
#pragma unroll
        for (int j = 0; j < kAcc; j++) MI355_DOT2_F32_BF16(acc[j], pair[j], b_pair);
    }
#pragma unroll
    for (int j = 0; j < kAcc; j++)   // xb <- bf16(acc), round to nearest even; x0b stays
      pair[j] = (uint32_t)mi355_f32_to_bf16(acc[j]) | (pair[j] & 0xffff0000u);
  }
  for (uint32_t r = 0; r < rem; r++)
#pragma unroll
    for (int j = 0; j < kAcc; j++) MI355_DOT2_F32_BF16(acc[j], pair[j], b_pair);
  float sum = 0.0f;
#pragma unroll
  for (int j = 0; j < kAcc; j++) sum += acc[j];
  out[item] = sum;
}

// ---- int32: x = x*a + x0, wrapping --------------------------------------------
template <int W>
__global__ void __launch_bounds__(256)
mad_i32_kernel(uint64_t seed, uint32_t a, uint32_t steps, uint64_t n_items, uint32_t *__restrict__ out) {
  const uint64_t item = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (item >= n_items) return;
  uint32_t x0[kAcc], x[kAcc];
#pragma unroll
  for (int j = 0; j < kAcc; j++) {
    x0[j] = (uint32_t)(mi355_rng_word(seed, MI355_STREAM_MAD, item * kAcc + j) >> 32);
    x[j] = x0[j];
  }
#pragma unroll 2
  for (uint32_t s = 0; s < steps; s++) {
#pragma unroll
    for (int j = 0; j < kAcc; j++) x[j] = x[j] * a + x0[j];
  }
  uint32_t sum = 0;
#pragma unroll
  for (int j = 0; j < kAcc; j++) sum += x[j];
  out[item] = sum;
}

// ---- int8 dot product: acc = sdot4(x, y, acc); y ^= acc; C independent chains -----
template <int C>
__global__ void __launch_bounds__(256)
mad_i8dp_kernel(uint64_t seed, uint32_t steps, uint64_t n_items, int32_t *__restrict__ out) {
  const uint64_t item = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (item >= n_items) return;
  int32_t x[C], y[C], acc[C];
#pragma unroll
  for (int c = 0; c < C; c++) {
    x[c] = (int32_t)(uint32_t)(mi355_rng_word(seed, MI355_STREAM_MAD, item * 8 + c) >> 32);
    y[c] = (int32_t)(uint32_t)(mi355_rng_word(seed, MI355_STREAM_MAD_Y, item * 8 + c) >> 32);
    acc[c] = 0;
  }
#pragma unroll 4
  for (uint32_t s = 0; s < steps; s++) {
#pragma unroll
    for (int c = 0; c < C; c++) {
      acc[c] = __builtin_amdgcn_sdot4(x[c], y[c], acc[c], false);
      y[c] ^= acc[c];
    }
  }
  uint32_t sum = 0;
#pragma unroll
  for (int c = 0; c < C; c++) sum += (uint32_t)acc[c];
  out[item] = (int32_t)sum;
}

}  // namespace

extern "C" int mi355_compute_mad(mi355_dev *dev, int kind, int width, uint64_t seed, uint64_t n_items,
                                 uint32_t steps, void *out, uint32_t block_size) {
  MI355_ENTER(dev);
  MI355_REQUIRE(dev, out != nullptr, "compute_mad: null output");
  MI355_REQUIRE(dev, n_items > 0, "compute_mad: zero items");
  MI355_REQUIRE(dev, block_size == 64 || block_size == 128 || block_size == 256,
                "compute_mad: block_size %u not in {64,128,256}", block_size);
  const uint64_t blocks64 = (n_items + block_size - 1) / block_size;
  MI355_REQUIRE(dev, blocks64 <= 0x7fffffffull, "compute_mad: too many items");
  const dim3 grid((uint32_t)blocks64), block(block_size);
  hipStream_t st = dev->stream;
#define BAD_WIDTH() return mi355_fail(dev, MI355_ERR_ARG, "compute_mad: width %d not valid for kind %d", width, kind)
  switch (kind) {
    case MI355_MAD_F32:
      if (width == 1) mad_fp_kernel<float, 1><<<grid, block, 0, st>>>(seed, steps, n_items, (float *)out);
      else if (width == 2) mad_fp_kernel<float, 2><<<grid, block, 0, st>>>(seed, steps, n_items, (float *)out);
      else if (width == 4) mad_fp_kernel<float, 4><<<grid, block, 0, st>>>(seed, steps, n_items, (float *)out);
      else BAD_WIDTH();
      break;
    case MI355_MAD_F64:
      if (width == 1) mad_fp_kernel<double, 1><<<grid, block, 0, st>>>(seed, steps, n_items, (double *)out);
      else if (width == 2) mad_fp_kernel<double, 2><<<grid, block, 0, st>>>(seed, steps, n_items, (double *)out);
      else if (width == 4) mad_fp_kernel<double, 4><<<grid, block, 0, st>>>(seed, steps, n_items, (double *)out);
      else BAD_WIDTH();
      break;
    case MI355_MAD_F16:  // a = 1 - 2^-10 (0x3bfe): 1.0001 itself rounds to 1.0 in half
      if (width == 1) mad_f16_kernel<1><<<grid, block, 0, st>>>(seed, 0x3bfe, steps, n_items, (uint16_t *)out);
      else if (width == 2) mad_f16_kernel<2><<<grid, block, 0, st>>>(seed, 0x3bfe, steps, n_items, (uint16_t *)out);
      else BAD_WIDTH();
      break;
    case MI355_MAD_MP:
      if (width != 1) BAD_WIDTH();
      mad_mp_kernel<<<grid, block, 0, st>>>(seed, steps, n_items, (float *)out);
      break;
    case MI355_MAD_BF16:
      if (width != 1) BAD_WIDTH();
      mad_bf16_kernel<<<grid, block, 0, st>>>(seed, steps, n_items, (float *)out);
      break;
    case MI355_MAD_I32:
      if (width == 1) mad_i32_kernel<1><<<grid, block, 0, st>>>(seed, 3u, steps, n_items, (uint32_t *)out);
      else if (width == 2) mad_i32_kernel<2><<<grid, block, 0, st>>>(seed, 3u, steps, n_items, (uint32_t *)out);
      else if (width == 4) mad_i32_kernel<4><<<grid, block, 0, st>>>(seed, 3u, steps, n_items, (uint32_t *)out);
      else BAD_WIDTH();
      break;
    case MI355_MAD_I8DP:
      if (width == 1) mad_i8dp_kernel<1><<<grid, block, 0, st>>>(seed, steps, n_items, (int32_t *)out);
      else if (width == 2) mad_i8dp_kernel<2><<<grid, block, 0, st>>>(seed, steps, n_items, (int32_t *)out);
      else if (width == 4) mad_i8dp_kernel<4><<<grid, block, 0, st>>>(seed, steps, n_items, (int32_t *)out);
      else if (width == 8) mad_i8dp_kernel<8><<<grid, block, 0, st>>>(seed, steps, n_items, (int32_t *)out);
      else BAD_WIDTH();
      break;
    default:
      return mi355_fail(dev, MI355_ERR_ARG, "compute_mad: unknown kind %d", kind);
  }
#undef BAD_WIDTH
  MI355_LAUNCH_CHECK(dev, "compute_mad");
  return MI355_OK;
}
