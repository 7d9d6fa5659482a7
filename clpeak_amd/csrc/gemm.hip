// Hand-written MFMA GEMM:  C[M][N] (bf16) = scale * A[M][K] . B[N][K]^T, fp32 accumulate.
// Both operands are K-contiguous ("row-major A, column-major B").
//
// Tiling.  One workgroup of 512 threads (8 waves, 2 per SIMD) owns a 256x256 tile
// of C and walks K in steps of one 128-byte row segment (64 bf16 or 128 fp8
// elements).  The A and B slabs of a step (256 rows x 128 B each) live in LDS,
// double buffered: 2 x 64 KiB of the CU's 160 KiB.  While the MFMAs consume slab s,
// the global loads of slab s+1 are already in flight into registers and are written
// to the other LDS buffer before the single barrier that ends the step.
//
// Waves form a 2 (M) x 4 (N) grid; each wave owns 128x64 of C = 8x4 MFMA tiles of
// 16x16, 128 fp32 accumulators per lane.
//
// LDS layout.  A row's 128 bytes are eight 16-byte chunks; chunk c of row r is stored
// at chunk position c ^ (r & 7).  A fragment read (16 lanes = 16 consecutive rows,
// same logical chunk) then spreads over all eight chunk positions instead of hitting
// one bank group 16 times.
//
// Workgroup -> tile mapping.  Workgroups are dealt round-robin to the 8 XCDs, each
// with its own L2.  The mapping hands every XCD a contiguous band of tile rows, so
// the A rows a band needs are fetched into one L2 only, and walks each band in
// column-major order of 4-row groups so that B slabs are reused while still hot.
#include "internal.h"
#include "mfma_common.h"
#include "numeric_formats.h"

namespace {

constexpr int kTile = 256;        // C tile edge
constexpr int kRowBytes = 128;    // bytes of K per step, per row
constexpr int kThreads = 512;
constexpr int kSlabBytes = kTile * kRowBytes;           // 32 KiB per operand per step
constexpr int kChunksPerThread = kSlabBytes / 16 / kThreads;  // 4

__device__ inline uint32_t swizzled(uint32_t row, uint32_t chunk) {
  return row * kRowBytes + ((chunk ^ (row & 7u)) << 4);
}

template <bool kFp8>
__global__ void __launch_bounds__(kThreads)
gemm_kernel(const uint8_t *__restrict__ A, const uint8_t *__restrict__ B, uint16_t *__restrict__ C,
            uint32_t M, uint32_t N, uint32_t k_bytes, float scale, uint32_t tiles_m, uint32_t tiles_n) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  // [buffer][operand][kSlabBytes]
  const uint32_t tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const uint32_t wm = wave / 4, wn = wave % 4;

  // --- workgroup -> tile ------------------------------------------------------
  uint32_t tm, tn;
  {
    const uint32_t bid = blockIdx.x, total = tiles_m * tiles_n;
    const uint32_t xcd = bid % 8u, slot = bid / 8u;
    const uint32_t per_xcd = (total + 7u) / 8u;
    uint32_t lin = xcd * per_xcd + slot;           // tiles of one XCD are consecutive
    if (total % 8u != 0u) lin = bid;               // ragged grids: plain order
    // consecutive tiles walk down a group of 4 tile rows, then move one column right
    const uint32_t group = lin / (4u * tiles_n), in_group = lin % (4u * tiles_n);
    const uint32_t rows_here = (tiles_m - group * 4u) < 4u ? (tiles_m - group * 4u) : 4u;
    tm = group * 4u + in_group % rows_here;
    tn = in_group / rows_here;
  }

  const uint8_t *a_tile = A + (size_t)tm * kTile * k_bytes;
  const uint8_t *b_tile = B + (size_t)tn * kTile * k_bytes;

  f32x4v acc[8][4];
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = (f32x4v){0.f, 0.f, 0.f, 0.f};

  // chunk q of a slab: row q/8, chunk q%8; this thread moves q = tid + 512*i
  i32x4v stage_a[kChunksPerThread], stage_b[kChunksPerThread];
  auto global_fetch = [&](uint32_t kb) {
#pragma unroll
    for (int i = 0; i < kChunksPerThread; i++) {
      const uint32_t q = tid + kThreads * i, row = q / 8u, c = q % 8u;
      stage_a[i] = *reinterpret_cast<const i32x4v *>(a_tile + (size_t)row * k_bytes + kb + c * 16u);
      stage_b[i] = *reinterpret_cast<const i32x4v *>(b_tile + (size_t)row * k_bytes + kb + c * 16u);
    }
  };
  auto lds_commit = [&](uint32_t buf) {
    uint8_t *sa = lds + (size_t)buf * 2 * kSlabBytes, *sb = sa + kSlabBytes;
#pragma unroll
    for (int i = 0; i < kChunksPerThread; i++) {
      const uint32_t q = tid + kThreads * i, row = q / 8u, c = q % 8u;
      *reinterpret_cast<i32x4v *>(sa + swizzled(row, c)) = stage_a[i];
      *reinterpret_cast<i32x4v *>(sb + swizzled(row, c)) = stage_b[i];
    }
  };

  const uint32_t steps = k_bytes / kRowBytes;
  global_fetch(0);
  lds_commit(0);
  __syncthreads();

  for (uint32_t s = 0; s < steps; s++) {
    const uint32_t buf = s & 1u;
    if (s + 1 < steps) global_fetch((s + 1) * kRowBytes);

    const uint8_t *sa = lds + (size_t)buf * 2 * kSlabBytes + (size_t)wm * 128 * kRowBytes;
    const uint8_t *sb = lds + (size_t)buf * 2 * kSlabBytes + kSlabBytes + (size_t)wn * 64 * kRowBytes;
    if constexpr (!kFp8) {
#pragma unroll
      for (int ks = 0; ks < 2; ks++) {  // two K=32 MFMA steps per 64-element slab
        bf16x8v af[8], bf[4];
        const uint32_t c = ks * 4u + lane / 16u;
#pragma unroll
        for (int i = 0; i < 8; i++) af[i] = *reinterpret_cast<const bf16x8v *>(sa + swizzled(i * 16u + lane % 16u, c));
#pragma unroll
        for (int j = 0; j < 4; j++) bf[j] = *reinterpret_cast<const bf16x8v *>(sb + swizzled(j * 16u + lane % 16u, c));
#pragma unroll
        for (int i = 0; i < 8; i++)
#pragma unroll
          for (int j = 0; j < 4; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], bf[j], acc[i][j], 0, 0, 0);
      }
    } else {
      // one K=128 MFMA step per slab: a lane's 32 codes are logical chunks 2*(lane/16), +1
      i32x8v bf[4];
      const uint32_t c0 = 2u * (lane / 16u);
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const uint32_t row = j * 16u + lane % 16u;
        const i32x4v lo = *reinterpret_cast<const i32x4v *>(sb + swizzled(row, c0));
        const i32x4v hi = *reinterpret_cast<const i32x4v *>(sb + swizzled(row, c0 + 1u));
        bf[j] = (i32x8v){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const uint32_t row = i * 16u + lane % 16u;
        const i32x4v lo = *reinterpret_cast<const i32x4v *>(sa + swizzled(row, c0));
        const i32x4v hi = *reinterpret_cast<const i32x4v *>(sa + swizzled(row, c0 + 1u));
        const i32x8v af = (i32x8v){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
#pragma unroll
        for (int j = 0; j < 4; j++)
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(af, bf[j], acc[i][j], MI355_F8F6F4_E4M3,
                                                                         MI355_F8F6F4_E4M3, 0, 0x7f, 0, 0x7f);
      }
    }

    if (s + 1 < steps) lds_commit(buf ^ 1u);
    __syncthreads();
  }

  // --- epilogue: scale, round to bf16, store ---------------------------------------
  const uint32_t row0 = tm * kTile + wm * 128u, col0 = tn * kTile + wn * 64u;
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const uint32_t row = row0 + i * 16u + 4u * (lane / 16u) + r, col = col0 + j * 16u + lane % 16u;
        C[(size_t)row * N + col] = mi355_f32_to_bf16(acc[i][j][r] * scale);
      }
  (void)M;
}

template <bool kFp8>
int launch(mi355_dev *dev, const void *A, const void *B, uint16_t *C, uint32_t M, uint32_t N, uint32_t K,
           float scale) {
  const uint32_t elem = kFp8 ? 1u : 2u;
  MI355_REQUIRE(dev, A && B && C, "gemm: null buffer");
  MI355_REQUIRE(dev, M > 0 && N > 0 && K > 0, "gemm: empty problem");
  MI355_REQUIRE(dev, M % kTile == 0 && N % kTile == 0, "gemm: M (%u) and N (%u) must be multiples of 256", M, N);
  MI355_REQUIRE(dev, (K * elem) % kRowBytes == 0, "gemm: K (%u) must be a multiple of %u", K, kRowBytes / elem);
  MI355_REQUIRE(dev, (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15u) == 0, "gemm: buffers must be 16-byte aligned");
  const uint32_t tiles_m = M / kTile, tiles_n = N / kTile;
  const size_t lds_bytes = 4 * (size_t)kSlabBytes;  // 128 KiB
  static bool attr_set[2] = {false, false};
  if (!attr_set[kFp8]) {
    MI355_HIP(dev, hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_kernel<kFp8>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
    attr_set[kFp8] = true;
  }
  gemm_kernel<kFp8><<<tiles_m * tiles_n, kThreads, lds_bytes, dev->stream>>>(
      (const uint8_t *)A, (const uint8_t *)B, C, M, N, K * elem, scale, tiles_m, tiles_n);
  MI355_LAUNCH_CHECK(dev, "gemm");
  return MI355_OK;
}

}  // namespace

extern "C" int mi355_gemm_bf16(mi355_dev *dev, const uint16_t *A, const uint16_t *B, uint16_t *C, uint32_t M,
                               uint32_t N, uint32_t K) {
  MI355_ENTER(dev);
  return launch<false>(dev, A, B, C, M, N, K, 1.0f);
}

extern "C" int mi355_gemm_fp8_e4m3(mi355_dev *dev, const uint8_t *A, const uint8_t *B, uint16_t *C, uint32_t M,
                                   uint32_t N, uint32_t K, float scale_a, float scale_b) {
  MI355_ENTER(dev);
  return launch<true>(dev, A, B, C, M, N, K, scale_a * scale_b);
}
