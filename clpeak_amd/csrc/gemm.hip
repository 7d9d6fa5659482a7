// Hand-written MFMA GEMM:  C[M][N] (bf16) = scale * A[M][K] . B[N][K]^T, fp32 accumulate.
// Both operands are K-contiguous ("row-major A, column-major B").
//
// Tiling.  One workgroup of 512 threads (8 waves, 2 per SIMD) owns a 256x256 tile
// of C and walks K in steps of one 128-byte row segment (64 bf16 or 128 fp8
// elements).  The A and B slabs of a step (256 rows x 128 B each) live in LDS,
// double buffered: 2 x 64 KiB of the CU's 160 KiB.  Waves form a 2 (M) x 4 (N) grid;
// each wave owns 128x64 of C = 8x4 MFMA tiles of 16x16, 128 fp32 accumulators per
// lane.
//
// Data movement.  Global memory goes straight into LDS (global_load_lds_dwordx4, 16
// bytes per lane, no staging registers, no ds_write): one such instruction moves 8
// rows x 128 B, a wave issues 4 for A and 4 for B per step.  The loads of slab s+2
// are issued in the middle of step s, right after the barrier that frees their
// buffer, so they have a whole step to land.
//
// LDS layout.  A row's 128 bytes are eight 16-byte chunks; chunk c of row r is stored
// at chunk position c ^ (r & 7).  A fragment read (16 lanes = 16 consecutive rows,
// same logical chunk) then spreads over all eight chunk positions instead of hitting
// one bank group 16 times.  The direct-to-LDS load writes lane i at position i of its
// 1 KiB destination, so lane i fetches the global chunk that belongs there.
//
// Schedule of one step (bf16: two K=32 halves, fragment sets F0 and F1):
//     32 MFMAs on F0, the 12 LDS reads of F1 slipped between the first 20
//     wait F1; wait own global loads; barrier      <- slab s+1 complete, slab s free
//     32 MFMAs on F1; between them the 12 LDS reads of the next step's F0 and the 8
//     global->LDS loads of slab s+2 into the freed buffer
// One barrier per step; an MFMA is always the first thing a wave issues after the barrier
// (its operands are already in registers), memory instructions are spread out so that a
// wave never sits on a full memory queue with MFMAs waiting behind it.  The loop body is inline assembly so that this order is the order issued;
// the compiler knows neither the LDS reads nor the MFMAs and therefore inserts no wait
// states of its own: every s_waitcnt below is part of the schedule.
//
// The MFMA is issued with the B fragment as the first operand, which produces the
// transposed 16x16 tile: a lane then holds 4 consecutive N elements of one C row and
// stores them as one 8-byte word.
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
constexpr int kSlabBytes = kTile * kRowBytes;   // 32 KiB per operand per step
constexpr int kBufBytes = 2 * kSlabBytes;       // A slab then B slab

typedef __attribute__((address_space(3))) void *lds_void_ptr;
typedef const __attribute__((address_space(1))) void *global_void_ptr;

// 16 bytes per lane from global memory straight into LDS; lane i lands at lds_dst + 16*i.
__device__ inline void load_to_lds(const uint8_t *gptr, uint32_t lds_dst) {
  __builtin_amdgcn_global_load_lds((global_void_ptr)gptr, (lds_void_ptr)(uintptr_t)lds_dst, 16, 0, 0);
}

#define MI355_DS_READ(dst, addr, off) \
  asm volatile("ds_read_b128 %0, %1 offset:" #off : "=v"(dst) : "v"(addr))

// 8 A fragments (rows i*16.., 2 KiB apart) and 4 B fragments from the given LDS addresses.
#define MI355_READ_FRAGS(fa, fb, a_addr, b_addr)                                                   \
  MI355_DS_READ(fb[0], b_addr, 0); MI355_DS_READ(fb[1], b_addr, 2048);                             \
  MI355_DS_READ(fa[0], a_addr, 0); MI355_DS_READ(fa[1], a_addr, 2048);                             \
  MI355_DS_READ(fb[2], b_addr, 4096); MI355_DS_READ(fb[3], b_addr, 6144);                          \
  MI355_DS_READ(fa[2], a_addr, 4096); MI355_DS_READ(fa[3], a_addr, 6144);                          \
  MI355_DS_READ(fa[4], a_addr, 8192); MI355_DS_READ(fa[5], a_addr, 10240);                         \
  MI355_DS_READ(fa[6], a_addr, 12288); MI355_DS_READ(fa[7], a_addr, 14336)

// All LDS reads issued so far have returned.  The fragments ride along as operands so that
// no consumer can be placed ahead of the wait.
#define MI355_WAIT_FRAGS(fa, fb)                                                                   \
  asm volatile("s_waitcnt lgkmcnt(0)"                                                              \
               : "+v"(fa[0]), "+v"(fa[1]), "+v"(fa[2]), "+v"(fa[3]), "+v"(fa[4]), "+v"(fa[5]),     \
                 "+v"(fa[6]), "+v"(fa[7]), "+v"(fb[0]), "+v"(fb[1]), "+v"(fb[2]), "+v"(fb[3]))

// acc(transposed tile) += B_frag . A_frag^T
#define MI355_MFMA_BF16(acc, fb, fa) \
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(fb), "v"(fa))

// One row of MFMAs: the 4 tiles that share A fragment i.
#define MI355_MFMA_ROW(acc, fa, fb, i)                                                             \
  MI355_MFMA_BF16(acc[i][0], fb[0], fa[i]); MI355_MFMA_BF16(acc[i][1], fb[1], fa[i]);              \
  MI355_MFMA_BF16(acc[i][2], fb[2], fa[i]); MI355_MFMA_BF16(acc[i][3], fb[3], fa[i])

__device__ inline void tile_of_block(uint32_t tiles_m, uint32_t tiles_n, uint32_t &tm, uint32_t &tn) {
  const uint32_t bid = blockIdx.x, total = tiles_m * tiles_n;
  uint32_t lin = bid;
  if (total % 8u == 0u) lin = (bid % 8u) * (total / 8u) + bid / 8u;   // tiles of one XCD are consecutive
  // consecutive tiles walk down a group of 4 tile rows, then move one column right
  const uint32_t group = lin / (4u * tiles_n), in_group = lin % (4u * tiles_n);
  const uint32_t rows_here = (tiles_m - group * 4u) < 4u ? (tiles_m - group * 4u) : 4u;
  tm = group * 4u + in_group % rows_here;
  tn = in_group / rows_here;
}

__global__ void __launch_bounds__(kThreads)
gemm_bf16_kernel(const uint8_t *__restrict__ A, const uint8_t *__restrict__ B, uint16_t *__restrict__ C,
                 uint32_t N, uint32_t k_bytes, uint32_t tiles_m, uint32_t tiles_n) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const uint32_t tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const uint32_t wm = wave / 4, wn = wave % 4;
  uint32_t tm, tn;
  tile_of_block(tiles_m, tiles_n, tm, tn);

  // --- global -> LDS: this lane's source pointers and this wave's destinations -------------
  // instruction q of a wave fills rows [(wave*4+q)*8, +8) of a slab; lane i is position i%8 of
  // row i/8, which holds logical chunk (i%8) ^ (row & 7) = (i%8) ^ (i/8).
  const uint32_t lrow = wave * 32u + lane / 8u, lchunk = (lane % 8u) ^ (lane / 8u);
  const uint8_t *ga = A + ((size_t)tm * kTile + lrow) * k_bytes + lchunk * 16u;
  const uint8_t *gb = B + ((size_t)tn * kTile + lrow) * k_bytes + lchunk * 16u;
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
  const uint32_t dst_wave = __builtin_amdgcn_readfirstlane(lds_base + wave * 4096u);
  auto fetch_slab = [&](uint32_t step, uint32_t buf) {
    const size_t kb = (size_t)step * kRowBytes;
    const uint32_t dst = dst_wave + buf * kBufBytes;
#pragma unroll
    for (uint32_t q = 0; q < 4; q++) {
      load_to_lds(ga + kb + (size_t)q * 8u * k_bytes, dst + q * 1024u);
      load_to_lds(gb + kb + (size_t)q * 8u * k_bytes, dst + kSlabBytes + q * 1024u);
    }
  };

  // --- LDS -> fragments: byte addresses of this lane's first A / B fragment -------------------
  // row (lane%16) of the wave's sub-tile, logical chunk ks*4 + lane/16, swizzled with row&7 = lane&7;
  // the second K half differs by bit 2 of the chunk index, i.e. by 64 bytes.
  const uint32_t swz0 = ((lane / 16u) ^ (lane & 7u)) << 4;
  uint32_t a_cur = lds_base + (wm * 128u + lane % 16u) * kRowBytes + swz0;
  uint32_t b_cur = lds_base + kSlabBytes + (wn * 64u + lane % 16u) * kRowBytes + swz0;
  uint32_t a_nxt = a_cur + kBufBytes, b_nxt = b_cur + kBufBytes;

  f32x4v acc[8][4];
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = (f32x4v){0.f, 0.f, 0.f, 0.f};
  bf16x8v fa0[8], fb0[4], fa1[8], fb1[4];

  const uint32_t steps = k_bytes / kRowBytes;
  fetch_slab(0, 0);
  if (steps > 1) fetch_slab(1, 1);
  asm volatile("s_waitcnt vmcnt(0)\n s_barrier" ::: "memory");
  MI355_READ_FRAGS(fa0, fb0, a_cur, b_cur);
  MI355_WAIT_FRAGS(fa0, fb0);

  // Per-lane global pointers of the next slab to fetch (advanced by one step per trip) and
  // the wave's LDS destination for it.
  const uint8_t *ga_next = ga + 2 * (size_t)kRowBytes, *gb_next = gb + 2 * (size_t)kRowBytes;
  const size_t row8 = 8 * (size_t)k_bytes;

  for (uint32_t s = 0; s < steps; s++) {
    const uint32_t buf = s & 1u;
    const uint32_t a1 = a_cur ^ 64u, b1 = b_cur ^ 64u;   // second K half of this step
    // ---- first half: MFMAs on F0, the reads of F1 slipped in between ---------------------------
    MI355_DS_READ(fb1[0], b1, 0);     MI355_DS_READ(fb1[1], b1, 2048);
    MI355_MFMA_ROW(acc, fa0, fb0, 0);
    MI355_DS_READ(fb1[2], b1, 4096);  MI355_DS_READ(fb1[3], b1, 6144);
    MI355_DS_READ(fa1[0], a1, 0);     MI355_DS_READ(fa1[1], a1, 2048);
    MI355_MFMA_ROW(acc, fa0, fb0, 1);
    MI355_DS_READ(fa1[2], a1, 4096);  MI355_DS_READ(fa1[3], a1, 6144);
    MI355_MFMA_ROW(acc, fa0, fb0, 2);
    MI355_DS_READ(fa1[4], a1, 8192);  MI355_DS_READ(fa1[5], a1, 10240);
    MI355_MFMA_ROW(acc, fa0, fb0, 3);
    MI355_DS_READ(fa1[6], a1, 12288); MI355_DS_READ(fa1[7], a1, 14336);
    MI355_MFMA_ROW(acc, fa0, fb0, 4);
    MI355_MFMA_ROW(acc, fa0, fb0, 5);
    MI355_MFMA_ROW(acc, fa0, fb0, 6);
    MI355_MFMA_ROW(acc, fa0, fb0, 7);
    MI355_WAIT_FRAGS(fa1, fb1);
    // every wave is done reading slab s; every wave's share of slab s+1 has landed
    asm volatile("s_waitcnt vmcnt(0)\n s_barrier" ::: "memory");
    // ---- second half: MFMAs on F1 first (they are ready), next F0 reads and the global loads
    //      of slab s+2 spread between them so that no wave sits on the memory queues ------------
    const bool more_reads = s + 1 < steps, more_loads = s + 2 < steps;
    const uint32_t dst = dst_wave + buf * kBufBytes;
    MI355_MFMA_ROW(acc, fa1, fb1, 0);
    if (more_reads) { MI355_DS_READ(fb0[0], b_nxt, 0);    MI355_DS_READ(fb0[1], b_nxt, 2048);
                      MI355_DS_READ(fb0[2], b_nxt, 4096); MI355_DS_READ(fb0[3], b_nxt, 6144); }
    MI355_MFMA_ROW(acc, fa1, fb1, 1);
    if (more_reads) { MI355_DS_READ(fa0[0], a_nxt, 0);    MI355_DS_READ(fa0[1], a_nxt, 2048);
                      MI355_DS_READ(fa0[2], a_nxt, 4096); MI355_DS_READ(fa0[3], a_nxt, 6144); }
    MI355_MFMA_ROW(acc, fa1, fb1, 2);
    if (more_reads) { MI355_DS_READ(fa0[4], a_nxt, 8192);  MI355_DS_READ(fa0[5], a_nxt, 10240);
                      MI355_DS_READ(fa0[6], a_nxt, 12288); MI355_DS_READ(fa0[7], a_nxt, 14336); }
    MI355_MFMA_ROW(acc, fa1, fb1, 3);
    if (more_loads) { load_to_lds(ga_next, dst);                  load_to_lds(gb_next, dst + kSlabBytes); }
    MI355_MFMA_ROW(acc, fa1, fb1, 4);
    if (more_loads) { load_to_lds(ga_next + row8, dst + 1024u);   load_to_lds(gb_next + row8, dst + kSlabBytes + 1024u); }
    MI355_MFMA_ROW(acc, fa1, fb1, 5);
    if (more_loads) { load_to_lds(ga_next + 2 * row8, dst + 2048u); load_to_lds(gb_next + 2 * row8, dst + kSlabBytes + 2048u); }
    MI355_MFMA_ROW(acc, fa1, fb1, 6);
    if (more_loads) { load_to_lds(ga_next + 3 * row8, dst + 3072u); load_to_lds(gb_next + 3 * row8, dst + kSlabBytes + 3072u); }
    MI355_MFMA_ROW(acc, fa1, fb1, 7);
    MI355_WAIT_FRAGS(fa0, fb0);
    ga_next += kRowBytes;
    gb_next += kRowBytes;
    uint32_t t = a_cur; a_cur = a_nxt; a_nxt = t;
    t = b_cur; b_cur = b_nxt; b_nxt = t;
  }
  // wait states the compiler cannot know about, before the accumulators are read
  asm volatile("s_nop 15\n s_nop 15" ::: "memory");

  // --- epilogue: round to bf16, 4 consecutive N elements per lane -----------------------------
  const uint32_t row0 = tm * kTile + wm * 128u + lane % 16u, col0 = tn * kTile + wn * 64u + 4u * (lane / 16u);
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const uint16_t h0 = mi355_f32_to_bf16(acc[i][j][0]), h1 = mi355_f32_to_bf16(acc[i][j][1]);
      const uint16_t h2 = mi355_f32_to_bf16(acc[i][j][2]), h3 = mi355_f32_to_bf16(acc[i][j][3]);
      const uint2 packed = make_uint2((uint32_t)h0 | ((uint32_t)h1 << 16), (uint32_t)h2 | ((uint32_t)h3 << 16));
      *reinterpret_cast<uint2 *>(C + (size_t)(row0 + i * 16u) * N + col0 + j * 16u) = packed;
    }
}

// fp8 e4m3 variant: one K=128 MFMA step per slab, compiler-scheduled.
__device__ inline uint32_t swizzled(uint32_t row, uint32_t chunk) {
  return row * kRowBytes + ((chunk ^ (row & 7u)) << 4);
}

__global__ void __launch_bounds__(kThreads)
gemm_fp8_kernel(const uint8_t *__restrict__ A, const uint8_t *__restrict__ B, uint16_t *__restrict__ C,
                uint32_t N, uint32_t k_bytes, float scale, uint32_t tiles_m, uint32_t tiles_n) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const uint32_t tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const uint32_t wm = wave / 4, wn = wave % 4;
  uint32_t tm, tn;
  tile_of_block(tiles_m, tiles_n, tm, tn);
  const uint8_t *a_tile = A + (size_t)tm * kTile * k_bytes;
  const uint8_t *b_tile = B + (size_t)tn * kTile * k_bytes;

  f32x4v acc[8][4];
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = (f32x4v){0.f, 0.f, 0.f, 0.f};

  constexpr int kChunksPerThread = kSlabBytes / 16 / kThreads;  // 4
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
    uint8_t *sa = lds + (size_t)buf * kBufBytes, *sb = sa + kSlabBytes;
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
    const uint8_t *sa = lds + (size_t)buf * kBufBytes + (size_t)wm * 128 * kRowBytes;
    const uint8_t *sb = lds + (size_t)buf * kBufBytes + kSlabBytes + (size_t)wn * 64 * kRowBytes;
    // a lane's 32 codes are logical chunks 2*(lane/16) and 2*(lane/16)+1 (the same choice for
    // A and B, which is all a dot product needs)
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
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf[j], af, acc[i][j], MI355_F8F6F4_E4M3,
                                                                       MI355_F8F6F4_E4M3, 0, 0x7f, 0, 0x7f);
    }
    if (s + 1 < steps) lds_commit(buf ^ 1u);
    __syncthreads();
  }

  const uint32_t row0 = tm * kTile + wm * 128u + lane % 16u, col0 = tn * kTile + wn * 64u + 4u * (lane / 16u);
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const uint16_t h0 = mi355_f32_to_bf16(acc[i][j][0] * scale), h1 = mi355_f32_to_bf16(acc[i][j][1] * scale);
      const uint16_t h2 = mi355_f32_to_bf16(acc[i][j][2] * scale), h3 = mi355_f32_to_bf16(acc[i][j][3] * scale);
      const uint2 packed = make_uint2((uint32_t)h0 | ((uint32_t)h1 << 16), (uint32_t)h2 | ((uint32_t)h3 << 16));
      *reinterpret_cast<uint2 *>(C + (size_t)(row0 + i * 16u) * N + col0 + j * 16u) = packed;
    }
}

int check_shapes(mi355_dev *dev, const void *A, const void *B, const void *C, uint32_t M, uint32_t N, uint32_t K,
                 uint32_t elem) {
  MI355_REQUIRE(dev, A && B && C, "gemm: null buffer");
  MI355_REQUIRE(dev, M > 0 && N > 0 && K > 0, "gemm: empty problem");
  MI355_REQUIRE(dev, M % kTile == 0 && N % kTile == 0, "gemm: M (%u) and N (%u) must be multiples of 256", M, N);
  MI355_REQUIRE(dev, (K * elem) % kRowBytes == 0, "gemm: K (%u) must be a multiple of %u", K, kRowBytes / elem);
  MI355_REQUIRE(dev, (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15u) == 0, "gemm: buffers must be 16-byte aligned");
  return MI355_OK;
}

constexpr size_t kLdsBytes = 2 * (size_t)kBufBytes;  // 128 KiB

}  // namespace

extern "C" int mi355_gemm_bf16(mi355_dev *dev, const uint16_t *A, const uint16_t *B, uint16_t *C, uint32_t M,
                               uint32_t N, uint32_t K) {
  MI355_ENTER(dev);
  if (int rc = check_shapes(dev, A, B, C, M, N, K, 2)) return rc;
  static bool attr_set = false;
  if (!attr_set) {
    MI355_HIP(dev, hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_bf16_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytes));
    attr_set = true;
  }
  const uint32_t tiles_m = M / kTile, tiles_n = N / kTile;
  gemm_bf16_kernel<<<tiles_m * tiles_n, kThreads, kLdsBytes, dev->stream>>>(
      (const uint8_t *)A, (const uint8_t *)B, C, N, K * 2u, tiles_m, tiles_n);
  MI355_LAUNCH_CHECK(dev, "gemm_bf16");
  return MI355_OK;
}

extern "C" int mi355_gemm_fp8_e4m3(mi355_dev *dev, const uint8_t *A, const uint8_t *B, uint16_t *C, uint32_t M,
                                   uint32_t N, uint32_t K, float scale_a, float scale_b) {
  MI355_ENTER(dev);
  if (int rc = check_shapes(dev, A, B, C, M, N, K, 1)) return rc;
  static bool attr_set = false;
  if (!attr_set) {
    MI355_HIP(dev, hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_fp8_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytes));
    attr_set = true;
  }
  const uint32_t tiles_m = M / kTile, tiles_n = N / kTile;
  gemm_fp8_kernel<<<tiles_m * tiles_n, kThreads, kLdsBytes, dev->stream>>>(
      A, B, C, N, K, scale_a * scale_b, tiles_m, tiles_n);
  MI355_LAUNCH_CHECK(dev, "gemm_fp8_e4m3");
  return MI355_OK;
}
