// Hand-written MFMA GEMM:  C[M][N] = scale * A[M][K] . B[N][K]^T.  Both operands are K-contiguous
// ("row-major A, column-major B").  This file holds the C entry points and the fp32 kernel; the kernel of the
// bf16, f16, int8, fp8 and block-scaled e2m1 kinds is gemm_quad.hip (four waves per workgroup), the fp64 kernel
// gemm_f64.hip.  Tiles, their order and the direct-to-LDS loads are shared (gemm_ring.h).
//
// The fp32 kernel.  One workgroup of 512 threads (8 waves, 2 per SIMD) owns a 256x256 tile of C and walks K in
// steps of one 128-byte row segment (32 floats): per step an A slab and a B slab of 256 rows x 128 B = 32 KiB
// each.  Waves form a 2 (M) x 4 (N) grid; each wave owns 128x64 of C = 8x4 MFMA tiles of 16x16, 128 fp32
// accumulators per lane.  The fp32 matrix instruction (16x16x4, 32 cycles for 2048 flop) leaves the memory
// system idle three quarters of the time, so this kernel needs none of what the narrow kinds need.
//
// LDS ring.  All 160 KiB of the CU's LDS are five 32 KiB slots; the A slab of step t
// lives in slot 2t mod 5, its B slab in slot (2t+1) mod 5.  When the barrier of step s
// frees the two slots of slab s, the B slab of step s+2 is fetched into the old A slot
// and the A slab of step s+3 into the old B slot.  Loads return in order, so the wait before a barrier
// lets the wave's 4 youngest loads (the A rows three steps ahead) stay in flight.
//
// Data movement.  Global memory goes straight into LDS (global_load_lds_dwordx4, 16
// bytes per lane, no staging registers, no ds_write): one such instruction moves 8
// rows x 128 B.
//
// LDS layout.  A row's 128 bytes are eight 16-byte chunks; chunk c of row r is stored
// at chunk position c ^ (r & 7).  A fragment read (16 lanes = 16 consecutive rows,
// same logical chunk) then spreads over all eight chunk positions instead of hitting
// one bank group 16 times.  The direct-to-LDS load writes lane i at position i of its
// 1 KiB destination, so lane i fetches the global chunk that belongs there.
//
// The MFMA is issued with the B fragment as the first operand, which produces the
// transposed 16x16 tile: a lane then holds 4 consecutive N elements of one C row.
//
// Workgroups are persistent: one per CU (the ring takes the whole LDS), each walking the
// tiles id, id + grid, id + 2*grid, ...  The ring does not stop at a tile boundary: slabs are
// numbered through all tiles of the workgroup.  After its last tile a workgroup keeps fetching (the slabs of
// its first tile again, which nobody reads) so that every step is the same code; those loads are waited for
// before the wave ends.
//
// Tile id -> tile mapping (tile_at in gemm_ring.h).  Workgroups are dealt round-robin to the 8 XCDs, each
// with its own L2, and id + k*grid stays on the XCD of id.  With 256 workgroups on a grid whose sides are
// multiples of 16 tiles, one round of the part is a square of 16x16 tiles (4x8 per XCD), squares in serpentine
// order, so that what is re-read from round to round fits the last-level cache; other grids hand every XCD a
// contiguous band of tile rows, walked in column-major order of 4-row groups so that B slabs are reused while hot.
#include "internal.h"
#include "mfma_common.h"
#include "gemm_ring.h"
#include "gemm_quad.h"
#include <utility>

namespace {

constexpr int kThreads = 512;   // 8 waves, 2 (M) x 4 (N), 128x64 of C each
using Ring = GemmRing<2, 4>;

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

// The barrier of a step: every wave holds all fragments of the step's slab (its two slots are free)
// and, loads returning in order, with its 4 youngest loads (the A rows three slabs ahead) still
// allowed in flight, its share of the next slab has landed.  In the first step of a tile that
// wait was done at the end of the tile before, and the stores issued since must not count.
#define MI355_STEP_BARRIER(first, lds_wait, youngest)                                              \
  asm volatile(lds_wait "s_cmp_lg_u32 %0, 0\n s_cbranch_scc1 1f\n s_waitcnt vmcnt(" youngest ")\n1:\n s_barrier"  \
               :: "s"(first) : "memory", "scc")

// Between the last matrix instruction of a tile and the first read of its accumulators: the wait
// states the compiler cannot know about (the operands tie the youngest results to this point), then
// the wave's loads but the 4 youngest, before any store joins the queue of outstanding memory
// operations: the first barrier of the next tile then needs no wait of its own.
#define MI355_END_OF_TILE(acc)                                                                     \
  asm volatile("s_nop 15\n s_nop 15\n s_waitcnt vmcnt(4)"                                          \
               : "+v"(acc[7][0]), "+v"(acc[7][1]), "+v"(acc[7][2]), "+v"(acc[7][3]), "+v"(acc[6][3]) :: "memory")

// ---- fp32 ----------------------------------------------------------------------------------------
// Two fragment sets (one per K half); a 128-byte row segment is 32 floats.  The fp32 matrix
// instruction is 16x16x4 with ONE float per lane and operand (row lane%16, k = lane/16).  A lane's
// 16-byte fragment read is chunk lane/16 of its row, i.e. floats 4*(lane/16) .. +3; register t of it,
// used as the operand of the t-th of four instructions, makes lane group g supply k = 4g + t: the four
// instructions together cover the 16 floats of a K half, in an order that is the same for A and B.
// 256 instructions of 32 cycles per wave and step: the matrix pipe has four times as long per slab as
// in the 16-bit kernel, so the memory instructions need no careful placement, only an order: the 12
// reads of the second K half in the first 6 gaps, the barrier after instruction 7, the wave's B loads
// then its A loads one every 16 instructions, the next step's first-half reads from instruction 208.
template <int E>
__device__ __forceinline__ void f32_read_fragment(f32x4v (&fa)[8], f32x4v (&fb)[4], uint32_t a_addr, uint32_t b_addr) {
  if constexpr (E < 4) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(fb[E]) : "v"(b_addr), "i"(2048 * E));
  else asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(fa[E - 4]) : "v"(a_addr), "i"(2048 * (E - 4)));
}

template <int M>
__device__ __forceinline__ void f32_slot(f32x4v (&acc)[8][4], f32x4v (&fa0)[8], f32x4v (&fb0)[4], f32x4v (&fa1)[8],
                                         f32x4v (&fb1)[4], const GemmWalk &w, uint32_t first, uint32_t a1, uint32_t b1) {
  constexpr int half = M / 128, t = (M / 32) % 4, i = (M / 4) % 8, j = M % 4;
  if constexpr (half == 0)
    asm volatile("v_mfma_f32_16x16x4_f32 %0, %1, %2, %0" : "+v"(acc[i][j]) : "v"(fb0[j][t]), "v"(fa0[i][t]));
  else
    asm volatile("v_mfma_f32_16x16x4_f32 %0, %1, %2, %0" : "+v"(acc[i][j]) : "v"(fb1[j][t]), "v"(fa1[i][t]));
  if constexpr (M < 6) {
    f32_read_fragment<2 * M>(fa1, fb1, a1, b1);
    f32_read_fragment<2 * M + 1>(fa1, fb1, a1, b1);
  }
  if constexpr (M == 7) {
    MI355_WAIT_FRAGS(fa1, fb1);
    MI355_STEP_BARRIER(first, "", "4");
  }
  if constexpr (M >= 16 && M < 80 && M % 16 == 0)
    MI355_LOAD_LDS(w.voff, w.gb + (uint64_t)((M - 16) / 16) * w.row8, w.dst_b + ((M - 16) / 16) * 1024u);
  if constexpr (M >= 136 && M < 200 && (M - 136) % 16 == 0)
    MI355_LOAD_LDS(w.voff, w.ga + (uint64_t)((M - 136) / 16) * w.row8, w.dst_a + ((M - 136) / 16) * 1024u);
  if constexpr (M >= 208 && (M - 208) % 4 == 0) f32_read_fragment<(M - 208) / 4>(fa0, fb0, w.a_nxt, w.b_nxt);
}

template <int... Ms>
__device__ __forceinline__ void f32_step(std::integer_sequence<int, Ms...>, f32x4v (&acc)[8][4], f32x4v (&fa0)[8],
                                         f32x4v (&fb0)[4], f32x4v (&fa1)[8], f32x4v (&fb1)[4], const GemmWalk &w,
                                         uint32_t first) {
  const uint32_t a1 = w.a_cur ^ 64u, b1 = w.b_cur ^ 64u;   // second K half of this step
  (f32_slot<Ms>(acc, fa0, fb0, fa1, fb1, w, first, a1, b1), ...);
  MI355_WAIT_FRAGS(fa0, fb0);
}

__global__ void __launch_bounds__(kThreads)
gemm_f32_kernel(const uint8_t *__restrict__ A, const uint8_t *__restrict__ B, float *__restrict__ C, uint32_t N,
                uint32_t k_bytes, uint32_t tiles_m, uint32_t tiles_n) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const uint32_t tid = threadIdx.x, lane = tid % 64;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const uint32_t wm = wave / 4, wn = wave % 4;
  const TileGrid grid = tiles_of_workgroup(tiles_m, tiles_n);

  Ring ring;
  ring.start(A, B, k_bytes, (uint32_t)(uintptr_t)lds, wave, lane, grid);
  const uint32_t steps = ring.steps;

  f32x4v acc[8][4];
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = (f32x4v){0.f, 0.f, 0.f, 0.f};
  f32x4v fa0[8], fb0[4], fa1[8], fb1[4];
  MI355_READ_FRAGS(fa0, fb0, ring.w.a_cur, ring.w.b_cur);
  MI355_WAIT_FRAGS(fa0, fb0);

  uint32_t round = 0, left = steps, first = 1;
  for (uint32_t g = grid.mine * steps; g > 0; g--) {
    f32_step(std::make_integer_sequence<int, 256>{}, acc, fa0, fb0, fa1, fb1, ring.w, first);
    ring.advance();
    first = 0;
    if (--left == 0) {
      MI355_END_OF_TILE(acc);
      uint32_t tm, tn;
      tile_at(grid, round, tm, tn);
      // 4 consecutive N elements per lane, 16 bytes: the four lane groups write 64 contiguous bytes per row
      const uint32_t row0 = tm * kTile + wm * 128u + lane % 16u, col0 = tn * kTile + wn * 64u + 4u * (lane / 16u);
#pragma unroll
      for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
          *reinterpret_cast<f32x4v *>(C + (size_t)(row0 + i * 16u) * N + col0 + j * 16u) = acc[i][j];
          acc[i][j] = (f32x4v){0.f, 0.f, 0.f, 0.f};
        }
      round++;
      left = steps;
      first = 1;
    }
  }
  MI355_DRAIN_RING();
}

int check_shapes(mi355_dev *dev, const void *A, const void *B, const void *C, uint32_t M, uint32_t N, uint32_t K,
                 uint32_t elem, uint32_t tile = kTile) {
  MI355_REQUIRE(dev, A && B && C, "gemm: null buffer");
  MI355_REQUIRE(dev, M > 0 && N > 0 && K > 0, "gemm: empty problem");
  MI355_REQUIRE(dev, M % tile == 0 && N % tile == 0, "gemm: M (%u) and N (%u) must be multiples of %u", M, N, tile);
  MI355_REQUIRE(dev, (uint64_t)K * elem <= (64u << 20), "gemm: a row of K is %llu bytes, the kernels take at most 64 MiB (32-bit lane offsets)",
                (unsigned long long)K * elem);
  MI355_REQUIRE(dev, (K * elem) % kRowBytes == 0, "gemm: K (%u) must be a multiple of %u", K, kRowBytes / elem);
  MI355_REQUIRE(dev, (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15u) == 0, "gemm: buffers must be 16-byte aligned");
  return MI355_OK;
}

// The 8- and 16-bit kinds run on the four-wave kernel of gemm_quad.hip (256x256 tiles, one persistent workgroup per
// CU), or, when that tiling has too few tiles for the part, on the 128x128 tiles of gemm_small.hip: four times the
// workgroups at half the arithmetic per byte of operand.  "Too few" is at most half a tile per CU: from there up the
// big tiles keep at least every second CU busy at twice the efficiency.  A product whose M or N is a multiple of 128
// only has no 256x256 tiling and runs on the small tiles whatever its size.
int launch_quad(mi355_dev *dev, int op, const char *what, const void *A, const void *B, void *C, uint32_t M, uint32_t N, uint32_t K,
                uint32_t elem, float scale) {
  if (int rc = check_shapes(dev, A, B, C, M, N, K, elem, kTile / 2)) return rc;
  const bool big_fits = M % kTile == 0 && N % kTile == 0;
  MI355_REQUIRE(dev, big_fits || dev->gemm_tiling != MI355_GEMM_TILING_256,
                "gemm: M (%u) and N (%u) must be multiples of 256 on the 256x256 tiles this handle is set to", M, N);
  const uint64_t tiles = (uint64_t)(M / kTile) * (N / kTile);
  const bool small = !big_fits || dev->gemm_tiling == MI355_GEMM_TILING_128 ||
                     (dev->gemm_tiling == MI355_GEMM_TILING_AUTO && 2u * tiles <= (uint64_t)(dev->props.num_cus > 0 ? dev->props.num_cus : 1));
  if (small) return mi355_launch_gemm_small(dev, op, what, A, B, C, M, N, K * elem, scale);
  return mi355_launch_gemm_quad(dev, op, what, A, B, C, M, N, K * elem, scale);
}

}  // namespace

extern "C" int mi355_gemm_tiling(mi355_dev *dev, int tiling) {
  if (!dev) return mi355_fail(nullptr, MI355_ERR_ARG, "null device handle");
  MI355_REQUIRE(dev, tiling == MI355_GEMM_TILING_AUTO || tiling == MI355_GEMM_TILING_256 || tiling == MI355_GEMM_TILING_128,
                "gemm_tiling: unknown tiling %d", tiling);
  dev->gemm_tiling = tiling;
  return MI355_OK;
}

extern "C" int mi355_gemm_bf16(mi355_dev *dev, const uint16_t *A, const uint16_t *B, uint16_t *C, uint32_t M,
                               uint32_t N, uint32_t K) {
  MI355_ENTER(dev);
  return launch_quad(dev, kQuadBf16, "gemm_bf16", A, B, C, M, N, K, 2, 1.0f);
}

extern "C" int mi355_gemm_f16(mi355_dev *dev, const uint16_t *A, const uint16_t *B, uint16_t *C, uint32_t M,
                              uint32_t N, uint32_t K) {
  MI355_ENTER(dev);
  return launch_quad(dev, kQuadF16, "gemm_f16", A, B, C, M, N, K, 2, 1.0f);
}

extern "C" int mi355_gemm_f32(mi355_dev *dev, const float *A, const float *B, float *C, uint32_t M, uint32_t N,
                              uint32_t K) {
  MI355_ENTER(dev);
  if (int rc = check_shapes(dev, A, B, C, M, N, K, 4)) return rc;
  if (int rc = allow_full_lds(dev, &gemm_f32_kernel, kLdsF32)) return rc;
  const uint32_t tiles_m = M / kTile, tiles_n = N / kTile;
  gemm_f32_kernel<<<gemm_workgroups(dev, tiles_m * tiles_n), kThreads, kRingBytes, dev->stream>>>(
      (const uint8_t *)A, (const uint8_t *)B, C, N, K * 4, tiles_m, tiles_n);
  MI355_LAUNCH_CHECK(dev, "gemm_f32");
  return MI355_OK;
}

extern "C" int mi355_gemm_i8(mi355_dev *dev, const int8_t *A, const int8_t *B, int32_t *C, uint32_t M, uint32_t N,
                             uint32_t K) {
  MI355_ENTER(dev);
  return launch_quad(dev, kQuadI8, "gemm_i8", A, B, C, M, N, K, 1, 1.0f);
}

extern "C" int mi355_gemm_fp8_e4m3(mi355_dev *dev, const uint8_t *A, const uint8_t *B, uint16_t *C, uint32_t M,
                                   uint32_t N, uint32_t K, float scale_a, float scale_b) {
  MI355_ENTER(dev);
  return launch_quad(dev, kQuadE4m3, "gemm_fp8_e4m3", A, B, C, M, N, K, 1, scale_a * scale_b);
}

extern "C" int mi355_gemm_fp8_e5m2(mi355_dev *dev, const uint8_t *A, const uint8_t *B, uint16_t *C, uint32_t M,
                                   uint32_t N, uint32_t K, float scale_a, float scale_b) {
  MI355_ENTER(dev);
  return launch_quad(dev, kQuadE5m2, "gemm_fp8_e5m2", A, B, C, M, N, K, 1, scale_a * scale_b);
}
