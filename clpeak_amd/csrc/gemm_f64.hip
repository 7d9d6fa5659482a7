// Double-precision GEMM:  C[M][N] = A[M][K] . B[N][K]^T, all fp64, both operands K-contiguous.
//
// The fp64 matrix instruction (16x16x4, one double per lane and operand) runs at 128 flop per clock and
// CU: a 128x128 tile needs 4096 cycles of the matrix pipe per 16 doubles of K and 32 KiB of operands,
// a sixteenth of the memory rate of the 16-bit GEMM.  So this kernel is the small sibling of gemm.hip:
// 128x128 tiles, 4 waves of 64x64 (16 accumulator tiles of 4 doubles per lane = 128 registers), two LDS
// buffers of 32 KiB per workgroup, two workgroups per CU, one barrier per step (in its middle, between the
// two K halves, so that every LDS read lands under 32 matrix instructions), and the loads of the next slab
// in flight for a whole step.  The fragment reads of one K half ride on the matrix instructions of the other, one
// read behind every second of its first 16 instructions (all 8 in a burst in front of them: 1 % slower; with no
// reads at all the loop would be another 1 % faster, with no barrier not at all), which fixes the order of the
// instructions: they are written as text, the accumulators in the accumulation registers.  It shares the LDS
// layout with its siblings (rows of 128 bytes, chunk c of row r at position c ^ (r & 7), global memory straight
// into LDS).
//
// A lane's 16-byte fragment read is chunk lane/16 (+4 for the second K half) of its row, two doubles;
// double t of it is the operand of the t-th of two instructions, so lane group g supplies
// k = 2g + t (+8): the same order for A and B.  The product is issued with the B fragment first.  The
// fp64 result layout differs from the 32-bit ones: register r of lane group g is row 4r + g of the first
// operand (not 4g + r).  So lane p of a B fragment reads B row 4(p%4) + p/4 instead of row p, which turns
// that into "register r of group g is column 4g + r of C": 4 consecutive N elements per lane, 32 bytes,
// 128 contiguous bytes per row and store instruction.  (SQ_LDS_BANK_CONFLICT reads 32 cycles per wave and
// step in this kernel, 3 % of its cycles, with this row order and equally with a B-slab swizzle built for
// it; the matrix pipe, 96 % busy, does not notice, so the layout stays the one of the sibling kernels.)
#include "internal.h"
#include "mfma_common.h"
#include "gemm_ring.h"

namespace {

constexpr int kTile64 = 128;                      // C tile edge of this kernel
constexpr int kThreads64 = 256;
constexpr int kSlab64 = kTile64 * kRowBytes;      // 16 KiB per operand per step
typedef double f64x2v __attribute__((ext_vector_type(2)));
typedef double f64x4v __attribute__((ext_vector_type(4)));

#define MI355_DS_READ64(dst, addr, off) \
  asm volatile("ds_read_b128 %0, %1 offset:" #off : "=v"(dst) : "v"(addr))
#define MI355_WAIT_FRAGS64(fa, fb)                                                                 \
  asm volatile("s_waitcnt lgkmcnt(0)"                                                              \
               : "+v"(fa[0]), "+v"(fa[1]), "+v"(fa[2]), "+v"(fa[3]), "+v"(fb[0]), "+v"(fb[1]), "+v"(fb[2]), "+v"(fb[3]))
#define MI355_READ_FRAGS64(fa, fb, a_addr, b_addr)                                                 \
  MI355_DS_READ64(fb[0], b_addr, 0); MI355_DS_READ64(fb[1], b_addr, 2048);                         \
  MI355_DS_READ64(fb[2], b_addr, 4096); MI355_DS_READ64(fb[3], b_addr, 6144);                      \
  MI355_DS_READ64(fa[0], a_addr, 0); MI355_DS_READ64(fa[1], a_addr, 2048);                         \
  MI355_DS_READ64(fa[2], a_addr, 4096); MI355_DS_READ64(fa[3], a_addr, 6144)

// The 32 matrix instructions of one K half (fragments fa, fb), and riding on the first 16 of them, one behind every
// second, the 8 reads of the other fragment set (ra, rb) for the half after this one.
__device__ __forceinline__ void mfma_sweep(f64x4v (&acc)[4][4], const f64x2v (&fa)[4], const f64x2v (&fb)[4], f64x2v (&ra)[4],
                                           f64x2v (&rb)[4], uint32_t a_addr, uint32_t b_addr, bool reads) {
#pragma unroll
  for (int t = 0; t < 2; t++)
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const double b = fb[j][t], a = fa[i][t];
        asm volatile("v_mfma_f64_16x16x4_f64 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(b), "v"(a));
        const int n = t * 16 + i * 4 + j;
        if (n % 2 == 0 && n < 16 && reads) {
          switch (n / 2) {
            case 0: MI355_DS_READ64(rb[0], b_addr, 0); break;
            case 1: MI355_DS_READ64(rb[1], b_addr, 2048); break;
            case 2: MI355_DS_READ64(rb[2], b_addr, 4096); break;
            case 3: MI355_DS_READ64(rb[3], b_addr, 6144); break;
            case 4: MI355_DS_READ64(ra[0], a_addr, 0); break;
            case 5: MI355_DS_READ64(ra[1], a_addr, 2048); break;
            case 6: MI355_DS_READ64(ra[2], a_addr, 4096); break;
            default: MI355_DS_READ64(ra[3], a_addr, 6144); break;
          }
        }
      }
}

__global__ void __launch_bounds__(kThreads64, 2)
gemm_f64_kernel(const uint8_t *__restrict__ A, const uint8_t *__restrict__ B, double *__restrict__ C, uint32_t N,
                uint32_t k_bytes, uint32_t tiles_m, uint32_t tiles_n) {
  __shared__ __attribute__((aligned(1024))) uint8_t lds[4 * kSlab64];   // A0 B0 A1 B1
  const uint32_t tid = threadIdx.x, lane = tid % 64;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const uint32_t wm = wave / 2, wn = wave % 2;
  TileGrid grid;
  grid.tiles_m = tiles_m; grid.tiles_n = tiles_n; grid.total = tiles_m * tiles_n;
  grid.first = blockIdx.x; grid.stride = gridDim.x; grid.mine = 1;
  uint32_t tm, tn;
  tile_at(grid, 0, tm, tn);

  // global -> LDS: wave w fills rows [32w, 32w+32) of the A slab and of the B slab, 8 rows per instruction;
  // lane i is position i%8 of row i/8, which holds logical chunk (i%8) ^ (i/8)
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
  const uint32_t dst_wave = __builtin_amdgcn_readfirstlane(lds_base + wave * 32u * (uint32_t)kRowBytes);
  const uint32_t voff = (lane / 8u) * k_bytes + ((lane % 8u) ^ (lane / 8u)) * 16u, row8 = 8u * k_bytes;
  uint64_t ga = (uint64_t)(uintptr_t)(A + ((size_t)tm * kTile64 + wave * 32u) * k_bytes);
  uint64_t gb = (uint64_t)(uintptr_t)(B + ((size_t)tn * kTile64 + wave * 32u) * k_bytes);
  auto fetch = [&](uint32_t buf) {
#pragma unroll
    for (uint32_t q = 0; q < 4; q++) MI355_LOAD_LDS(voff, ga + (uint64_t)q * row8, dst_wave + buf * 2u * kSlab64 + q * 1024u);
#pragma unroll
    for (uint32_t q = 0; q < 4; q++) MI355_LOAD_LDS(voff, gb + (uint64_t)q * row8, dst_wave + buf * 2u * kSlab64 + kSlab64 + q * 1024u);
    ga += kRowBytes;
    gb += kRowBytes;
  };
  // LDS -> fragments: row lane%16 of the wave's part, chunk lane/16, swizzled with row&7 = lane&7
  const uint32_t swz0 = ((lane / 16u) ^ (lane & 7u)) << 4;
  const uint32_t lane_a = lds_base + (wm * 64u + lane % 16u) * kRowBytes + swz0;
  const uint32_t row_b = 4u * (lane % 4u) + (lane % 16u) / 4u;
  const uint32_t lane_b = lds_base + kSlab64 + (wn * 64u + row_b) * kRowBytes + (((lane / 16u) ^ (row_b & 7u)) << 4);

  f64x4v acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = (f64x4v){0.0, 0.0, 0.0, 0.0};
  f64x2v fa0[4], fb0[4], fa1[4], fb1[4];

  // Two fragment sets, one per K half of a slab, refilled while the other is being multiplied: the reads of
  // the second half go out under the instructions of the first half; in the middle of the step this wave's loads
  // of the next slab have landed and, after the barrier, everybody's, and everybody has read all of this slab: its
  // buffer takes the slab after the next, and the first half of the next slab is read under the instructions of
  // the second half.
  const uint32_t steps = k_bytes / kRowBytes;
  fetch(0);
  asm volatile("s_waitcnt vmcnt(0)\n s_barrier" ::: "memory");
  if (steps > 1) fetch(1);
  MI355_READ_FRAGS64(fa0, fb0, lane_a, lane_b);
  for (uint32_t s = 0; s < steps; s++) {
    const uint32_t cur = (s & 1u) * 2u * kSlab64, nxt = cur ^ (2u * kSlab64);
    MI355_WAIT_FRAGS64(fa0, fb0);
    mfma_sweep(acc, fa0, fb0, fa1, fb1, (lane_a + cur) ^ 64u, (lane_b + cur) ^ 64u, true);
    // (the second fragment set rides along as an operand so that nothing that uses it can be placed before the wait)
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n s_barrier"
                 : "+v"(fa1[0]), "+v"(fa1[1]), "+v"(fa1[2]), "+v"(fa1[3]), "+v"(fb1[0]), "+v"(fb1[1]), "+v"(fb1[2]), "+v"(fb1[3])
                 :: "memory");
    if (s + 2 < steps) fetch(s & 1u);
    mfma_sweep(acc, fa1, fb1, fa0, fb0, lane_a + nxt, lane_b + nxt, s + 1 < steps);
  }
  // the matrix instructions are text to the compiler: the wait states between the last of them and the stores
  asm volatile("s_nop 15\n s_nop 15" ::: "memory");

  const uint32_t row0 = tm * kTile64 + wm * 64u + lane % 16u, col0 = tn * kTile64 + wn * 64u + 4u * (lane / 16u);
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) *reinterpret_cast<f64x4v *>(C + (size_t)(row0 + i * 16u) * N + col0 + j * 16u) = acc[i][j];
}

}  // namespace

extern "C" int mi355_gemm_f64(mi355_dev *dev, const double *A, const double *B, double *C, uint32_t M, uint32_t N,
                              uint32_t K) {
  MI355_ENTER(dev);
  MI355_REQUIRE(dev, A && B && C, "gemm_f64: null buffer");
  MI355_REQUIRE(dev, M > 0 && N > 0 && K > 0, "gemm_f64: empty problem");
  MI355_REQUIRE(dev, M % kTile64 == 0 && N % kTile64 == 0, "gemm_f64: M (%u) and N (%u) must be multiples of 128", M, N);
  MI355_REQUIRE(dev, (uint64_t)K * 8u <= (64u << 20), "gemm_f64: a row of K is %llu bytes, the kernel takes at most 64 MiB (32-bit lane offsets)",
                (unsigned long long)K * 8u);
  MI355_REQUIRE(dev, K % 16 == 0, "gemm_f64: K (%u) must be a multiple of 16", K);
  MI355_REQUIRE(dev, (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 31u) == 0, "gemm_f64: buffers must be 32-byte aligned");
  const uint32_t tiles_m = M / kTile64, tiles_n = N / kTile64;
  gemm_f64_kernel<<<tiles_m * tiles_n, kThreads64, 0, dev->stream>>>((const uint8_t *)A, (const uint8_t *)B, C, N, K * 8u,
                                                                     tiles_m, tiles_n);
  MI355_LAUNCH_CHECK(dev, "gemm_f64");
  return MI355_OK;
}
