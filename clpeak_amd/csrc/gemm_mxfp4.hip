// Block-scaled FP4 GEMM (OCP MXFP4):  C[M][N] (bf16) = sum_k (A[m][k] * 2^(SA[m][k/32]-127)) * (B[n][k] * 2^(SB[n][k/32]-127)).
// A and B hold e2m1 codes, two per byte, K contiguous; SA / SB hold one E8M0 byte per 32 elements.
//
// Same tile walk, LDS ring, swizzle and direct-to-LDS loads as the 16-bit GEMM (gemm.hip): a 256x256
// tile of C per workgroup, K in steps of 128 bytes per row (256 elements), five 32 KiB LDS slots.
// What differs:
//   * One wave per SIMD (4 waves of 128x128) instead of two of 128x64.  The 64 accumulator tiles of a
//     wave live in the 256 accumulation registers, which leaves the vector registers to two fragment
//     sets and to the scale bytes of two steps; with two waves per SIMD there is no room for the scales.
//   * A K=128 instruction takes 16 bytes per lane, i.e. one 16-byte chunk of a row like a bf16 K=32
//     instruction: the first K half of a slab is chunks 0-3, the second chunks 4-7.
//   * Scales do not pass through LDS (it is full).  Lane r+16g of a fragment must hold the scale byte of
//     row r, 32-element block g.  A pre-pass kernel rewrites scale_a / scale_b into that shape once per
//     call: for every block of 128 rows and every K step, 64 lanes x 16 bytes, byte 2i+h of lane (r,g)
//     being the scale of row 16i+r, block 8s+4h+g (fragment i, K half h).  The main loop then fetches
//     the scales of a step with ONE 16-byte load per operand, fully coalesced, one step ahead, and the
//     matrix instruction picks byte 2(i%2)+h of register i/2 with its op_sel field.  (Fetching the bytes
//     from the row-major arrays inside the loop, one gather per fragment and half, more than doubled
//     the run time.)
// Vector-memory instructions return in issue order, which is what the counted waits rely on: per step
// a wave issues its 2 scale loads first, then 8 loads of B rows and 8 of A rows into LDS.  On entry to
// the next step "at most 16 outstanding" means the scales are there; at its barrier "at most 8
// outstanding" means the B rows (and everything older) have landed.
// Workgroups are persistent and the ring runs through tile boundaries, as in gemm.hip; the scale bytes
// are a third stream, one step ahead of the slab being multiplied.  At the end of a tile a wave waits for
// its loads but the 8 youngest before its stores join the queue; the first step of the next tile then
// takes neither the wait for its scale bytes nor the one at its barrier (both would count the stores).
#include "internal.h"
#include "mfma_common.h"
#include "gemm_ring.h"

namespace {

constexpr int kThreads = 256;   // 4 waves, 2 (M) x 2 (N), 128x128 of C each
#define MI355_WAIT_FRAGS16(fa, fb)                                                                 \
  asm volatile("s_waitcnt lgkmcnt(0)"                                                              \
               : "+v"(fa[0]), "+v"(fa[1]), "+v"(fa[2]), "+v"(fa[3]), "+v"(fa[4]), "+v"(fa[5]),     \
                 "+v"(fa[6]), "+v"(fa[7]), "+v"(fb[0]), "+v"(fb[1]), "+v"(fb[2]), "+v"(fb[3]),     \
                 "+v"(fb[4]), "+v"(fb[5]), "+v"(fb[6]), "+v"(fb[7]))
// The 16 scale bytes of this lane for one operand and step (8 fragments x 2 K halves).
#define MI355_SCALE16(reg, voff, sbase) \
  asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(reg) : "v"(voff), "s"(sbase) : "memory")
// acc(transposed tile) += (B_frag * scale_b) . (A_frag * scale_a)^T, e2m1 codes.  The scale byte of an operand
// is byte (op_sel + 2 * op_sel_hi) of its register: H picks the K half, JB / IB the odd fragment.
#define MI355_MFMA_MX(H, JB, IB, acc, fb, fa, sb, sa)                                              \
  asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:[" #H "," #H ",0] op_sel_hi:[" #JB "," #IB \
               ",0] cbsz:4 blgp:4"                                                                 \
               : "+a"(acc) : "v"(fb), "v"(fa), "v"(sb), "v"(sa))

// The ring of the 16-bit GEMM plus the stream of lane-ordered scale bytes, one step ahead: 1 KiB per
// block of 128 rows and step, steps of one block consecutive.
struct MxRing : GemmRing<2, 2> {
  const uint8_t *sal, *sbl;      // lane-ordered scales of A / B
  uint32_t wm, wn;
  uint64_t sa_next, sb_next;     // uniform addresses of the next step's 1 KiB per operand
  uint32_t soff;                 // this lane's offset there (16 * lane)
  uint32_t s_round, s_left;

  __device__ __forceinline__ void scales_of(uint32_t round) {
    uint32_t tm, tn;
    tile_at(grid, round, tm, tn);
    sa_next = (uint64_t)(uintptr_t)(sal + (size_t)(tm * 2u + wm) * steps * 1024u);
    sb_next = (uint64_t)(uintptr_t)(sbl + (size_t)(tn * 2u + wn) * steps * 1024u);
  }
  __device__ __forceinline__ void next_scales() {
    if (--s_left == 0u) {
      s_round = s_round + 1u == grid.mine ? 0u : s_round + 1u;
      scales_of(s_round);
      s_left = steps;
    } else {
      sa_next += 1024;
      sb_next += 1024;
    }
  }
  __device__ __forceinline__ void advance_all() {
    advance();
    next_scales();
  }
};

// The same starting a fresh accumulator tile (C = 0): what the first K half of a tile's first step issues.
#define MI355_MFMA_MX0(H, JB, IB, acc, fb, fa, sb, sa)                                             \
  asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, 0, %3, %4 op_sel:[" #H "," #H ",0] op_sel_hi:[" #JB "," #IB \
               ",0] cbsz:4 blgp:4"                                                                 \
               : "=a"(acc) : "v"(fb), "v"(fa), "v"(sb), "v"(sa))

struct MxFrags {
  i32x4v a0[8], b0[8], a1[8], b1[8];     // fragment sets of the two K halves
  i32x4v sa, sb;                         // scale bytes in use: byte 2i+h of the 16 is fragment i, K half h
  i32x4v sa_n, sb_n;                     // scale bytes being loaded for the next step
};

// One step of K: 128 instructions per wave, 64 on the first K half then 64 on the second, each half walked
// row by row in alternating directions so that consecutive instructions share one operand's registers.
// FIRST: the first step of a tile.  Its first K half starts the accumulators from zero, and it takes no
// counted wait for loads: every outstanding load that matters was waited for at the end of the tile before,
// and the stores issued since must not be counted.
template <bool FIRST>
__device__ __forceinline__ void mx_step(f32x4v (&acc)[8][8], MxFrags &f, const MxRing &ring) {
  const GemmWalk &w = ring.w;
  const uint32_t a1 = w.a_cur ^ 64u, b1 = w.b_cur ^ 64u;
  i32x4v(&fa0)[8] = f.a0; i32x4v(&fb0)[8] = f.b0; i32x4v(&fa1)[8] = f.a1; i32x4v(&fb1)[8] = f.b1;
  // the scale bytes of this step were requested a step ago, before the 16 loads into LDS
  if (!FIRST) asm volatile("s_waitcnt vmcnt(16)" : "+v"(f.sa_n), "+v"(f.sb_n));
  f.sa = f.sa_n;
  f.sb = f.sb_n;
  // the copies are ordinary vector moves; the matrix instruction that reads one as a scale must not issue
  // right behind it, and the compiler cannot see into the assembly to space them
  asm volatile("s_nop 7" : "+v"(f.sa), "+v"(f.sb));
#define MM(H, i, j, JB, IB)                                                                        \
  do {                                                                                             \
    if (FIRST && H == 0) MI355_MFMA_MX0(H, JB, IB, acc[i][j], fb0[j], fa0[i], f.sb[(j) / 2], f.sa[(i) / 2]); \
    else MI355_MFMA_MX(H, JB, IB, acc[i][j], (H ? fb1 : fb0)[j], (H ? fa1 : fa0)[i], f.sb[(j) / 2], f.sa[(i) / 2]); \
  } while (0)
#define LDA(q) MI355_LOAD_LDS(w.voff, w.ga + (uint64_t)(q) * w.row8, w.dst_a + (q) * 1024u)
#define LDB(q) MI355_LOAD_LDS(w.voff, w.gb + (uint64_t)(q) * w.row8, w.dst_b + (q) * 1024u)
#define SCL_A() MI355_SCALE16(f.sa_n, ring.soff, ring.sa_next)
#define SCL_B() MI355_SCALE16(f.sb_n, ring.soff, ring.sb_next)
  MM(0, 0, 0, 0, 0); MI355_DS_READ(fb1[0], b1, 0);
  MM(0, 0, 1, 1, 0); MI355_DS_READ(fb1[1], b1, 2048);
  MM(0, 0, 2, 0, 0); MI355_DS_READ(fb1[2], b1, 4096);
  MM(0, 0, 3, 1, 0); MI355_DS_READ(fb1[3], b1, 6144);
  MM(0, 0, 4, 0, 0); MI355_DS_READ(fb1[4], b1, 8192);
  MM(0, 0, 5, 1, 0); MI355_DS_READ(fb1[5], b1, 10240);
  MM(0, 0, 6, 0, 0); MI355_DS_READ(fb1[6], b1, 12288);
  MM(0, 0, 7, 1, 0); MI355_DS_READ(fb1[7], b1, 14336);
  MM(0, 1, 7, 1, 1); MI355_DS_READ(fa1[0], a1, 0);
  MM(0, 1, 6, 0, 1); MI355_DS_READ(fa1[1], a1, 2048);
  MM(0, 1, 5, 1, 1); MI355_DS_READ(fa1[2], a1, 4096);
  MM(0, 1, 4, 0, 1); MI355_DS_READ(fa1[3], a1, 6144);
  MM(0, 1, 3, 1, 1); MI355_DS_READ(fa1[4], a1, 8192);
  MM(0, 1, 2, 0, 1); MI355_DS_READ(fa1[5], a1, 10240);
  MM(0, 1, 1, 1, 1); MI355_DS_READ(fa1[6], a1, 12288);
  MM(0, 1, 0, 0, 1); MI355_DS_READ(fa1[7], a1, 14336);
  MM(0, 2, 0, 0, 0);
  MM(0, 2, 1, 1, 0);
  MM(0, 2, 2, 0, 0);
  MM(0, 2, 3, 1, 0);
  MM(0, 2, 4, 0, 0);
  MM(0, 2, 5, 1, 0);
  MM(0, 2, 6, 0, 0);
  MM(0, 2, 7, 1, 0);
  MI355_WAIT_FRAGS16(fa1, fb1);
  // every read of this step's slab has returned (its two slots are free); only the 8 youngest loads, the A
  // rows three steps ahead, may still be in flight: this wave's B rows of the next slab have landed
  if (FIRST) asm volatile("s_barrier" ::: "memory");
  else asm volatile("s_waitcnt vmcnt(8)\n s_barrier" ::: "memory");
  MM(0, 3, 7, 1, 1); SCL_B();
  MM(0, 3, 6, 0, 1); SCL_A();
  MM(0, 3, 5, 1, 1);
  MM(0, 3, 4, 0, 1);
  MM(0, 3, 3, 1, 1);
  MM(0, 3, 2, 0, 1);
  MM(0, 3, 1, 1, 1);
  MM(0, 3, 0, 0, 1);
  MM(0, 4, 0, 0, 0);
  MM(0, 4, 1, 1, 0);
  MM(0, 4, 2, 0, 0);
  MM(0, 4, 3, 1, 0);
  MM(0, 4, 4, 0, 0);
  MM(0, 4, 5, 1, 0);
  MM(0, 4, 6, 0, 0);
  MM(0, 4, 7, 1, 0);
  MM(0, 5, 7, 1, 1);
  MM(0, 5, 6, 0, 1);
  MM(0, 5, 5, 1, 1);
  MM(0, 5, 4, 0, 1);
  MM(0, 5, 3, 1, 1);
  MM(0, 5, 2, 0, 1);
  MM(0, 5, 1, 1, 1);
  MM(0, 5, 0, 0, 1);
  MM(0, 6, 0, 0, 0);
  MM(0, 6, 1, 1, 0);
  MM(0, 6, 2, 0, 0);
  MM(0, 6, 3, 1, 0);
  MM(0, 6, 4, 0, 0);
  MM(0, 6, 5, 1, 0);
  MM(0, 6, 6, 0, 0);
  MM(0, 6, 7, 1, 0);
  MM(0, 7, 7, 1, 1); LDB(0);
  MM(0, 7, 6, 0, 1);
  MM(0, 7, 5, 1, 1);
  MM(0, 7, 4, 0, 1);
  MM(0, 7, 3, 1, 1); LDB(1);
  MM(0, 7, 2, 0, 1);
  MM(0, 7, 1, 1, 1);
  MM(0, 7, 0, 0, 1);
  MM(1, 0, 0, 0, 0); LDB(2);
  MM(1, 0, 1, 1, 0); MI355_DS_READ(fb0[0], w.b_nxt, 0);
  MM(1, 0, 2, 0, 0);
  MM(1, 0, 3, 1, 0); MI355_DS_READ(fb0[1], w.b_nxt, 2048);
  MM(1, 0, 4, 0, 0); LDB(3);
  MM(1, 0, 5, 1, 0); MI355_DS_READ(fb0[2], w.b_nxt, 4096);
  MM(1, 0, 6, 0, 0);
  MM(1, 0, 7, 1, 0); MI355_DS_READ(fb0[3], w.b_nxt, 6144);
  MM(1, 1, 7, 1, 1); LDB(4);
  MM(1, 1, 6, 0, 1); MI355_DS_READ(fb0[4], w.b_nxt, 8192);
  MM(1, 1, 5, 1, 1);
  MM(1, 1, 4, 0, 1); MI355_DS_READ(fb0[5], w.b_nxt, 10240);
  MM(1, 1, 3, 1, 1); LDB(5);
  MM(1, 1, 2, 0, 1); MI355_DS_READ(fb0[6], w.b_nxt, 12288);
  MM(1, 1, 1, 1, 1);
  MM(1, 1, 0, 0, 1); MI355_DS_READ(fb0[7], w.b_nxt, 14336);
  MM(1, 2, 0, 0, 0); LDB(6);
  MM(1, 2, 1, 1, 0); MI355_DS_READ(fa0[0], w.a_nxt, 0);
  MM(1, 2, 2, 0, 0);
  MM(1, 2, 3, 1, 0); MI355_DS_READ(fa0[1], w.a_nxt, 2048);
  MM(1, 2, 4, 0, 0); LDB(7);
  MM(1, 2, 5, 1, 0); MI355_DS_READ(fa0[2], w.a_nxt, 4096);
  MM(1, 2, 6, 0, 0);
  MM(1, 2, 7, 1, 0); MI355_DS_READ(fa0[3], w.a_nxt, 6144);
  MM(1, 3, 7, 1, 1); LDA(0);
  MM(1, 3, 6, 0, 1); MI355_DS_READ(fa0[4], w.a_nxt, 8192);
  MM(1, 3, 5, 1, 1);
  MM(1, 3, 4, 0, 1); MI355_DS_READ(fa0[5], w.a_nxt, 10240);
  MM(1, 3, 3, 1, 1); LDA(1);
  MM(1, 3, 2, 0, 1); MI355_DS_READ(fa0[6], w.a_nxt, 12288);
  MM(1, 3, 1, 1, 1);
  MM(1, 3, 0, 0, 1); MI355_DS_READ(fa0[7], w.a_nxt, 14336);
  MM(1, 4, 0, 0, 0); LDA(2);
  MM(1, 4, 1, 1, 0);
  MM(1, 4, 2, 0, 0);
  MM(1, 4, 3, 1, 0);
  MM(1, 4, 4, 0, 0); LDA(3);
  MM(1, 4, 5, 1, 0);
  MM(1, 4, 6, 0, 0);
  MM(1, 4, 7, 1, 0);
  MM(1, 5, 7, 1, 1); LDA(4);
  MM(1, 5, 6, 0, 1);
  MM(1, 5, 5, 1, 1);
  MM(1, 5, 4, 0, 1);
  MM(1, 5, 3, 1, 1); LDA(5);
  MM(1, 5, 2, 0, 1);
  MM(1, 5, 1, 1, 1);
  MM(1, 5, 0, 0, 1);
  MM(1, 6, 0, 0, 0); LDA(6);
  MM(1, 6, 1, 1, 0);
  MM(1, 6, 2, 0, 0);
  MM(1, 6, 3, 1, 0);
  MM(1, 6, 4, 0, 0); LDA(7);
  MM(1, 6, 5, 1, 0);
  MM(1, 6, 6, 0, 0);
  MM(1, 6, 7, 1, 0);
  MM(1, 7, 7, 1, 1);
  MM(1, 7, 6, 0, 1);
  MM(1, 7, 5, 1, 1);
  MM(1, 7, 4, 0, 1);
  MM(1, 7, 3, 1, 1);
  MM(1, 7, 2, 0, 1);
  MM(1, 7, 1, 1, 1);
  MM(1, 7, 0, 0, 1);
  MI355_WAIT_FRAGS16(fa0, fb0);
#undef MM
#undef LDA
#undef LDB
#undef SCL_A
#undef SCL_B
}

// Pre-pass: scales from row-major [rows][k32] to the per-lane order the main loop loads, both operands
// in one launch.  One wave per (block of 128 rows, K step); lane (r,g) gathers its 16 bytes and stores them
// as one word.
__global__ void __launch_bounds__(256)
mx_scale_layout_kernel(const uint8_t *__restrict__ SA, const uint8_t *__restrict__ SB, uint8_t *__restrict__ out_a,
                       uint8_t *__restrict__ out_b, uint32_t k32, uint32_t steps, uint32_t units_a, uint32_t units_b) {
  uint32_t unit = blockIdx.x * (blockDim.x / 64u) + threadIdx.x / 64u;
  const uint32_t lane = threadIdx.x % 64u;
  if (unit >= units_a + units_b) return;
  const uint8_t *S = SA;
  uint8_t *out = out_a;
  if (unit >= units_a) { unit -= units_a; S = SB; out = out_b; }
  const uint32_t rb = unit / steps, s = unit % steps, r = lane % 16u, g = lane / 16u;
  uint32_t word[4];
#pragma unroll
  for (uint32_t i = 0; i < 8; i++) {
    const uint8_t *row = S + (size_t)(rb * 128u + 16u * i + r) * k32 + 8u * s + g;
    const uint32_t pair = (uint32_t)row[0] | ((uint32_t)row[4] << 8);
    if (i % 2 == 0) word[i / 2] = pair;
    else word[i / 2] |= pair << 16;
  }
  *reinterpret_cast<uint4 *>(out + ((size_t)unit * 64u + lane) * 16u) = make_uint4(word[0], word[1], word[2], word[3]);
}

__global__ void __launch_bounds__(kThreads)
gemm_mxfp4_kernel(const uint8_t *__restrict__ A, const uint8_t *__restrict__ B, const uint8_t *__restrict__ SAl,
                  const uint8_t *__restrict__ SBl, uint16_t *__restrict__ C, uint32_t N, uint32_t k_bytes,
                  uint32_t tiles_m, uint32_t tiles_n) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const uint32_t tid = threadIdx.x, lane = tid % 64;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const uint32_t wm = wave / 2, wn = wave % 2;
  const TileGrid grid = tiles_of_workgroup(tiles_m, tiles_n);

  MxRing ring;
  MxFrags f;
  // the scale bytes of the first step go out first; the start of the ring waits for every load
  ring.grid = grid;
  ring.steps = k_bytes / kRowBytes;
  ring.sal = SAl; ring.sbl = SBl; ring.wm = wm; ring.wn = wn;
  ring.soff = lane * 16u;
  ring.s_round = 0;
  ring.s_left = ring.steps;
  ring.scales_of(0);
  MI355_SCALE16(f.sa_n, ring.soff, ring.sa_next);
  MI355_SCALE16(f.sb_n, ring.soff, ring.sb_next);
  ring.next_scales();
  ring.start(A, B, k_bytes, (uint32_t)(uintptr_t)lds, wave, lane, grid);
  const uint32_t steps = ring.steps;

  f32x4v acc[8][8];
#pragma unroll
  for (int j = 0; j < 8; j++) asm volatile("ds_read_b128 %0, %1" : "=v"(f.b0[j]) : "v"(ring.w.b_cur + j * 2048u));
#pragma unroll
  for (int i = 0; i < 8; i++) asm volatile("ds_read_b128 %0, %1" : "=v"(f.a0[i]) : "v"(ring.w.a_cur + i * 2048u));
  MI355_WAIT_FRAGS16(f.a0, f.b0);

  // A lane holds 4 consecutive N elements per 16x16 tile.  Two neighbouring tiles (j, j+1) trade halves
  // first (v_permlane16_swap: the odd lane groups of tile j against the even groups of tile j+1), so that a
  // lane stores 8 consecutive bf16 and an instruction 64 contiguous bytes per row instead of 32.
  const uint32_t g = lane / 16u;
  const uint32_t row_in_tile = wm * 128u + lane % 16u, col_in_tile = wn * 128u + 16u * (g & 1u) + 8u * (g >> 1);

  for (uint32_t round = 0; round < grid.mine; round++) {
    mx_step<true>(acc, f, ring);
    ring.advance_all();
    for (uint32_t s = 1; s < steps; s++) {
      mx_step<false>(acc, f, ring);
      ring.advance_all();
    }
    // wait states the compiler cannot know about before the accumulators are read (the operands tie the
    // youngest results to this point), then this wave's loads but the 8 youngest before any store
    asm volatile("s_nop 15\n s_nop 15\n s_waitcnt vmcnt(8)"
                 : "+a"(acc[7][4]), "+a"(acc[7][5]), "+a"(acc[7][6]), "+a"(acc[7][7]) :: "memory");
    uint32_t tm, tn;
    tile_at(grid, round, tm, tn);
    const uint32_t row0 = tm * kTile + row_in_tile, col0 = tn * kTile + col_in_tile;
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
      for (int jp = 0; jp < 8; jp += 2) {
        const uint32_t p00 = mi355_pack_bf16x2(acc[i][jp][0], acc[i][jp][1]), p01 = mi355_pack_bf16x2(acc[i][jp][2], acc[i][jp][3]);
        const uint32_t p10 = mi355_pack_bf16x2(acc[i][jp + 1][0], acc[i][jp + 1][1]), p11 = mi355_pack_bf16x2(acc[i][jp + 1][2], acc[i][jp + 1][3]);
        const auto q01 = __builtin_amdgcn_permlane16_swap(p00, p10, false, false);
        const auto q23 = __builtin_amdgcn_permlane16_swap(p01, p11, false, false);
        *reinterpret_cast<uint4 *>(C + (size_t)(row0 + i * 16u) * N + col0 + jp * 16u) = make_uint4(q01[0], q23[0], q01[1], q23[1]);
      }
  }
  MI355_DRAIN_RING();
}

}  // namespace

extern "C" int mi355_gemm_mxfp4(mi355_dev *dev, const uint8_t *A, const uint8_t *B, const uint8_t *scale_a,
                                const uint8_t *scale_b, uint16_t *C, uint32_t M, uint32_t N, uint32_t K) {
  MI355_ENTER(dev);
  MI355_REQUIRE(dev, A && B && C && scale_a && scale_b, "gemm_mxfp4: null buffer");
  MI355_REQUIRE(dev, M > 0 && N > 0 && K > 0, "gemm_mxfp4: empty problem");
  MI355_REQUIRE(dev, M % kTile == 0 && N % kTile == 0, "gemm_mxfp4: M (%u) and N (%u) must be multiples of 256", M, N);
  MI355_REQUIRE(dev, K % 256 == 0, "gemm_mxfp4: K (%u) must be a multiple of 256", K);
  MI355_REQUIRE(dev, (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15u) == 0, "gemm_mxfp4: buffers must be 16-byte aligned");
  if (int rc = allow_full_lds(dev, &gemm_mxfp4_kernel, kLdsMxfp4)) return rc;
  // lane-ordered copies of the scales live in a scratch buffer the handle keeps (same size as the scales)
  const uint32_t k32 = K / 32u, steps = K / 256u;
  const size_t sa_bytes = (size_t)M * k32, sb_bytes = (size_t)N * k32;
  if (dev->mx_scratch_bytes < sa_bytes + sb_bytes) {
    MI355_HIP(dev, hipStreamSynchronize(dev->stream));
    if (dev->mx_scratch) MI355_HIP(dev, hipFree(dev->mx_scratch));
    dev->mx_scratch = nullptr;
    dev->mx_scratch_bytes = 0;
    const hipError_t e = hipMalloc(&dev->mx_scratch, sa_bytes + sb_bytes);
    if (e != hipSuccess) return mi355_fail(dev, e == hipErrorOutOfMemory ? MI355_ERR_OOM : MI355_ERR_HIP,
                                           "gemm_mxfp4: scratch of %zu bytes: %s", sa_bytes + sb_bytes, hipGetErrorString(e));
    dev->mx_scratch_bytes = sa_bytes + sb_bytes;
  }
  uint8_t *sal = static_cast<uint8_t *>(dev->mx_scratch), *sbl = sal + sa_bytes;
  const uint32_t units_a = M / 128u * steps, units_b = N / 128u * steps;
  mx_scale_layout_kernel<<<(units_a + units_b + 3) / 4, 256, 0, dev->stream>>>(scale_a, scale_b, sal, sbl, k32, steps, units_a, units_b);
  MI355_LAUNCH_CHECK(dev, "mx_scale_layout");
  const uint32_t tiles_m = M / kTile, tiles_n = N / kTile;
  gemm_mxfp4_kernel<<<gemm_workgroups(dev, tiles_m * tiles_n), kThreads, kRingBytes, dev->stream>>>(A, B, sal, sbl, C, N, K / 2u, tiles_m, tiles_n);
  MI355_LAUNCH_CHECK(dev, "gemm_mxfp4");
  return MI355_OK;
}
