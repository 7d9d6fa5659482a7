// Hand-written MFMA GEMM:  C[M][N] = scale * A[M][K] . B[N][K]^T.  Both operands are K-contiguous
// ("row-major A, column-major B").  Operand types: bf16, f16, fp8 (e4m3, or an e5m2 A against an e4m3 B) and
// block-scaled e2m1 (entry point and scale pre-pass in gemm_mxfp4.hip) with fp32 accumulation and a 16-bit C;
// int8 with an int32 C; fp32.  The tile walk, the LDS ring and the persistent workgroups live in gemm_ring.h.
//
// Tiling.  One workgroup of 512 threads (8 waves, 2 per SIMD) owns a 256x256 tile
// of C and walks K in steps of one 128-byte row segment (64 bf16 or 128 fp8
// elements): per step an A slab and a B slab of 256 rows x 128 B = 32 KiB each.  Waves
// form a 2 (M) x 4 (N) grid; each wave owns 128x64 of C = 8x4 MFMA tiles of 16x16,
// 128 fp32 accumulators per lane.
//
// LDS ring.  All 160 KiB of the CU's LDS are five 32 KiB slots; the A slab of step t
// lives in slot 2t mod 5, its B slab in slot (2t+1) mod 5.  When the barrier of step s
// frees the two slots of slab s, the B slab of step s+2 is fetched into the old A slot
// and the A slab of step s+3 into the old B slot: two and a half slabs are resident or
// in flight at any time, half of the fetches have two steps to land, and the fill path
// always has work queued.  Loads return in order, so the wait before a barrier lets the
// wave's 4 youngest loads (the A rows three steps ahead) stay in flight.
//
// Data movement.  Global memory goes straight into LDS (global_load_lds_dwordx4, 16
// bytes per lane, no staging registers, no ds_write): one such instruction moves 8
// rows x 128 B; a wave issues 4 for its B rows and 4 for its A rows per step, spread
// over the whole step.
//
// LDS layout.  A row's 128 bytes are eight 16-byte chunks; chunk c of row r is stored
// at chunk position c ^ (r & 7).  A fragment read (16 lanes = 16 consecutive rows,
// same logical chunk) then spreads over all eight chunk positions instead of hitting
// one bank group 16 times.  The direct-to-LDS load writes lane i at position i of its
// 1 KiB destination, so lane i fetches the global chunk that belongs there.
//
// Schedule of one step (gemm_ring_step): 32 slots per wave, one per 16x16 tile of its 128x64, each slot 32
// cycles of the matrix pipe: one K=128 fp8 instruction, or two K=32 (bf16, f16) / K=64 (int8) instructions on
// the two K halves of the slab, back to back on the same accumulator.  There are no registers for a second
// set of fragments (128 accumulators + 96 fragment registers), so fragments are reloaded in place as soon as
// their last use has issued, with counted waits so that a row starts as soon as its own fragment has arrived;
// one barrier per step, placed as early as the fragment reads allow.  The loop body is inline assembly so
// that this order is the order issued; the compiler knows neither the LDS reads nor the MFMAs and therefore
// inserts no wait states of its own: every s_waitcnt below is part of the schedule.
//
// The MFMA is issued with the B fragment as the first operand, which produces the
// transposed 16x16 tile: a lane then holds 4 consecutive N elements of one C row (see store_tile for
// how they leave).
//
// Workgroups are persistent: one per CU (the ring takes the whole LDS), each walking the
// tiles id, id + grid, id + 2*grid, ...  The ring does not stop at a tile boundary: slabs are
// numbered through all tiles of the workgroup, so while the last steps of one tile compute, the
// first slabs of the next tile are already being fetched, and the only time the matrix pipe is
// not fed between two tiles is the time it takes to convert and store the accumulators.  After
// its last tile a workgroup keeps fetching (the slabs of its first tile again, which nobody
// reads) so that every step is the same code; those loads are waited for before the wave ends.
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

// Output types of store_tile: bf16, f16, int32 (bits as they are), bf16 after a scale (the fp8 kinds).
enum { kBf16 = 0, kF16 = 1, kI8 = 2, kScaledBf16 = 3 };

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

// Store a wave's 128x64 accumulators.  A lane holds 4 consecutive N elements of one row per 16x16 tile
// (8 bytes of bf16 / f16, 16 bytes of int32), lane group g = lane/16 the 4 elements 4g..4g+3.  Stored as
// they are, the four groups of a 16-bit row would write 32 contiguous bytes per instruction, a quarter of a
// cache line; with every workgroup of the part storing its tile at the same moment that pattern reaches
// 4.7 TB/s where 64-byte pieces reach 7.0 TB/s.  So two neighbouring tiles (j, j+1) first trade halves:
// v_permlane16_swap exchanges the odd lane groups of tile j with the even groups of tile j+1, after which
// groups 0,2 hold columns 0..7 and 8..15 of tile j and groups 1,3 those of tile j+1, 16 bytes per lane,
// 64 contiguous bytes per row and instruction.
template <int KIND>
__device__ __forceinline__ void store_tile(const f32x4v (&acc)[8][4], void *__restrict__ Cout, uint32_t N, uint32_t row0,
                                           uint32_t col0, uint32_t lane, float scale) {
  if (KIND == kI8) {
    const uint32_t col = col0 + 4u * (lane / 16u);
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
      for (int j = 0; j < 4; j++) {
        i32x4v bits;
        __builtin_memcpy(&bits, &acc[i][j], sizeof(bits));
        *reinterpret_cast<i32x4v *>(static_cast<int32_t *>(Cout) + (size_t)(row0 + i * 16u) * N + col + j * 16u) = bits;
      }
    return;
  }
  const uint32_t g = lane / 16u;
  const uint32_t col = col0 + 16u * (g & 1u) + 8u * (g >> 1);   // of the pair (0,1); the pair (2,3) is 32 further
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int jp = 0; jp < 4; jp += 2) {
      uint32_t p[2][2];   // [tile of the pair][elements 0,1 | 2,3]
#pragma unroll
      for (int t = 0; t < 2; t++)
#pragma unroll
        for (int h = 0; h < 2; h++) {
          float lo = acc[i][jp + t][2 * h], hi = acc[i][jp + t][2 * h + 1];
          if (KIND == kScaledBf16) { lo *= scale; hi *= scale; }
          p[t][h] = KIND == kF16 ? mi355_pack_f16x2(lo, hi) : mi355_pack_bf16x2(lo, hi);
        }
      // q[0]: this group's elements 0..1 (even groups: of tile jp, odd groups: of tile jp+1), q[1]: the next
      // group's elements 0..1 of the same tile, i.e. elements 4..5 of the 8 contiguous ones
      const auto q01 = __builtin_amdgcn_permlane16_swap(p[0][0], p[1][0], false, false);
      const auto q23 = __builtin_amdgcn_permlane16_swap(p[0][1], p[1][1], false, false);
      const uint4 packed = make_uint4(q01[0], q23[0], q01[1], q23[1]);
      *reinterpret_cast<uint4 *>(static_cast<uint16_t *>(Cout) + (size_t)(row0 + i * 16u) * N + col + jp * 16u) = packed;
    }
}

// ---- the step of the 4-, 8- and 16-bit kinds -----------------------------------------------------------
// A slab of 128 bytes per row is one K=128 fp8 instruction per 16x16 tile, or two instructions of the
// 16-bit / int8 kinds.  A lane's operand bytes are the two 16-byte chunks g and g+4 of its row (g = lane/16),
// which in the swizzled layout are the addresses x and x^64: two ds_read_b128 fill the low and the high half
// (the 8-register fp8 operand, or the operands of the first and of the second instruction of a pair).
//
// Fragments are reloaded in place as soon as their last use has issued.  The 32 slots run as two sweeps over
// the 8 A fragments, first against B fragments 0,1 and then against 2,3:
//     MFMA  0..9    (i,0),(i,1): this step's A fragment 7 and B fragments 2,3 are read in gaps 0..2;
//                   counted waits let row i start as soon as its own fragment has arrived
//     wait all reads; wait own loads but the 4 youngest; barrier   <- slab s+1 complete, slab s free
//     MFMA 10..15   the wave's 4 loads of B rows (slab s+2)
//     MFMA 16..31   (i,2),(i,3): next step's B fragments 0,1 in gaps 16,17, next step's A fragment
//                   i-1 after row i (a fragment is overwritten no sooner than one instruction after
//                   its last use); the wave's 4 loads of A rows (slab s+3) in the even gaps 18..24
// What one (i, j) slot of the step issues on a lane's two 16-byte halves (first and second K half of the slab):
//   fp8: one K=128 instruction on the 32-byte operands (e5m2 A: format field blgp, the A fragment being the
//        second source of the transposed product);
//   bf16 / f16 / int8: two instructions, first half then second, BACK TO BACK ON THE SAME ACCUMULATOR.  The
//        matrix pipe forwards the accumulator to the next instruction that names it, so the pair issues like
//        two independent instructions, and an instruction that names its predecessor's accumulator costs less
//        power than one that switches (see mfma_dense.hip), which is what bounds these kernels.
//   block-scaled e2m1: likewise two K=128 instructions (a 16-byte chunk is 32 codes, one scale block), each
//        with the scale bytes of its blocks; the wave's scale bytes of the next step are requested at the top
//        of the step, ahead of its 8 loads into LDS, and waited for at the top of the next.
enum { kOpE4m3 = 0, kOpE5m2 = 1, kOpBf16 = 2, kOpF16 = 3, kOpI8 = 4, kOpMx = 5 };
#define MI355_MFMA_SLOT(OP, acc, blo, bhi, alo, ahi)                                               \
  do {                                                                                             \
    if (OP == kOpE4m3 || OP == kOpE5m2) {                                                          \
      const i32x8v b8_ = __builtin_shufflevector(blo, bhi, 0, 1, 2, 3, 4, 5, 6, 7);                \
      const i32x8v a8_ = __builtin_shufflevector(alo, ahi, 0, 1, 2, 3, 4, 5, 6, 7);                \
      if (OP == kOpE5m2)                                                                           \
        asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0 blgp:1" : "+v"(acc) : "v"(b8_), "v"(a8_));       \
      else                                                                                         \
        asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+v"(acc) : "v"(b8_), "v"(a8_)); \
    } else if (OP == kOpBf16) {                                                                    \
      asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0\n v_mfma_f32_16x16x32_bf16 %0, %3, %4, %0" \
                   : "+v"(acc) : "v"(blo), "v"(alo), "v"(bhi), "v"(ahi));                          \
    } else if (OP == kOpF16) {                                                                     \
      asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0\n v_mfma_f32_16x16x32_f16 %0, %3, %4, %0" \
                   : "+v"(acc) : "v"(blo), "v"(alo), "v"(bhi), "v"(ahi));                          \
    } else {                                                                                       \
      asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0\n v_mfma_i32_16x16x64_i8 %0, %3, %4, %0"   \
                   : "+v"(acc) : "v"(blo), "v"(alo), "v"(bhi), "v"(ahi));                          \
    }                                                                                              \
  } while (0)

// Block-scaled e2m1 (OCP MXFP4): the pair of a slot with the scale bytes of its two K halves.  A lane's 16-byte
// chunk is the 32 codes of one scale block; byte (op_sel + 2 * op_sel_hi) of the scale register is used:
// op_sel = K half, op_sel_hi = parity of the fragment (JB for B, IB for A), register = fragment / 2.
#define MI355_MFMA_MX_PAIR(JB, IB, acc, blo, bhi, alo, ahi, sb, sa)                                \
  asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %5, %6 op_sel:[0,0,0] op_sel_hi:[" #JB "," #IB ",0] cbsz:4 blgp:4\n" \
               "v_mfma_scale_f32_16x16x128_f8f6f4 %0, %3, %4, %0, %5, %6 op_sel:[1,1,0] op_sel_hi:[" #JB "," #IB ",0] cbsz:4 blgp:4"   \
               : "+v"(acc) : "v"(blo), "v"(alo), "v"(bhi), "v"(ahi), "v"(sb), "v"(sa))
#define MI355_PARITY_0 0
#define MI355_PARITY_1 1
#define MI355_PARITY_2 0
#define MI355_PARITY_3 1
#define MI355_PARITY_4 0
#define MI355_PARITY_5 1
#define MI355_PARITY_6 0
#define MI355_PARITY_7 1
#define MI355_MX_SLOT2(JB, IB, acc, blo, bhi, alo, ahi, sb, sa) MI355_MFMA_MX_PAIR(JB, IB, acc, blo, bhi, alo, ahi, sb, sa)
#define MI355_MX_SLOT(i, j, acc, blo, bhi, alo, ahi, sb, sa) \
  MI355_MX_SLOT2(MI355_PARITY_##j, MI355_PARITY_##i, acc, blo, bhi, alo, ahi, sb, sa)

// The scale bytes of a wave, per lane: byte 2i+h of `sa` belongs to A fragment i, K half h (16 bytes for the
// 8 fragments), byte 2j+h of `sb` to B fragment j (8 bytes).  They do not pass through LDS (it is full): a
// pre-pass has written them in this order, and the step loads those of the next step with one instruction per
// operand, the wave's oldest loads of the step.
struct MxScales {
  i32x4v sa, sa_n;
  i32x2v sb, sb_n;
  uint64_t sa_next, sb_next;   // uniform addresses of the next step's 1 KiB (A) and 512 bytes (B)
  uint32_t off_a, off_b;       // this lane's offset there
};

// At most `n` LDS reads still outstanding (they return in order).
#define MI355_WAIT_LGKM(n) asm volatile("s_waitcnt lgkmcnt(" #n ")" ::: "memory")

struct RingFrags {
  i32x4v a_lo[8], a_hi[8], b_lo[4], b_hi[4];
};

template <int OP>
__device__ __forceinline__ void gemm_ring_step(f32x4v (&acc)[8][4], RingFrags &f, const GemmWalk &w, uint32_t first,
                                               MxScales &sc) {
  constexpr bool READS = true;
  const uint32_t a_hi = w.a_cur ^ 64u, b_hi = w.b_cur ^ 64u, an_hi = w.a_nxt ^ 64u, bn_hi = w.b_nxt ^ 64u;
  if constexpr (OP == kOpMx) {
    // this step's scale bytes were requested a step ago, ahead of that step's 8 loads into LDS (in the first
    // step of a tile they were waited for at the end of the tile before, and the stores since must not count)
    asm volatile("s_cmp_lg_u32 %2, 0\n s_cbranch_scc1 1f\n s_waitcnt vmcnt(8)\n1:" : "+v"(sc.sa_n), "+v"(sc.sb_n) : "s"(first) : "scc");
    sc.sa = sc.sa_n;
    sc.sb = sc.sb_n;
    // ordinary vector moves; the matrix instruction that reads one as a scale must not issue right behind it
    asm volatile("s_nop 7" : "+v"(sc.sa), "+v"(sc.sb));
    // the next step's scale bytes: the wave's oldest loads of this step, a whole step to land
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(sc.sa_n) : "v"(sc.off_a), "s"(sc.sa_next) : "memory");
    asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(sc.sb_n) : "v"(sc.off_b), "s"(sc.sb_next) : "memory");
  }
#define MM(i, j)                                                                                   \
  do {                                                                                             \
    if constexpr (OP == kOpMx)                                                                     \
      MI355_MX_SLOT(i, j, acc[i][j], f.b_lo[j], f.b_hi[j], f.a_lo[i], f.a_hi[i], sc.sb[(j) / 2], sc.sa[(i) / 2]); \
    else                                                                                           \
      MI355_MFMA_SLOT(OP, acc[i][j], f.b_lo[j], f.b_hi[j], f.a_lo[i], f.a_hi[i]);                  \
  } while (0)
#define LDA(q) MI355_LOAD_LDS(w.voff, w.ga + (uint64_t)(q) * w.row8, w.dst_a + (q) * 1024u)
#define LDB(q) MI355_LOAD_LDS(w.voff, w.gb + (uint64_t)(q) * w.row8, w.dst_b + (q) * 1024u)
#define RD_A_NEXT(i, off)                                                                          \
  if (READS) { MI355_DS_READ(f.a_lo[i], w.a_nxt, off); MI355_DS_READ(f.a_hi[i], an_hi, off); }
#define RD_B_NEXT(j, off)                                                                          \
  if (READS) { MI355_DS_READ(f.b_lo[j], w.b_nxt, off); MI355_DS_READ(f.b_hi[j], bn_hi, off); }
  // On entry the reads of B fragments 0,1 and A fragments 0..6 of this step are in flight, in that order.
  MI355_WAIT_LGKM(12);                                   // B0, B1, A0 have arrived
  MM(0, 0); MI355_DS_READ(f.a_lo[7], w.a_cur, 14336); MI355_DS_READ(f.a_hi[7], a_hi, 14336);
  MM(0, 1); MI355_DS_READ(f.b_lo[2], w.b_cur, 4096); MI355_DS_READ(f.b_hi[2], b_hi, 4096);
  MI355_WAIT_LGKM(14);                                   // A1
  MM(1, 0); MI355_DS_READ(f.b_lo[3], w.b_cur, 6144); MI355_DS_READ(f.b_hi[3], b_hi, 6144);
  MM(1, 1);
  MI355_WAIT_LGKM(14);                                   // A2
  MM(2, 0); MM(2, 1);
  MI355_WAIT_LGKM(12);                                   // A3
  MM(3, 0); MM(3, 1);
  MI355_WAIT_LGKM(10);                                   // A4
  MM(4, 0); MM(4, 1);
  // every read of this step's slab has returned (its two slots are free); with the 4 A loads of the
  // last step still allowed in flight, this wave's share of the next slab has landed
  // (block-scaled kind: the two scale loads of this step are younger still)
  if constexpr (OP == kOpMx) MI355_STEP_BARRIER(first, "s_waitcnt lgkmcnt(0)\n", "6");
  else MI355_STEP_BARRIER(first, "s_waitcnt lgkmcnt(0)\n", "4");
  MM(5, 0); LDB(0);
  MM(5, 1);
  MM(6, 0); LDB(1);
  MM(6, 1);
  MM(7, 0); LDB(2);
  MM(7, 1); LDB(3);
  MM(0, 2); RD_B_NEXT(0, 0);
  MM(0, 3); RD_B_NEXT(1, 2048);
  MM(1, 2); LDA(0);
  MM(1, 3); RD_A_NEXT(0, 0);
  MM(2, 2); LDA(1);
  MM(2, 3); RD_A_NEXT(1, 2048);
  MM(3, 2); LDA(2);
  MM(3, 3); RD_A_NEXT(2, 4096);
  MM(4, 2); LDA(3);
  MM(4, 3); RD_A_NEXT(3, 6144);
  MM(5, 2);
  MM(5, 3); RD_A_NEXT(4, 8192);
  MM(6, 2);
  MM(6, 3); RD_A_NEXT(5, 10240);
  MM(7, 2);
  MM(7, 3); RD_A_NEXT(6, 12288);
#undef RD_A_NEXT
#undef RD_B_NEXT
#undef LDA
#undef LDB
#undef MM
}

template <int OP>
__global__ void __launch_bounds__(kThreads)
gemm_ring_kernel(const uint8_t *__restrict__ A, const uint8_t *__restrict__ B, void *__restrict__ C,
                uint32_t N, uint32_t k_bytes, float scale, uint32_t tiles_m, uint32_t tiles_n,
                const uint8_t *__restrict__ scales_a, const uint8_t *__restrict__ scales_b) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const uint32_t tid = threadIdx.x, lane = tid % 64;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const uint32_t wm = wave / 4, wn = wave % 4;
  const TileGrid grid = tiles_of_workgroup(tiles_m, tiles_n);

  // block-scaled kind: the stream of lane-ordered scale bytes, one step ahead of the slab being multiplied
  // (per block of 128 A rows / 64 B rows and step 1 KiB / 512 bytes, the steps of a block consecutive)
  MxScales sc{};
  const uint32_t steps_of_tile = k_bytes / kRowBytes;
  uint32_t s_round = 0, s_left = steps_of_tile;
  auto scales_of = [&](uint32_t rnd) {
    uint32_t tm, tn;
    tile_at(grid, rnd, tm, tn);
    sc.sa_next = (uint64_t)(uintptr_t)(scales_a + (size_t)(tm * 2u + wm) * steps_of_tile * 1024u);
    sc.sb_next = (uint64_t)(uintptr_t)(scales_b + (size_t)(tn * 4u + wn) * steps_of_tile * 512u);
  };
  auto next_scales = [&]() {
    if (--s_left == 0u) {
      s_round = s_round + 1u == grid.mine ? 0u : s_round + 1u;
      scales_of(s_round);
      s_left = steps_of_tile;
    } else {
      sc.sa_next += 1024;
      sc.sb_next += 512;
    }
  };
  if constexpr (OP == kOpMx) {   // the first step's scales go out first; the start of the ring waits for every load
    sc.off_a = lane * 16u;
    sc.off_b = lane * 8u;
    scales_of(0);
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(sc.sa_n) : "v"(sc.off_a), "s"(sc.sa_next) : "memory");
    asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(sc.sb_n) : "v"(sc.off_b), "s"(sc.sb_next) : "memory");
    next_scales();
  }

  Ring ring;
  ring.start(A, B, k_bytes, (uint32_t)(uintptr_t)lds, wave, lane, grid);
  const uint32_t steps = ring.steps;

  f32x4v acc[8][4];
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = (f32x4v){0.f, 0.f, 0.f, 0.f};
  RingFrags f;
  // what a step expects in flight on entry: B fragments 0,1 then A fragments 0..6
  {
    const GemmWalk &w = ring.w;
    const uint32_t a_hi = w.a_cur ^ 64u, b_hi = w.b_cur ^ 64u;
    MI355_DS_READ(f.b_lo[0], w.b_cur, 0); MI355_DS_READ(f.b_hi[0], b_hi, 0);
    MI355_DS_READ(f.b_lo[1], w.b_cur, 2048); MI355_DS_READ(f.b_hi[1], b_hi, 2048);
    MI355_DS_READ(f.a_lo[0], w.a_cur, 0); MI355_DS_READ(f.a_hi[0], a_hi, 0);
    MI355_DS_READ(f.a_lo[1], w.a_cur, 2048); MI355_DS_READ(f.a_hi[1], a_hi, 2048);
    MI355_DS_READ(f.a_lo[2], w.a_cur, 4096); MI355_DS_READ(f.a_hi[2], a_hi, 4096);
    MI355_DS_READ(f.a_lo[3], w.a_cur, 6144); MI355_DS_READ(f.a_hi[3], a_hi, 6144);
    MI355_DS_READ(f.a_lo[4], w.a_cur, 8192); MI355_DS_READ(f.a_hi[4], a_hi, 8192);
    MI355_DS_READ(f.a_lo[5], w.a_cur, 10240); MI355_DS_READ(f.a_hi[5], a_hi, 10240);
    MI355_DS_READ(f.a_lo[6], w.a_cur, 12288); MI355_DS_READ(f.a_hi[6], a_hi, 12288);
  }

  // one loop over the steps of all tiles of the workgroup
  uint32_t round = 0, left = steps, first = 1;
  for (uint32_t g = grid.mine * steps; g > 0; g--) {
    gemm_ring_step<OP>(acc, f, ring.w, first, sc);
    ring.advance();
    if constexpr (OP == kOpMx) next_scales();
    first = 0;
    if (--left == 0) {
      MI355_END_OF_TILE(acc);
      uint32_t tm, tn;
      tile_at(grid, round, tm, tn);
      store_tile<(OP == kOpBf16 || OP == kOpMx ? kBf16 : OP == kOpF16 ? kF16 : OP == kOpI8 ? kI8 : kScaledBf16)>(
          acc, C, N, tm * kTile + wm * 128u + lane % 16u, tn * kTile + wn * 64u, lane, scale);
#pragma unroll
      for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = (f32x4v){0.f, 0.f, 0.f, 0.f};
      round++;
      left = steps;
      first = 1;
    }
  }
  MI355_DRAIN_RING();
}

// ---- fp32 ----------------------------------------------------------------------------------------
// Same tiling, ring, loads and LDS layout, but two fragment sets (one per K half); a 128-byte row segment is
// 32 floats.  The fp32 matrix
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
                 uint32_t elem) {
  MI355_REQUIRE(dev, A && B && C, "gemm: null buffer");
  MI355_REQUIRE(dev, M > 0 && N > 0 && K > 0, "gemm: empty problem");
  MI355_REQUIRE(dev, M % kTile == 0 && N % kTile == 0, "gemm: M (%u) and N (%u) must be multiples of 256", M, N);
  MI355_REQUIRE(dev, (K * elem) % kRowBytes == 0, "gemm: K (%u) must be a multiple of %u", K, kRowBytes / elem);
  MI355_REQUIRE(dev, (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15u) == 0, "gemm: buffers must be 16-byte aligned");
  return MI355_OK;
}

int g_quad = 1;
template <int OP>
int launch_ring(mi355_dev *dev, const char *what, const void *A, const void *B, void *C, uint32_t M,
               uint32_t N, uint32_t K, uint32_t elem, float scale) {
  if (int rc = check_shapes(dev, A, B, C, M, N, K, elem)) return rc;
  if (g_quad) return mi355_launch_gemm_quad(dev, OP, what, A, B, C, M, N, K * elem, scale);
  if (int rc = allow_full_lds(dev, &gemm_ring_kernel<OP>, kLdsRing0 + OP)) return rc;
  const uint32_t tiles_m = M / kTile, tiles_n = N / kTile;
  gemm_ring_kernel<OP><<<gemm_workgroups(dev, tiles_m * tiles_n), kThreads, kRingBytes, dev->stream>>>(
      (const uint8_t *)A, (const uint8_t *)B, C, N, K * elem, scale, tiles_m, tiles_n, nullptr, nullptr);
  MI355_LAUNCH_CHECK(dev, what);
  return MI355_OK;
}

}  // namespace

// The block-scaled FP4 product on the ring kernel; the caller (gemm_mxfp4.hip) has checked the shapes and laid
// the scale bytes out per lane: A in blocks of 128 rows (16 bytes per lane and step), B in blocks of 64 rows (8).
int mi355_launch_gemm_mx_ring(mi355_dev *dev, const uint8_t *A, const uint8_t *B, const uint8_t *scales_a,
                              const uint8_t *scales_b, uint16_t *C, uint32_t M, uint32_t N, uint32_t K) {
  if (int rc = allow_full_lds(dev, &gemm_ring_kernel<kOpMx>, kLdsRing0 + kOpMx)) return rc;
  const uint32_t tiles_m = M / kTile, tiles_n = N / kTile;
  gemm_ring_kernel<kOpMx><<<gemm_workgroups(dev, tiles_m * tiles_n), kThreads, kRingBytes, dev->stream>>>(
      A, B, C, N, K / 2u, 1.0f, tiles_m, tiles_n, scales_a, scales_b);
  MI355_LAUNCH_CHECK(dev, "gemm_mxfp4");
  return MI355_OK;
}

extern "C" void mi355x_use_quad(int v) { g_quad = v; }

extern "C" int mi355_gemm_bf16(mi355_dev *dev, const uint16_t *A, const uint16_t *B, uint16_t *C, uint32_t M,
                               uint32_t N, uint32_t K) {
  MI355_ENTER(dev);
  return launch_ring<kOpBf16>(dev, "gemm_bf16", A, B, C, M, N, K, 2, 1.0f);
}

extern "C" int mi355_gemm_f16(mi355_dev *dev, const uint16_t *A, const uint16_t *B, uint16_t *C, uint32_t M,
                              uint32_t N, uint32_t K) {
  MI355_ENTER(dev);
  return launch_ring<kOpF16>(dev, "gemm_f16", A, B, C, M, N, K, 2, 1.0f);
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
  return launch_ring<kOpI8>(dev, "gemm_i8", A, B, C, M, N, K, 1, 1.0f);
}

extern "C" int mi355_gemm_fp8_e4m3(mi355_dev *dev, const uint8_t *A, const uint8_t *B, uint16_t *C, uint32_t M,
                                   uint32_t N, uint32_t K, float scale_a, float scale_b) {
  MI355_ENTER(dev);
  return launch_ring<kOpE4m3>(dev, "gemm_fp8_e4m3", A, B, C, M, N, K, 1, scale_a * scale_b);
}

extern "C" int mi355_gemm_fp8_e5m2(mi355_dev *dev, const uint8_t *A, const uint8_t *B, uint16_t *C, uint32_t M,
                                   uint32_t N, uint32_t K, float scale_a, float scale_b) {
  MI355_ENTER(dev);
  return launch_ring<kOpE5m2>(dev, "gemm_fp8_e5m2", A, B, C, M, N, K, 1, scale_a * scale_b);
}
