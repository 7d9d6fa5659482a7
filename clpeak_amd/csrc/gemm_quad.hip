// The 4-, 8- and 16-bit GEMM kernel:  C[M][N] = scale * A[M][K] . B[N][K]^T, both operands K-contiguous, fp32 (int32)
// accumulation.  One workgroup of FOUR waves, one per SIMD, owns a 256x256 tile of C; a wave owns 128x128 of it,
// 8x8 tiles of 16x16, its 256 accumulators in the accumulation registers.  K is walked in steps of one 128-byte row
// segment (a slab: 256 rows x 128 B = 32 KiB per operand).  Tiles, their order, the LDS layout of a slab (rows
// XOR-swizzled in 16-byte chunks) and the direct global->LDS load are those of gemm_ring.h / gemm.hip.
//
// What this arrangement is for.  A workgroup's slab stream (64 KiB per step, 2048 cycles of the matrix pipe) is bound
// by latency, not by bandwidth: with the real addresses and tile order the part delivers a step's 64 KiB in 0.94 us
// when a CU keeps 0..64 KiB in flight, in 0.67 us at 32..96 KiB and in 0.65 us from 64..128 KiB on, against 0.85 us for
// the matrix instructions.  LDS holds 160 KiB, so at most 32 KiB of it may be "being read" at any time:
//   * the B fragments of a step (8 fragments x 32 bytes per lane) are read in ONE BURST into a second register set
//     during rows 5..7 of the step before, and their slot is free again at the barrier that follows;
//   * the A fragments are streamed, row by row, two rows ahead of the matrix instructions, through four rotating
//     register slots; the A slab being streamed is the only resident slab that is not in flight.
// LDS is three A slots and two B slots of 32 KiB.  Slab s has its A rows in A slot s mod 3, its B rows in B slot
// s mod 2.  A step has two barriers:
//   X (slot 40, row 5 of step s):  every wave's loads of slab s+1 (issued a step and a half before) have landed: the
//                         burst of B(s+1) and the reads of rows 0,1 of A(s+1) follow;
//   Y (slot 60 of step s):  every wave has read B(s+1) into registers and all of A(s): the wave's 16 loads of slab s+3
//                         go out from the top of step s+1 on, into B slot (s+1) mod 2 and A slot s mod 3.
// Between Y and the next X, 128 KiB are in flight; never less than 64 KiB.
//
// A step of a wave is 64 slots (row i = 0..7 of A fragments against the 8 B fragments), each slot the pair of
// instructions on the two K halves of the slab, back to back on one accumulator (one K=128 instruction for fp8).  The
// loop body is inline assembly; every s_waitcnt in it is part of the schedule.  The step is written once per parity
// of s (which B register set is current), so no register is ever copied.  With one wave per SIMD nothing hides a
// bubble, so everything a step does besides its matrix instructions rides on fixed slots (see quad_slot) and the
// boundary between two steps is one countdown and a branch that is not taken.
//
// Workgroups of different XCDs walk K from different starting points (XCD x at step x * steps / 8, wrapping around),
// so that at any moment the part reads eight places of every row instead of one; sums are order-independent up to
// rounding, the int8 kind exactly.
#include "internal.h"
#include "mfma_common.h"
#include "gemm_ring.h"
#include "gemm_quad.h"
#include <utility>

namespace {

constexpr int kQuadThreads = 256;
constexpr uint32_t kSlotA0 = 0, kSlotB0 = 3u * kSlabBytes;   // three A slots, then two B slots

struct QuadFrags {
  i32x4v b_lo[2][8], b_hi[2][8];   // two register sets of B fragments (current step / next step)
  i32x4v a_lo[4], a_hi[4];         // four rotating A fragment slots: row i lives in slot i mod 4
  i32x4v sa[2], sb[2];             // block-scaled kind: the scale bytes of the current / next step (see quad_mx_scales)
};

struct QuadWalk {
  uint32_t a_cur, a_cur_hi;  // LDS address of this lane's A fragment of row 0, first / second K half, in the slot of slab s
  uint32_t a_nxt, a_nxt_hi;  // ... in the slot of slab s+1
  uint32_t lane_a;           // ... within an A slot
  uint32_t b_base, b_base_hi;   // the same for the B fragment, in B slot 0 (B slot 1 is reached through the offset field)
  uint32_t off_cur, off_nxt, off_dst;   // byte offsets of the A slots of slabs s, s+1 and s+2 (uniform)
  uint32_t dst_a;            // LDS destination of this wave's A rows of slab s+2 (uniform)
  uint32_t dst_wave;         // this wave's rows within a slot (uniform)
  uint64_t ga, gb;           // global addresses of this wave's first A / B row of slab s+2 (uniform)
  uint32_t voff[8];          // this lane's byte offset from ga / gb for each of the wave's 8 loads of a slab
  uint32_t first;            // the step is the first of a tile (uniform)
  uint64_t sa_next, sb_next; // block-scaled kind: addresses of the next step's 1 KiB of A / B scale bytes (uniform)
  uint32_t s_off;            // ... and this lane's offset there
};

#define Q_DS_READ(dst, addr, off) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(off))
#define Q_WAIT_LGKM(n) asm volatile("s_waitcnt lgkmcnt(%0)" :: "n"(n) : "memory")

// The accumulators are the accumulation registers a[0:255], named in the instruction text: tile (i, j) of the wave is
// a[4T : 4T+3], T = 8i + j.  The compiler is told once that they are taken (quad_claim_accumulators) and never sees them
// as values: with 256 of 256 in use as operands of its own it finds no allocation without spills.
//
// One matrix instruction of a pair kind, optionally with one direct-to-LDS load riding along: M0 is set before the
// matrix instruction (which is the wait state M0 needs before a load reads it) and the load is issued behind it.
#define Q_INSN_BF16 "v_mfma_f32_16x16x32_bf16"
#define Q_INSN_F16 "v_mfma_f32_16x16x32_f16"
#define Q_INSN_I8 "v_mfma_i32_16x16x64_i8"
#define Q_INSN_F8 "v_mfma_f32_16x16x128_f8f6f4"
template <int OP, int T>
__device__ __forceinline__ void q_mfma(const i32x4v &b, const i32x4v &a) {
#define Q_PLAIN(insn) asm volatile(insn " a[%2:%3], %0, %1, a[%2:%3]" :: "v"(b), "v"(a), "n"(4 * T), "n"(4 * T + 3))
  if constexpr (OP == kQuadBf16) Q_PLAIN(Q_INSN_BF16);
  else if constexpr (OP == kQuadF16) Q_PLAIN(Q_INSN_F16);
  else Q_PLAIN(Q_INSN_I8);
#undef Q_PLAIN
}
template <int OP, int T, int IMM>
__device__ __forceinline__ void q_mfma_load(const i32x4v &b, const i32x4v &a, uint32_t dst, uint32_t voff, uint64_t base) {
#define Q_WITH_LOAD(insn)                                                                                              \
  asm volatile("s_add_u32 m0, %4, %5\n " insn " a[%2:%3], %0, %1, a[%2:%3]\n global_load_lds_dwordx4 %6, %7"           \
               :: "v"(b), "v"(a), "n"(4 * T), "n"(4 * T + 3), "s"(dst), "n"(IMM), "v"(voff), "s"(base) : "memory", "m0", "scc")
  if constexpr (OP == kQuadBf16) Q_WITH_LOAD(Q_INSN_BF16);
  else if constexpr (OP == kQuadF16) Q_WITH_LOAD(Q_INSN_F16);
  else Q_WITH_LOAD(Q_INSN_I8);
#undef Q_WITH_LOAD
}
// fp8: one K=128 instruction on the 32-byte operands (e5m2 A: format field blgp, the A fragment being the second
// source of the transposed product).
template <int OP, int T>
__device__ __forceinline__ void q_mfma8(const i32x8v &b, const i32x8v &a) {
  if constexpr (OP == kQuadE5m2) asm volatile(Q_INSN_F8 " a[%2:%3], %0, %1, a[%2:%3] blgp:1" :: "v"(b), "v"(a), "n"(4 * T), "n"(4 * T + 3));
  else asm volatile(Q_INSN_F8 " a[%2:%3], %0, %1, a[%2:%3]" :: "v"(b), "v"(a), "n"(4 * T), "n"(4 * T + 3));
}
template <int OP, int T, int IMM>
__device__ __forceinline__ void q_mfma8_load(const i32x8v &b, const i32x8v &a, uint32_t dst, uint32_t voff, uint64_t base) {
#define Q_WITH_LOAD8(fmt)                                                                                              \
  asm volatile("s_add_u32 m0, %4, %5\n " Q_INSN_F8 " a[%2:%3], %0, %1, a[%2:%3]" fmt "\n global_load_lds_dwordx4 %6, %7" \
               :: "v"(b), "v"(a), "n"(4 * T), "n"(4 * T + 3), "s"(dst), "n"(IMM), "v"(voff), "s"(base) : "memory", "m0", "scc")
  if constexpr (OP == kQuadE5m2) Q_WITH_LOAD8(" blgp:1");
  else Q_WITH_LOAD8("");
#undef Q_WITH_LOAD8
}

// Block-scaled e2m1 (OCP MXFP4): a lane's 16-byte chunk is the 32 codes of one scale block, so a slot is again a pair of
// K=128 instructions on the two K halves, each with the scale bytes of its blocks.  A wave's scale bytes of a step are
// 16 bytes per lane and operand, byte 2i+h belonging to fragment i, K half h: the instruction takes byte
// (op_sel + 2 * op_sel_hi) of the register it is given: op_sel = K half, op_sel_hi = parity of the fragment, register =
// fragment / 2.  They do not pass through LDS: a pre-pass (gemm_mxfp4.hip) has written them in this order, and a step
// loads those of the next step with one instruction per operand, its oldest loads.
#define Q_INSN_MX "v_mfma_scale_f32_16x16x128_f8f6f4"
template <int T, int H, int JB, int IB>
__device__ __forceinline__ void q_mfma_mx(const i32x4v &b, const i32x4v &a, int sb, int sa) {
  asm volatile(Q_INSN_MX " a[%2:%3], %0, %1, a[%2:%3], %4, %5 op_sel:[%6,%6,0] op_sel_hi:[%7,%8,0] cbsz:4 blgp:4"
               :: "v"(b), "v"(a), "n"(4 * T), "n"(4 * T + 3), "v"(sb), "v"(sa), "n"(H), "n"(JB), "n"(IB));
}
template <int T, int JB, int IB, int IMM>
__device__ __forceinline__ void q_mfma_mx_load(const i32x4v &b, const i32x4v &a, int sb, int sa, uint32_t dst, uint32_t voff, uint64_t base) {
  asm volatile("s_add_u32 m0, %8, %9\n " Q_INSN_MX " a[%2:%3], %0, %1, a[%2:%3], %4, %5 op_sel:[0,0,0] op_sel_hi:[%6,%7,0] cbsz:4 blgp:4\n"
               " global_load_lds_dwordx4 %10, %11"
               :: "v"(b), "v"(a), "n"(4 * T), "n"(4 * T + 3), "v"(sb), "v"(sa), "n"(JB), "n"(IB), "s"(dst), "n"(IMM), "v"(voff), "s"(base)
               : "memory", "m0", "scc");
}

constexpr bool quad_is_fp8(int op) { return op == kQuadE4m3 || op == kQuadE5m2; }

// Slot P of a step of parity PAR (the B register set in use): row i = P / 8 of the A fragments, B fragment j = P % 8.
// Besides its matrix instructions a slot carries its share of everything else a step does, so that nothing is left
// for the boundary between two steps, where a single wave per SIMD has nothing to hide it behind:
//   slots 0, 3, .. 45   one load each (8 of B rows, then 8 of A rows, of slab s+2): the texture path takes a load's
//                       1 KiB in 16 cycles, the four waves' 64 KiB of a step in half of the step
//   slots 8i            the reads of A row i+2 go out (rows 6, 7: rows 0, 1 of slab s+1), then row i must have arrived
//   slot 40             barrier X
//   slots 41..56        the burst of B(s+1)
//   slots 23, 46, 47    the fetch addresses and the A slots move on; slot 57: the fragment addresses
//   slot 60             every read has arrived; barrier Y of the NEXT step
#define Q_PIN() __builtin_amdgcn_sched_barrier(0)
constexpr int kLoadEvery = 3;   // the wave's 16 loads of a slab ride on slots 0, 3, 6, .. 45 (every 2: 5 % slower; 4: the same)
constexpr int kAhead = 2;       // rows between the read of an A fragment and its use (at most 3: four register slots; 3: the same)
constexpr int kSlotX = 40;      // barrier X follows this slot; the 16 reads of the burst follow it, one per slot (36, 43: the same)
constexpr int quad_burst_reads(int from, int to) {   // reads of the burst issued in slots from..to
  int n = 0;
  for (int p = from; p <= to; p++) n += p > kSlotX && p <= kSlotX + 16;
  return n;
}
// loads of the step's own slab that are issued before barrier X (they are the ones that may still be in flight there)
constexpr int kKeepAtX = kSlotX / kLoadEvery + 1 < 16 ? kSlotX / kLoadEvery + 1 : 16;
static_assert(15 * kLoadEvery + 2 <= 57, "the loads of a step and the bookkeeping behind them end before the addresses move on");
static_assert(kAhead >= 1 && kAhead <= 3 && kSlotX + 16 < 60 && kSlotX >= 46 - 16, "schedule of a step");
template <int OP, int PAR, int P>
__device__ __forceinline__ void quad_slot(QuadFrags &f, QuadWalk &w) {
  constexpr int i = P / 8, j = P % 8, sl = i % 4, T = P;
  if constexpr (j == 0) {
    // the reads of the A row kAhead rows on go out (past row 7: of the next slab), then this row's fragment must have
    // arrived: reads return in order, so the count is that of the reads issued behind it (the counter holds 15)
    constexpr int r = i + kAhead;
    if constexpr (r <= 7) {
      Q_DS_READ(f.a_lo[r % 4], w.a_cur, r * 2048);
      Q_DS_READ(f.a_hi[r % 4], w.a_cur_hi, r * 2048);
    } else {
      Q_DS_READ(f.a_lo[r % 4], w.a_nxt, (r - 8) * 2048);
      Q_DS_READ(f.a_hi[r % 4], w.a_nxt_hi, (r - 8) * 2048);
    }
    if constexpr (i >= kAhead) {
      constexpr int behind = 2 * kAhead + quad_burst_reads(8 * (i - kAhead), 8 * i - 1);
      Q_WAIT_LGKM(behind < 15 ? behind : 15);
    }
  }
  constexpr int q = P / kLoadEvery;
  constexpr bool with_load = P % kLoadEvery == 0 && q < 16;
  if constexpr (quad_is_fp8(OP)) {
    const i32x8v b8 = __builtin_shufflevector(f.b_lo[PAR][j], f.b_hi[PAR][j], 0, 1, 2, 3, 4, 5, 6, 7);
    const i32x8v a8 = __builtin_shufflevector(f.a_lo[sl], f.a_hi[sl], 0, 1, 2, 3, 4, 5, 6, 7);
    if constexpr (with_load && q < 8) q_mfma8_load<OP, T, kSlotB0 + PAR * kSlabBytes + q * 1024>(b8, a8, w.dst_wave, w.voff[q], w.gb);
    else if constexpr (with_load) q_mfma8_load<OP, T, (q - 8) * 1024>(b8, a8, w.dst_a, w.voff[q - 8], w.ga);
    else q_mfma8<OP, T>(b8, a8);
  } else if constexpr (OP == kQuadMx) {
    const int sb = f.sb[PAR][j / 2], sa = f.sa[PAR][i / 2];
    if constexpr (with_load && q < 8)
      q_mfma_mx_load<T, j % 2, i % 2, kSlotB0 + PAR * kSlabBytes + q * 1024>(f.b_lo[PAR][j], f.a_lo[sl], sb, sa, w.dst_wave, w.voff[q], w.gb);
    else if constexpr (with_load)
      q_mfma_mx_load<T, j % 2, i % 2, (q - 8) * 1024>(f.b_lo[PAR][j], f.a_lo[sl], sb, sa, w.dst_a, w.voff[q - 8], w.ga);
    else
      q_mfma_mx<T, 0, j % 2, i % 2>(f.b_lo[PAR][j], f.a_lo[sl], sb, sa);
    q_mfma_mx<T, 1, j % 2, i % 2>(f.b_hi[PAR][j], f.a_hi[sl], sb, sa);
  } else {
    if constexpr (with_load && q < 8)
      q_mfma_load<OP, T, kSlotB0 + PAR * kSlabBytes + q * 1024>(f.b_lo[PAR][j], f.a_lo[sl], w.dst_wave, w.voff[q], w.gb);
    else if constexpr (with_load)
      q_mfma_load<OP, T, (q - 8) * 1024>(f.b_lo[PAR][j], f.a_lo[sl], w.dst_a, w.voff[q - 8], w.ga);
    else
      q_mfma<OP, T>(f.b_lo[PAR][j], f.a_lo[sl]);
    q_mfma<OP, T>(f.b_hi[PAR][j], f.a_hi[sl]);
  }
  if constexpr (P == kSlotX) {
    // barrier X: this wave's loads of slab s+1 have landed (the 16 of slab s+2 may be in flight).  In the first step
    // of a tile that wait was done before the stores of the tile before, which must not be counted here.
    asm volatile("s_cmp_lg_u32 %0, 0\n s_cbranch_scc1 1f\n s_waitcnt vmcnt(%1)\n1:\n s_barrier" :: "s"(w.first), "n"(kKeepAtX + (OP == kQuadMx ? 2 : 0)) : "memory", "scc");
  }
  if constexpr (P > kSlotX && P <= kSlotX + 16) {
    // the burst: B fragment r/2, K half r%2 of slab s+1 into the other register set
    constexpr int r = P - kSlotX - 1, jb = r / 2;
    if constexpr (r % 2 == 0) Q_DS_READ(f.b_lo[PAR ^ 1][jb], w.b_base, (PAR ^ 1) * kSlabBytes + jb * 2048);
    else Q_DS_READ(f.b_hi[PAR ^ 1][jb], w.b_base_hi, (PAR ^ 1) * kSlabBytes + jb * 2048);
  }
  if constexpr (P == 7 * kLoadEvery + 1) { Q_PIN(); w.gb += kRowBytes; Q_PIN(); }
  if constexpr (OP == kQuadMx && P == 5) { Q_PIN(); w.sa_next += 1024; w.sb_next += 1024; Q_PIN(); }
  if constexpr (P == kSlotX + 1) { Q_PIN(); w.first = 0; Q_PIN(); }
  if constexpr (P == 15 * kLoadEvery + 1) { Q_PIN(); w.ga += kRowBytes; Q_PIN(); }
  if constexpr (P == 15 * kLoadEvery + 2) {
    Q_PIN();
    const uint32_t t = w.off_cur;
    w.off_cur = w.off_nxt; w.off_nxt = w.off_dst; w.off_dst = t;
    w.dst_a = w.dst_wave + w.off_dst;
    Q_PIN();
  }
  if constexpr (P == 57) {
    Q_PIN();
    w.a_cur = w.a_nxt; w.a_cur_hi = w.a_nxt_hi;
    w.a_nxt = w.lane_a + w.off_nxt; w.a_nxt_hi = w.a_nxt ^ 64u;
    Q_PIN();
  }
  if constexpr (P == 60) {
    // Everything read in this step has arrived; the registers ride along so that nothing that uses them (a copy the
    // compiler might place where control flow joins, the next step) can come before the wait.  Then barrier Y of the
    // next step: every wave has read B(s+1) and all of A(s), whose slots the loads of the next step overwrite.
#define Q_TIE8(x) "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]), "+v"(x[4]), "+v"(x[5]), "+v"(x[6]), "+v"(x[7])
    asm volatile("s_waitcnt lgkmcnt(0)\n s_barrier"
                 : Q_TIE8(f.b_lo[PAR ^ 1]), Q_TIE8(f.b_hi[PAR ^ 1]), "+v"(f.a_lo[0]), "+v"(f.a_hi[0]), "+v"(f.a_lo[1]), "+v"(f.a_hi[1]),
                   "+v"(f.a_lo[2]), "+v"(f.a_hi[2])
                 :: "memory");
  }
}

__device__ __forceinline__ void quad_mx_scales(i32x4v &sa, i32x4v &sb, const QuadWalk &w) {
  asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(sa) : "v"(w.s_off), "s"(w.sa_next) : "memory");
  asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(sb) : "v"(w.s_off), "s"(w.sb_next) : "memory");
}

template <int OP, int PAR, int... Ps>
__device__ __forceinline__ void quad_step(std::integer_sequence<int, Ps...>, QuadFrags &f, QuadWalk &w) {
  if constexpr (OP == kQuadMx) {
    // this step's scale bytes were requested at the top of the step before, ahead of its 16 loads into LDS (in the first
    // step of a tile they were waited for before the stores of the tile before); then those of the next step go out
    asm volatile("s_cmp_lg_u32 %2, 0\n s_cbranch_scc1 1f\n s_waitcnt vmcnt(16)\n1:" : "+v"(f.sa[PAR]), "+v"(f.sb[PAR]) : "s"(w.first) : "scc");
    quad_mx_scales(f.sa[PAR ^ 1], f.sb[PAR ^ 1], w);
  }
  (quad_slot<OP, PAR, Ps>(f, w), ...);
}

// The accumulation registers belong to the hand-written code from here on.
__device__ __forceinline__ void quad_claim_accumulators() {
#define Q_A8(n) "a" #n "0", "a" #n "1", "a" #n "2", "a" #n "3", "a" #n "4", "a" #n "5", "a" #n "6", "a" #n "7", "a" #n "8", "a" #n "9"
  asm volatile("" ::: "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", Q_A8(1), Q_A8(2), Q_A8(3), Q_A8(4), Q_A8(5), Q_A8(6),
               Q_A8(7), Q_A8(8), Q_A8(9), Q_A8(10), Q_A8(11), Q_A8(12), Q_A8(13), Q_A8(14), Q_A8(15), Q_A8(16), Q_A8(17), Q_A8(18),
               Q_A8(19), Q_A8(20), Q_A8(21), Q_A8(22), Q_A8(23), Q_A8(24), "a250", "a251", "a252", "a253", "a254", "a255");
#undef Q_A8
}

// Tile T of the wave out of the accumulation registers (as raw bits), and zero in its place.
template <int T>
__device__ __forceinline__ i32x4v quad_take_tile() {
  int v0, v1, v2, v3;
  asm volatile("v_accvgpr_read_b32 %0, a[%4]\n v_accvgpr_read_b32 %1, a[%5]\n v_accvgpr_read_b32 %2, a[%6]\n v_accvgpr_read_b32 %3, a[%7]\n"
               " v_accvgpr_write_b32 a[%4], 0\n v_accvgpr_write_b32 a[%5], 0\n v_accvgpr_write_b32 a[%6], 0\n v_accvgpr_write_b32 a[%7], 0"
               : "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3) : "n"(4 * T), "n"(4 * T + 1), "n"(4 * T + 2), "n"(4 * T + 3));
  return (i32x4v){v0, v1, v2, v3};
}
template <int R>
__device__ __forceinline__ void quad_zero_register() { asm volatile("v_accvgpr_write_b32 a[%0], 0" :: "n"(R)); }
template <int... Rs>
__device__ __forceinline__ void quad_zero_accumulators(std::integer_sequence<int, Rs...>) {
  (quad_zero_register<Rs>(), ...);
  asm volatile("s_nop 7");
}

// Store a wave's 128x128 accumulators and clear them.  A lane holds 4 consecutive N elements of one row per 16x16 tile
// (the product is issued transposed), lane group g = lane/16 the elements 4g..4g+3.  16-bit kinds: two neighbouring
// tiles (j, j+1) first trade halves (v_permlane16_swap exchanges the odd lane groups of tile j with the even groups of
// tile j+1), after which a lane holds 8 consecutive elements: 16 bytes per lane, 64 contiguous bytes per row and
// instruction.
template <int OP, int I, int JP>
__device__ __forceinline__ void quad_store_pair(void *__restrict__ Cout, uint32_t N, uint32_t row0, uint32_t col0, uint32_t lane, float scale,
                                                bool c_streams) {
  const i32x4v t0 = quad_take_tile<I * 8 + JP>(), t1 = quad_take_tile<I * 8 + JP + 1>();
  if constexpr (OP == kQuadI8) {
    int32_t *dst = static_cast<int32_t *>(Cout) + (size_t)(row0 + I * 16u) * N + col0 + 4u * (lane / 16u) + JP * 16u;
    *reinterpret_cast<i32x4v *>(dst) = t0;
    *reinterpret_cast<i32x4v *>(dst + 16) = t1;
  } else {
    const uint32_t g = lane / 16u;
    const uint32_t col = col0 + 16u * (g & 1u) + 8u * (g >> 1);
    uint32_t p[2][2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
      // (through scalar copies: __builtin_bit_cast applied to an element of a vector reads element 0)
      const int b00 = t0[2 * h], b01 = t0[2 * h + 1], b10 = t1[2 * h], b11 = t1[2 * h + 1];
      float x[2][2] = {{__builtin_bit_cast(float, b00), __builtin_bit_cast(float, b01)},
                       {__builtin_bit_cast(float, b10), __builtin_bit_cast(float, b11)}};
#pragma unroll
      for (int t = 0; t < 2; t++) {
        if constexpr (quad_is_fp8(OP)) { x[t][0] *= scale; x[t][1] *= scale; }
        p[t][h] = OP == kQuadF16 ? mi355_pack_f16x2(x[t][0], x[t][1]) : mi355_pack_bf16x2(x[t][0], x[t][1]);
      }
    }
    const auto q01 = __builtin_amdgcn_permlane16_swap(p[0][0], p[1][0], false, false);
    const auto q23 = __builtin_amdgcn_permlane16_swap(p[0][1], p[1][1], false, false);
    const uint4 packed = make_uint4(q01[0], q23[0], q01[1], q23[1]);
    i32x4v *dst = reinterpret_cast<i32x4v *>(static_cast<uint16_t *>(Cout) + (size_t)(row0 + I * 16u) * N + col + JP * 16u);
    const i32x4v bits = {(int)packed.x, (int)packed.y, (int)packed.z, (int)packed.w};
    // (as text: the compiler merges the two arms of a branch that differ only in the cache policy of a store)
    if (c_streams) asm volatile("global_store_dwordx4 %0, %1, off nt" :: "v"(dst), "v"(bits) : "memory");
    else *dst = bits;
  }
  __builtin_amdgcn_sched_barrier(0);   // one pair of tiles at a time: the fragment registers stay live, few are free
}
template <int OP, int... Qs>
__device__ __forceinline__ void quad_store(std::integer_sequence<int, Qs...>, void *__restrict__ Cout, uint32_t N, uint32_t row0,
                                           uint32_t col0, uint32_t lane, float scale, bool c_streams) {
  (quad_store_pair<OP, Qs / 4, 2 * (Qs % 4)>(Cout, N, row0, col0, lane, scale, c_streams), ...);
  asm volatile("s_nop 7");   // accumulation registers written by the vector unit, read next by the matrix unit
}

template <int OP>
__global__ void __launch_bounds__(kQuadThreads)
gemm_quad_kernel(const uint8_t *__restrict__ A, const uint8_t *__restrict__ B, void *__restrict__ C, uint32_t N, uint32_t k_bytes,
                 float scale, uint32_t tiles_m, uint32_t tiles_n, const uint8_t *__restrict__ scales_a,
                 const uint8_t *__restrict__ scales_b, uint32_t c_streams) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const uint32_t tid = threadIdx.x, lane = tid % 64;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const uint32_t wm = wave / 2, wn = wave % 2;
  const TileGrid grid = tiles_of_workgroup(tiles_m, tiles_n);
  const uint32_t steps = k_bytes / kRowBytes;
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;

  QuadWalk w;
  // global -> LDS: load q of a wave fills rows [wave*64 + 8q, +8) of a slab; lane i is position i%8 of row i/8,
  // which holds logical chunk (i%8) ^ (row & 7) = (i%8) ^ (i/8)
  const uint32_t lchunk = (lane % 8u) ^ (lane / 8u);
#pragma unroll
  for (uint32_t q = 0; q < 8; q++) w.voff[q] = (lane / 8u + 8u * q) * k_bytes + lchunk * 16u;
  w.dst_wave = __builtin_amdgcn_readfirstlane(lds_base + wave * 64u * (uint32_t)kRowBytes);
  // LDS -> fragments: row lane%16 of the wave's rows, logical chunk lane/16 (+4 for the second K half, the address
  // with bit 6 flipped), swizzled with row & 7 = lane & 7
  const uint32_t swz0 = ((lane / 16u) ^ (lane & 7u)) << 4;
  w.lane_a = lds_base + (wm * 128u + lane % 16u) * kRowBytes + swz0;
  w.b_base = lds_base + kSlotB0 + (wn * 128u + lane % 16u) * kRowBytes + swz0;
  w.b_base_hi = w.b_base ^ 64u;
  const uint64_t a_origin = (uint64_t)(uintptr_t)(A + (size_t)wave * 64u * k_bytes);
  const uint64_t b_origin = (uint64_t)(uintptr_t)(B + (size_t)wave * 64u * k_bytes);

  // the fetch stream: slabs numbered through all tiles of the workgroup (after the last tile it runs on into the
  // first tile again, two slabs that nobody reads, so that every step is the same code)
  // Workgroups of different XCDs walk K from different starting points (and wrap around): at any moment the part then
  // reads eight different places of every row instead of the same one.
  uint32_t f_round = 0, f_left = steps, w_left = steps;
  const uint32_t k_rot = (grid.first % 8u) * (steps / 8u);
  auto rows_of = [&](uint32_t rnd) {
    uint32_t tm, tn;
    tile_at(grid, rnd, tm, tn);
    w.ga = a_origin + (uint64_t)tm * kTile * k_bytes;
    w.gb = b_origin + (uint64_t)tn * kTile * k_bytes;
    w.ga += k_rot * kRowBytes;
    w.gb += k_rot * kRowBytes;
    w_left = steps - k_rot;
  };
  auto next_fetch_tile = [&]() {
    f_round = f_round + 1u == grid.mine ? 0u : f_round + 1u;
    rows_of(f_round);
    f_left = steps;
  };
  auto fetch = [&](uint32_t slot_a, uint32_t slot_b) {
#pragma unroll
    for (uint32_t q = 0; q < 8; q++) MI355_LOAD_LDS(w.voff[q], w.gb, w.dst_wave + kSlotB0 + slot_b * kSlabBytes + q * 1024u);
#pragma unroll
    for (uint32_t q = 0; q < 8; q++) MI355_LOAD_LDS(w.voff[q], w.ga, w.dst_wave + kSlotA0 + slot_a * kSlabBytes + q * 1024u);
    w.ga += kRowBytes;
    w.gb += kRowBytes;
    if (--w_left == 0u) { w.ga -= k_bytes; w.gb -= k_bytes; w_left = steps; }
    if (--f_left == 0u) next_fetch_tile();
  };
  // block-scaled kind: the stream of scale bytes, one step ahead of the multiplication and walking K the same way
  // (per block of 128 rows and step 1 KiB, the steps of a block consecutive)
  uint32_t s_round = 0, s_left = steps, sw_left = steps;
  auto scales_of = [&](uint32_t rnd) {
    uint32_t tm, tn;
    tile_at(grid, rnd, tm, tn);
    w.sa_next = (uint64_t)(uintptr_t)(scales_a + ((size_t)(tm * 2u + wm) * steps + k_rot) * 1024u);
    w.sb_next = (uint64_t)(uintptr_t)(scales_b + ((size_t)(tn * 2u + wn) * steps + k_rot) * 1024u);
    sw_left = steps - k_rot;
    s_left = steps;
  };
  auto scales_wrap = [&]() { w.sa_next -= (uint64_t)steps * 1024u; w.sb_next -= (uint64_t)steps * 1024u; sw_left = steps; };
  auto next_scale_tile = [&]() { s_round = s_round + 1u == grid.mine ? 0u : s_round + 1u; scales_of(s_round); };
  QuadFrags f;
  if constexpr (OP == kQuadMx) {   // the first step's scales go out first; the start below waits for every load
    w.s_off = lane * 16u;
    scales_of(0);
    quad_mx_scales(f.sa[0], f.sb[0], w);
    w.sa_next += 1024; w.sb_next += 1024;
    if (--sw_left == 0u) scales_wrap();
    if (--s_left == 0u) next_scale_tile();
  }
  rows_of(0);
  fetch(0, 0);
  fetch(1, 1);
  asm volatile("s_waitcnt vmcnt(16)\n s_barrier" ::: "memory");   // slab 0 (and, older, the first scale bytes) has landed

  quad_claim_accumulators();
  quad_zero_accumulators(std::make_integer_sequence<int, 256>{});
  w.off_cur = 0; w.off_nxt = kSlabBytes; w.off_dst = 2u * kSlabBytes;
  w.dst_a = w.dst_wave + w.off_dst;
  w.a_cur = w.lane_a; w.a_cur_hi = w.a_cur ^ 64u;
  w.a_nxt = w.lane_a + w.off_nxt; w.a_nxt_hi = w.a_nxt ^ 64u;
  w.first = 0;
  {   // what a step expects on entry: the B fragments of its slab in register set 0, rows 0,1 of its A fragments, and
      // its barrier Y behind it
#pragma unroll
    for (int j = 0; j < 8; j++) { Q_DS_READ(f.b_lo[0][j], w.b_base, j * 2048); Q_DS_READ(f.b_hi[0][j], w.b_base_hi, j * 2048); }
#pragma unroll
    for (int r = 0; r < kAhead; r++) { Q_DS_READ(f.a_lo[r], w.a_cur, r * 2048); Q_DS_READ(f.a_hi[r], w.a_cur_hi, r * 2048); }
    asm volatile("s_waitcnt lgkmcnt(0)\n s_barrier"
                 : Q_TIE8(f.b_lo[0]), Q_TIE8(f.b_hi[0]), "+v"(f.a_lo[0]), "+v"(f.a_hi[0]), "+v"(f.a_lo[1]), "+v"(f.a_hi[1]),
                   "+v"(f.a_lo[2]), "+v"(f.a_hi[2]) :: "memory");
  }

  // One countdown to the next event: the fetch stream moves on to its next tile (f_left steps from now), or the tile
  // being multiplied is complete (left steps from now).
  uint32_t round = 0, left = steps;
  auto next_span = [&]() {
    uint32_t m = left < f_left ? left : f_left;
    m = m < w_left ? m : w_left;
    if constexpr (OP == kQuadMx) { m = m < s_left ? m : s_left; m = m < sw_left ? m : sw_left; }
    return m;
  };
  uint32_t span = next_span(), ev = span;
  auto event = [&]() -> bool {   // true after the last tile
    left -= span;
    f_left -= span;
    w_left -= span;
    if (w_left == 0u) { w.ga -= k_bytes; w.gb -= k_bytes; w_left = steps; }   // the fetch stream wraps around to the row's start
    if (f_left == 0u) next_fetch_tile();   // (the step has already moved ga / gb on by a slab: overwritten here)
    if constexpr (OP == kQuadMx) {
      s_left -= span;
      sw_left -= span;
      if (sw_left == 0u) scales_wrap();
      if (s_left == 0u) next_scale_tile();
    }
    bool done = false;
    if (left == 0u) {
      // the wait states the compiler cannot know about, then every load of this wave (the next barrier X then needs
      // no wait of its own, and the stores issued here do not enter its count)
      asm volatile("s_nop 15\n s_nop 15\n s_waitcnt vmcnt(0)" ::: "memory");
      uint32_t tm, tn;
      tile_at(grid, round, tm, tn);
      quad_store<OP>(std::make_integer_sequence<int, 32>{}, C, N, tm * kTile + wm * 128u + lane % 16u, tn * kTile + wn * 128u, lane, scale, c_streams != 0u);
      left = steps;
      w.first = 1;
      done = ++round == grid.mine;
    }
    span = next_span();
    ev = span;
    return done;
  };
  constexpr auto slots = std::make_integer_sequence<int, 64>{};
  for (;;) {
    quad_step<OP, 0>(slots, f, w);
    if (__builtin_expect(--ev == 0u, 0) && event()) break;
    quad_step<OP, 1>(slots, f, w);
    if (__builtin_expect(--ev == 0u, 0) && event()) break;
  }
  MI355_DRAIN_RING();
}

template <int OP>
int launch_quad(mi355_dev *dev, const char *what, const void *A, const void *B, void *C, uint32_t M, uint32_t N, uint32_t k_bytes,
                float scale, const uint8_t *scales_a = nullptr, const uint8_t *scales_b = nullptr) {
  if (int rc = allow_full_lds(dev, &gemm_quad_kernel<OP>, kLdsQuad0 + OP)) return rc;
  const uint32_t tiles_m = M / kTile, tiles_n = N / kTile;
  // A 16-bit C goes past the caches (non-temporal stores) when the operands alone fill the 256 MiB last-level cache: C
  // lines kept there would only push out operand rows that the next round of tiles reads again (bf16 8192^3: 524 ->
  // 512 us on constant, 671 -> 663 us on seeded operands; smaller operands, fp8 8192^3: 2 % slower; a 4-byte C: 10 %).
  const uint32_t c_streams = OP != kQuadI8 && ((uint64_t)M + N) * k_bytes >= (256ull << 20) ? 1u : 0u;
  gemm_quad_kernel<OP><<<gemm_workgroups(dev, tiles_m * tiles_n), kQuadThreads, kRingBytes, dev->stream>>>(
      (const uint8_t *)A, (const uint8_t *)B, C, N, k_bytes, scale, tiles_m, tiles_n, scales_a, scales_b, c_streams);
  MI355_LAUNCH_CHECK(dev, what);
  return MI355_OK;
}

}  // namespace

// A lane's offsets within its wave's 64 rows of a slab are 32-bit: a row may be at most 64 MiB long.
constexpr uint32_t kMaxRowBytes = 64u << 20;

int mi355_launch_gemm_quad(mi355_dev *dev, int op, const char *what, const void *A, const void *B, void *C, uint32_t M, uint32_t N,
                           uint32_t k_bytes, float scale) {
  MI355_REQUIRE(dev, k_bytes <= kMaxRowBytes, "%s: a row of K is %u bytes, the kernel takes at most %u", what, k_bytes, kMaxRowBytes);
  switch (op) {
    case kQuadE4m3: return launch_quad<kQuadE4m3>(dev, what, A, B, C, M, N, k_bytes, scale);
    case kQuadE5m2: return launch_quad<kQuadE5m2>(dev, what, A, B, C, M, N, k_bytes, scale);
    case kQuadBf16: return launch_quad<kQuadBf16>(dev, what, A, B, C, M, N, k_bytes, scale);
    case kQuadF16: return launch_quad<kQuadF16>(dev, what, A, B, C, M, N, k_bytes, scale);
    case kQuadI8: return launch_quad<kQuadI8>(dev, what, A, B, C, M, N, k_bytes, scale);
  }
  return mi355_fail(dev, MI355_ERR_ARG, "gemm: unknown operand kind %d", op);
}

// The block-scaled FP4 product; the caller (gemm_mxfp4.hip) has checked the shapes (the row length among them) and
// laid the scale bytes out per lane, both operands in blocks of 128 rows (16 bytes per lane and step).
int mi355_launch_gemm_quad_mx(mi355_dev *dev, const uint8_t *A, const uint8_t *B, const uint8_t *scales_a, const uint8_t *scales_b,
                              uint16_t *C, uint32_t M, uint32_t N, uint32_t K) {
  return launch_quad<kQuadMx>(dev, "gemm_mxfp4", A, B, C, M, N, K / 2u, 1.0f, scales_a, scales_b);
}
