// The 8- and 16-bit GEMM kinds on 128x128 tiles, for products whose 256x256 tiling would leave most of the part idle.
//
// gemm_quad.hip gives every workgroup a 256x256 tile of C and the whole LDS of a CU; a product of fewer than 256 such
// tiles (2048^3 has 64) then runs on a fraction of the CUs.  This kernel is the small sibling: one workgroup of four
// waves per 128x128 tile (a wave owns 64x64 = 4x4 tiles of 16x16, in 64 accumulation registers), K walked in steps of
// one 128-byte row segment, a slab of 128 rows x 128 B = 16 KiB per operand and step, global memory straight into
// LDS with the row swizzle of the other GEMM kernels (the 16-byte chunk c of row r lies at position c ^ (r & 7) of the
// row: fragment reads without bank conflicts).
//
// A step is 32 matrix instructions per wave (16 for fp8), 512 cycles of the matrix pipe, a fifth of a microsecond: far
// less than a load takes to arrive.  So the LDS of the CU is a ring of five 32 KiB slots (A and B slab of a step side
// by side), the loads of a slab go out three steps before its fragments are read, and those are read a step before
// they are multiplied, into the other of two fragment sets, in the shadow of the matrix instructions of the step
// before.  Step s: wait until this wave's loads of slab s+1 have landed (loads complete in order: all but the newest
// 16), barrier (now everybody's have, and everybody holds the fragments of slab s in registers, so the slot of slab
// s-1 is free); the matrix instructions on the fragments of slab s, with the 16 reads of slab s+1 behind those of the
// first half and the 8 loads of slab s+4 riding on every fourth; wait for the reads.  The last step reads and loads
// nothing.  Past the last
// slab the loads wrap around to the start of the rows (fetches nobody reads, so that every step but the last is the
// same code); they are waited for before the wave ends.
//
// What bounds it: the issue slots of the wave.  With one wave per SIMD every instruction of a step is issued by the
// wave whose matrix instructions it sits between, about one per four cycles: beside the 32 matrix instructions a step
// has 16 reads, 8 loads with their M0 writes and some scalar bookkeeping, and a direct-to-LDS load holds the issue
// port longer than other instructions.  Measured on constant operands, per step: 0.29-0.30 us (0.21 us is the 512
// cycles of the matrix instructions at 2.4 GHz); with the loads taken out 0.24, with the reads taken out 0.29.  The
// same on 4 and on 128 CUs and for operands of 0.5 MiB (L2) and of 128 MiB (HBM): not a matter of where the data comes
// from, and four slabs in flight instead of three change nothing.  On the whole part under random operands a step
// takes 0.40 us (the clock is lower there, and waves wait more).  (An earlier form of the loads - M0 written, a wait state and the address
// arithmetic in front of every load, all eight behind matrix instructions of the first half - took 0.34 us.)
//
// The sums run over K in order, one step after the other: results differ from the 256x256 kernel's only in rounding
// (that kernel starts its walk over K at a different place on every XCD); the int8 kind is exact either way.
#include "internal.h"
#include "mfma_common.h"
#include "gemm_ring.h"
#include "gemm_quad.h"
#include <utility>

namespace {

constexpr int kSmallTile = 128, kSmallThreads = 256;
constexpr uint32_t kSmallSlab = kSmallTile * kRowBytes;   // 16 KiB per operand and step
constexpr uint32_t kSmallSlot = 2u * kSmallSlab;          // A slab, then B slab
constexpr uint32_t kSmallSlots = 5, kSmallAhead = 4;      // ring depth; how many steps ahead of its use a slab is fetched
static_assert(kSmallSlots * kSmallSlot == kRingBytes && kSmallAhead + 1 == kSmallSlots, "the ring is the whole LDS of a CU");

constexpr bool small_is_fp8(int op) { return op == kQuadE4m3 || op == kQuadE5m2; }

#define S_DS_READ(dst, addr, off) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(off))
#define S_TIE4(x) "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3])

// The fragments of one step: rows [16i, 16i+16) of the wave's 64 rows of A (a_*[i]) and of B (b_*[i]), K halves lo / hi.
struct SmallFrags {
  i32x4v a_lo[4], a_hi[4], b_lo[4], b_hi[4];
};

// What a step needs to know beside its fragments.
struct SmallWalk {
  uint32_t a0, a1, b0, b1;   // LDS addresses of this lane's first A / B fragment in the slab to read, K halves lo / hi
  uint32_t dst;              // LDS destination of the wave's first rows in the slot to fill
  uint32_t voff[4];          // this lane's byte offset from ga / gb in each of the wave's four groups of 8 rows
  uint64_t ga, gb;           // the wave's A / B rows in the slab to fetch
};

// The accumulators are the accumulation registers a[0:63], named in the instruction text: tile (i, j) of the wave's
// 4x4 tiles is a[4T : 4T+3], T = 4i + j.  The compiler is told once that they are taken and never sees them as values:
// what it holds as a value it may copy where paths of the program join, and it does not know that a register written
// by a matrix instruction of this file's text must not be read for some cycles.
__device__ __forceinline__ void small_claim_accumulators() {
#define S_A10(n) "a" #n "0", "a" #n "1", "a" #n "2", "a" #n "3", "a" #n "4", "a" #n "5", "a" #n "6", "a" #n "7", "a" #n "8", "a" #n "9"
  asm volatile("" ::: "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", S_A10(1), S_A10(2), S_A10(3), S_A10(4), S_A10(5), "a60", "a61",
               "a62", "a63");
#undef S_A10
}
template <int R>
__device__ __forceinline__ void small_zero_register() { asm volatile("v_accvgpr_write_b32 a[%0], 0" :: "n"(R)); }
template <int... Rs>
__device__ __forceinline__ void small_zero_accumulators(std::integer_sequence<int, Rs...>) {
  (small_zero_register<Rs>(), ...);
  asm volatile("s_nop 7");   // written by the vector unit, read next by the matrix unit
}
// Tile T out of the accumulation registers, as raw bits.
template <int T>
__device__ __forceinline__ i32x4v small_take_tile() {
  int v0, v1, v2, v3;
  asm volatile("v_accvgpr_read_b32 %0, a[%4]\n v_accvgpr_read_b32 %1, a[%5]\n v_accvgpr_read_b32 %2, a[%6]\n v_accvgpr_read_b32 %3, a[%7]"
               : "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3) : "n"(4 * T), "n"(4 * T + 1), "n"(4 * T + 2), "n"(4 * T + 3));
  return (i32x4v){v0, v1, v2, v3};
}

// Matrix instruction number S of a step.  The 16-bit and int8 kinds take 32, an instruction per K half: row i of the
// wave's 4x4 tiles is instructions 8i .. 8i+7, its four first halves and then its four second halves, so that an
// instruction never waits for the one just before it.  fp8 takes 16, one K = 128 instruction on both halves (the A
// fragment is the second source of the transposed product: format field blgp for an e5m2 A).
// Q >= 0: load number Q of the slab to fetch rides along (8 rows of A for Q < 4, of B otherwise, into the slot being
// filled): M0, which holds the LDS destination, is written in front of the matrix instruction, which is the wait state
// M0 needs before a load reads it, and the load is issued behind it; three instructions in all.
template <int OP, int S, int Q = -1>
__device__ __forceinline__ void small_mfma(const SmallFrags &f, const SmallWalk &w) {
#define S_MFMA(insn, fmt, T, b, a)                                                                                              \
  if constexpr (Q < 0) asm volatile(insn " a[%2:%3], %0, %1, a[%2:%3]" fmt :: "v"(b), "v"(a), "n"(4 * (T)), "n"(4 * (T) + 3));    \
  else asm volatile("s_add_u32 m0, %4, %5\n " insn " a[%2:%3], %0, %1, a[%2:%3]" fmt "\n global_load_lds_dwordx4 %6, %7"         \
                    :: "v"(b), "v"(a), "n"(4 * (T)), "n"(4 * (T) + 3), "s"(w.dst), "n"(Q < 4 ? Q * 1024 : (int)kSmallSlab + (Q - 4) * 1024), \
                       "v"(w.voff[Q < 0 ? 0 : Q % 4]), "s"(Q < 4 ? w.ga : w.gb) : "memory", "m0", "scc")
  if constexpr (small_is_fp8(OP)) {
    constexpr int i = S / 4, j = S % 4;
    const i32x8v a8 = __builtin_shufflevector(f.a_lo[i], f.a_hi[i], 0, 1, 2, 3, 4, 5, 6, 7);
    const i32x8v b8 = __builtin_shufflevector(f.b_lo[j], f.b_hi[j], 0, 1, 2, 3, 4, 5, 6, 7);
    if constexpr (OP == kQuadE5m2) { S_MFMA("v_mfma_f32_16x16x128_f8f6f4", " blgp:1", 4 * i + j, b8, a8); }
    else { S_MFMA("v_mfma_f32_16x16x128_f8f6f4", "", 4 * i + j, b8, a8); }
  } else {
    constexpr int i = S / 8, hi = (S % 8) / 4, j = S % 4;
    const i32x4v &a = hi ? f.a_hi[i] : f.a_lo[i], &b = hi ? f.b_hi[j] : f.b_lo[j];
    if constexpr (OP == kQuadBf16) { S_MFMA("v_mfma_f32_16x16x32_bf16", "", 4 * i + j, b, a); }
    else if constexpr (OP == kQuadF16) { S_MFMA("v_mfma_f32_16x16x32_f16", "", 4 * i + j, b, a); }
    else { S_MFMA("v_mfma_i32_16x16x64_i8", "", 4 * i + j, b, a); }
  }
#undef S_MFMA
}

// Fragment read number R of 16: the B fragments (rows 16j.. of the wave's part of the B slab), then the A fragments.
template <int R>
__device__ __forceinline__ void small_read(SmallFrags &f, const SmallWalk &w) {
  constexpr int i = (R % 8) / 2, off = i * 16 * kRowBytes;
  if constexpr (R < 8) {
    if constexpr (R % 2 == 0) S_DS_READ(f.b_lo[i], w.b0, off); else S_DS_READ(f.b_hi[i], w.b1, off);
  } else {
    if constexpr (R % 2 == 0) S_DS_READ(f.a_lo[i], w.a0, off); else S_DS_READ(f.a_hi[i], w.a1, off);
  }
}

// Load number Q of 8 of a slab on its own (filling the ring before the first step).
template <int Q>
__device__ __forceinline__ void small_load(const SmallWalk &w) {
  if constexpr (Q < 4) MI355_LOAD_LDS(w.voff[Q], w.ga, w.dst + Q * 1024u);
  else MI355_LOAD_LDS(w.voff[Q - 4], w.gb, w.dst + kSmallSlab + (Q - 4) * 1024u);
}

// The reads of a fragment set have arrived.  The registers ride along so that nothing that uses them can be placed
// before the wait (an asm statement takes 30 operands at most: two statements).  Between issuing reads and this wait
// there must be no branch: where paths join, the compiler may copy registers, and it does not know that these are
// still being written.
__device__ __forceinline__ void small_arrived(SmallFrags &f) {
  asm volatile("s_waitcnt lgkmcnt(0)" : S_TIE4(f.a_lo), S_TIE4(f.a_hi)
               : "v"(f.b_lo[0]), "v"(f.b_lo[1]), "v"(f.b_lo[2]), "v"(f.b_lo[3]), "v"(f.b_hi[0]), "v"(f.b_hi[1]), "v"(f.b_hi[2]), "v"(f.b_hi[3]));
  asm volatile("" : S_TIE4(f.b_lo), S_TIE4(f.b_hi));
}

// One step: the matrix instructions on `cur`, and in their shadow the 16 reads of the next step's fragments into
// `nxt` and the 8 loads of the slab four steps on.  A lone wave issues an instruction every four cycles or so, whatever
// it is, so a 16-cycle matrix instruction has room for three others beside it: the loads ride one on every fourth
// matrix instruction (every second for fp8) over the whole step, the reads one behind each of the first 16 (fp8: two
// behind each of the first 8), so that they have arrived when the second half is through.
// LAST: the step behind which nothing follows reads and loads nothing.
template <int OP, bool LAST, int S>
__device__ __forceinline__ void small_slot(const SmallFrags &cur, SmallFrags &nxt, const SmallWalk &w) {
  constexpr int kEvery = small_is_fp8(OP) ? 2 : 4;
  if constexpr (LAST || S % kEvery != 0) small_mfma<OP, S>(cur, w);
  else small_mfma<OP, S, S / kEvery>(cur, w);
  if constexpr (LAST) return;
  if constexpr (small_is_fp8(OP)) {
    if constexpr (S < 8) { small_read<2 * S>(nxt, w); small_read<2 * S + 1>(nxt, w); }
  } else {
    if constexpr (S < 16) small_read<S>(nxt, w);
  }
}

template <int OP, bool LAST, int... S>
__device__ __forceinline__ void small_step(std::integer_sequence<int, S...>, SmallFrags &cur, SmallFrags &nxt, const SmallWalk &w) {
  // This wave's loads of the slab to read have landed (loads complete in order, 8 per slab; the two slabs behind it
  // may be in flight); after the barrier everybody's have, and every wave has `cur` in registers, so that the slot
  // `cur` came from can be filled by the loads of the next step.
  if constexpr (!LAST) asm volatile("s_waitcnt vmcnt(16)\n s_barrier" ::: "memory");
  (small_slot<OP, LAST, S>(cur, nxt, w), ...);
  if constexpr (!LAST) small_arrived(nxt);
}

// Tile T = 4i + j of the wave to C: a lane holds 4 consecutive N elements of a row (the product is issued transposed).
template <int OP, int T>
__device__ __forceinline__ void small_store_tile(void *__restrict__ C, uint32_t N, uint32_t row0, uint32_t col0, float scale) {
  const i32x4v t = small_take_tile<T>();
  const size_t at = (size_t)(row0 + (T / 4) * 16u) * N + col0 + (T % 4) * 16u;
  if constexpr (OP == kQuadI8) {
    *reinterpret_cast<i32x4v *>(static_cast<int32_t *>(C) + at) = t;
  } else {
    float x[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int bits = t[r];   // (through a scalar copy: __builtin_bit_cast applied to an element of a vector reads element 0)
      x[r] = __builtin_bit_cast(float, bits);
      if constexpr (small_is_fp8(OP)) x[r] *= scale;
    }
    uint2 packed;
    packed.x = OP == kQuadF16 ? mi355_pack_f16x2(x[0], x[1]) : mi355_pack_bf16x2(x[0], x[1]);
    packed.y = OP == kQuadF16 ? mi355_pack_f16x2(x[2], x[3]) : mi355_pack_bf16x2(x[2], x[3]);
    *reinterpret_cast<uint2 *>(static_cast<uint16_t *>(C) + at) = packed;
  }
}
template <int OP, int... Ts>
__device__ __forceinline__ void small_store(std::integer_sequence<int, Ts...>, void *__restrict__ C, uint32_t N, uint32_t row0, uint32_t col0, float scale) {
  (small_store_tile<OP, Ts>(C, N, row0, col0, scale), ...);
}

template <int OP>
__global__ void __launch_bounds__(kSmallThreads)
gemm_small_kernel(const uint8_t *__restrict__ A, const uint8_t *__restrict__ B, void *__restrict__ C, uint32_t N, uint32_t k_bytes,
                  float scale, uint32_t tiles_m, uint32_t tiles_n) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const uint32_t tid = threadIdx.x, lane = tid % 64;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const uint32_t wm = wave / 2, wn = wave % 2;
  TileGrid grid;
  grid.tiles_m = tiles_m; grid.tiles_n = tiles_n; grid.total = tiles_m * tiles_n;
  grid.first = blockIdx.x; grid.stride = gridDim.x; grid.mine = 1;
  uint32_t tm, tn;
  tile_at(grid, 0, tm, tn);
  const uint32_t steps = k_bytes / kRowBytes;
  constexpr uint32_t kRing = kSmallSlots * kSmallSlot;
  auto after = [](uint32_t slot_off) { return slot_off + kSmallSlot == kRing ? 0u : slot_off + kSmallSlot; };

  // global -> LDS: wave w fills rows [32w, 32w+32) of the A slab and of the B slab, 8 rows per instruction; lane i is
  // position i%8 of row i/8, which holds logical chunk (i%8) ^ (i/8)
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
  const uint32_t dst_wave = __builtin_amdgcn_readfirstlane(lds_base + wave * 32u * (uint32_t)kRowBytes);
  SmallWalk w;
#pragma unroll
  for (uint32_t q = 0; q < 4; q++) w.voff[q] = (lane / 8u + 8u * q) * k_bytes + ((lane % 8u) ^ (lane / 8u)) * 16u;
  w.ga = (uint64_t)(uintptr_t)(A + ((size_t)tm * kSmallTile + wave * 32u) * k_bytes);
  w.gb = (uint64_t)(uintptr_t)(B + ((size_t)tn * kSmallTile + wave * 32u) * k_bytes);
  uint32_t fetch_left = steps, fill = 0, look = 0;   // slot offsets: the one to fill, the one to read
  auto fetched = [&]() {                             // on to the next slab; past the last one: the first again
    w.ga += kRowBytes;
    w.gb += kRowBytes;
    if (--fetch_left == 0u) { w.ga -= k_bytes; w.gb -= k_bytes; fetch_left = steps; }
    fill = after(fill);
  };
  // LDS -> fragments: row lane%16 of the wave's part, chunk lane/16 (+4 for the second K half: bit 6 of the address),
  // swizzled with row & 7 = lane & 7
  const uint32_t swz0 = ((lane / 16u) ^ (lane & 7u)) << 4;
  const uint32_t lane_a = lds_base + (wm * 64u + lane % 16u) * kRowBytes + swz0;
  const uint32_t lane_b = lds_base + kSmallSlab + (wn * 64u + lane % 16u) * kRowBytes + swz0;
  auto place = [&]() {
    w.a0 = lane_a + look; w.a1 = w.a0 ^ 64u;
    w.b0 = lane_b + look; w.b1 = w.b0 ^ 64u;
    w.dst = dst_wave + fill;
  };

  small_claim_accumulators();
  small_zero_accumulators(std::make_integer_sequence<int, 64>{});

  // slabs 0..3 into slots 0..3; the fragments of slab 0
  for (uint32_t d = 0; d < kSmallAhead; d++) {
    place();
    small_load<0>(w); small_load<1>(w); small_load<2>(w); small_load<3>(w);
    small_load<4>(w); small_load<5>(w); small_load<6>(w); small_load<7>(w);
    fetched();
  }
  asm volatile("s_waitcnt vmcnt(%0)\n s_barrier" :: "n"(8 * (kSmallAhead - 1)) : "memory");
  SmallFrags f0, f1;
  place();
  small_read<0>(f0, w); small_read<1>(f0, w); small_read<2>(f0, w); small_read<3>(f0, w);
  small_read<4>(f0, w); small_read<5>(f0, w); small_read<6>(f0, w); small_read<7>(f0, w);
  small_read<8>(f0, w); small_read<9>(f0, w); small_read<10>(f0, w); small_read<11>(f0, w);
  small_read<12>(f0, w); small_read<13>(f0, w); small_read<14>(f0, w); small_read<15>(f0, w);
  small_arrived(f0);

  // Step s multiplies the fragments of slab s, reads those of slab s+1 and fills the slot of slab s-1, which every
  // wave had in registers before it came to the barrier of step s-1, with slab s+4 (past the last slab: with the
  // first ones again, fetches nobody reads).  Two steps per turn, so that the two fragment sets swap by name.
  constexpr auto kSlots = std::make_integer_sequence<int, small_is_fp8(OP) ? 16 : 32>{};
  uint32_t s = 0;
  for (; s + 2 < steps; s += 2) {
    look = after(look); place();
    small_step<OP, false>(kSlots, f0, f1, w);
    fetched();
    look = after(look); place();
    small_step<OP, false>(kSlots, f1, f0, w);
    fetched();
  }
  if (s + 2 == steps) {
    look = after(look); place();
    small_step<OP, false>(kSlots, f0, f1, w);
    small_step<OP, true>(kSlots, f1, f0, w);
  } else {
    small_step<OP, true>(kSlots, f0, f1, w);
  }
  // the wait states between the last matrix instruction and the first read of its result; the fetches that ran
  // ahead of the last step still write LDS
  asm volatile("s_nop 15\n s_nop 15\n s_waitcnt vmcnt(0)" ::: "memory");
  small_store<OP>(std::make_integer_sequence<int, 16>{}, C, N, tm * kSmallTile + wm * 64u + lane % 16u, tn * kSmallTile + wn * 64u + 4u * (lane / 16u), scale);
}

template <int OP>
int launch_small(mi355_dev *dev, const char *what, const void *A, const void *B, void *C, uint32_t M, uint32_t N, uint32_t k_bytes, float scale) {
  if (int rc = allow_full_lds(dev, &gemm_small_kernel<OP>, kLdsSmall0 + OP)) return rc;
  const uint32_t tiles_m = M / kSmallTile, tiles_n = N / kSmallTile;
  gemm_small_kernel<OP><<<tiles_m * tiles_n, kSmallThreads, kRingBytes, dev->stream>>>((const uint8_t *)A, (const uint8_t *)B, C, N, k_bytes, scale,
                                                                                         tiles_m, tiles_n);
  MI355_LAUNCH_CHECK(dev, what);
  return MI355_OK;
}

}  // namespace

// Shapes have been checked by the caller (M and N multiples of 128; K a multiple of 128 bytes; 16-byte aligned buffers;
// a row of K at most 64 MiB).
int mi355_launch_gemm_small(mi355_dev *dev, int op, const char *what, const void *A, const void *B, void *C, uint32_t M, uint32_t N,
                            uint32_t k_bytes, float scale) {
  switch (op) {
    case kQuadE4m3: return launch_small<kQuadE4m3>(dev, what, A, B, C, M, N, k_bytes, scale);
    case kQuadE5m2: return launch_small<kQuadE5m2>(dev, what, A, B, C, M, N, k_bytes, scale);
    case kQuadBf16: return launch_small<kQuadBf16>(dev, what, A, B, C, M, N, k_bytes, scale);
    case kQuadF16: return launch_small<kQuadF16>(dev, what, A, B, C, M, N, k_bytes, scale);
    case kQuadI8: return launch_small<kQuadI8>(dev, what, A, B, C, M, N, k_bytes, scale);
  }
  return mi355_fail(dev, MI355_ERR_ARG, "gemm: unknown operand kind %d", op);
}
