// Shared by the GEMM kernels: 256x256 tiles of C and their order (every kernel), the direct global->LDS load (every
// kernel), and the ring of five 32 KiB LDS slots with its persistent-workgroup tile walk (the fp32 kernel of gemm.hip).
#pragma once
#include "internal.h"

constexpr int kTile = 256;        // C tile edge
constexpr int kRowBytes = 128;    // bytes of K per step, per row
constexpr int kSlabBytes = kTile * kRowBytes;   // 32 KiB per operand per step

typedef __attribute__((address_space(3))) void *lds_void_ptr;
typedef const __attribute__((address_space(1))) void *global_void_ptr;

// 16 bytes per lane from global memory straight into LDS; lane i lands at lds_dst + 16*i.
__device__ inline void load_to_lds(const uint8_t *gptr, uint32_t lds_dst) {
  __builtin_amdgcn_global_load_lds((global_void_ptr)gptr, (lds_void_ptr)(uintptr_t)lds_dst, 16, 0, 0);
}

// The same as instructions in the hand-scheduled loop: scalar base + per-lane 32-bit offset (no
// vector ALU work per load), LDS destination through M0 (one wait state after writing it).
#ifndef MI355_LOAD_LDS_BITS
#define MI355_LOAD_LDS_BITS ""   // cache-policy bits of the slab loads (none: the default policy measured best)
#endif
#define MI355_LOAD_LDS(voff, sbase, m0val)                                                         \
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" MI355_LOAD_LDS_BITS \
               :: "v"(voff), "s"(sbase), "s"(m0val) : "memory", "m0")

#define MI355_DS_READ(dst, addr, off) \
  asm volatile("ds_read_b128 %0, %1 offset:" #off : "=v"(dst) : "v"(addr))

// State of one wave's walk along K that the step function reads.
struct GemmWalk {
  uint32_t a_cur, b_cur, a_nxt, b_nxt;   // LDS byte addresses of this lane's first A / B fragment, both buffers
  uint32_t dst_a, dst_b;                 // LDS destinations of the wave's A rows / B rows to fetch
  uint64_t ga, gb;                       // uniform global addresses of those A / B rows in the next slab to fetch
  uint32_t voff;                         // this lane's byte offset from ga / gb within a group of 8 rows
  uint32_t row8;                         // bytes between rows r and r+8 (load q reads from base + q*row8)
};

// The tiles one workgroup owns: ids first, first + stride, ... (`mine` of them) out of tiles_m x tiles_n.
struct TileGrid {
  uint32_t tiles_m, tiles_n, total, first, stride, mine;
};

__device__ __forceinline__ void tile_at(const TileGrid &g, uint32_t round, uint32_t &tm, uint32_t &tn) {
  const uint32_t id = g.first + round * g.stride;
#ifndef MI355_GEMM_BAND_ORDER
  // 256 workgroups on a grid whose sides are multiples of 16 tiles: one round of the part is a square of 16x16
  // tiles, and the squares are visited in serpentine order, so that a round needs 16 tile rows of A and 16 tile
  // columns of B (128 MiB of bf16 at K = 8192, half of them the round before's) instead of all of A and a few
  // columns of B: what the part re-reads from round to round stays well inside the 256 MiB last-level cache while
  // the C tiles stream through it.  Inside a square, XCD x (workgroup id % 8) owns a block of 4 rows x 8 columns
  // of tiles, walked column-major by its 32 workgroups: 12 slab streams per XCD, as in the general order below.
  if (g.stride == 256u && g.tiles_m % 16u == 0u && g.tiles_n % 16u == 0u) {
    const uint32_t xcd = g.first % 8u, i = g.first / 8u;     // i: this workgroup among the 32 of its XCD
    const uint32_t qcols = g.tiles_n / 16u, qm = round / qcols, qr = round % qcols;
    const uint32_t qn = (qm & 1u) ? qcols - 1u - qr : qr;
    tm = qm * 16u + (xcd % 4u) * 4u + (i & 3u);
    tn = qn * 16u + (xcd / 4u) * 8u + (i >> 2);
    return;
  }
#endif
  uint32_t lin = id;
  if (g.total % 8u == 0u) lin = (id % 8u) * (g.total / 8u) + id / 8u;   // tiles of one XCD are consecutive
  // consecutive tiles walk down a group of 4 tile rows, then move one column right
  const uint32_t per_group = 4u * g.tiles_n;
  const uint32_t group = lin / per_group, in_group = lin - group * per_group;
  const uint32_t rows_here = g.tiles_m - group * 4u;
  if (rows_here >= 4u) {
    tm = group * 4u + (in_group & 3u);
    tn = in_group >> 2;
  } else {
    tm = group * 4u + in_group % rows_here;
    tn = in_group / rows_here;
  }
}

__device__ __forceinline__ TileGrid tiles_of_workgroup(uint32_t tiles_m, uint32_t tiles_n) {
  TileGrid g;
  g.tiles_m = tiles_m; g.tiles_n = tiles_n; g.total = tiles_m * tiles_n;
  g.first = blockIdx.x; g.stride = gridDim.x;
  g.mine = (g.total - g.first + g.stride - 1u) / g.stride;   // the host launches at most `total` workgroups
  return g;
}

// The LDS ring of one wave and the two fetch streams (A rows three slabs ahead of the slab being
// multiplied, B rows two ahead) through all tiles of the workgroup.  Slabs are numbered through the
// tiles: slab g has its A rows in slot 2g mod 5 and its B rows in slot (2g+1) mod 5.
template <int WAVES_M, int WAVES_N>
struct GemmRing {
  static constexpr uint32_t kWaves = WAVES_M * WAVES_N;
  static constexpr uint32_t kLoadRows = kTile / kWaves;    // rows of a slab one wave fetches: 32 or 64
  static constexpr uint32_t kLoads = kLoadRows / 8;        // 8 rows per instruction
  static constexpr uint32_t kWaveRows = kTile / WAVES_M;   // extent of a wave's part of C
  static constexpr uint32_t kWaveCols = kTile / WAVES_N;

  GemmWalk w;
  TileGrid grid;
  uint64_t a_origin, b_origin;   // A / B plus this wave's rows within a tile (uniform)
  uint32_t k_bytes, steps;
  uint32_t lane_a, lane_b;       // this lane's first A / B fragment within a slot
  uint32_t dst_wave;             // this wave's rows within a slot
  uint32_t k0;                   // slot of the current slab's A rows
  uint32_t a_round, a_left, b_round, b_left;   // tile (as a round of the workgroup) and steps left in it, per stream

  __device__ __forceinline__ static uint32_t slot_off(uint32_t k) { return (k >= 5u ? k - 5u : k) * (uint32_t)kSlabBytes; }

  __device__ __forceinline__ uint64_t a_rows(uint32_t round) const {
    uint32_t tm, tn;
    tile_at(grid, round, tm, tn);
    return a_origin + (uint64_t)tm * kTile * k_bytes;
  }
  __device__ __forceinline__ uint64_t b_rows(uint32_t round) const {
    uint32_t tm, tn;
    tile_at(grid, round, tm, tn);
    return b_origin + (uint64_t)tn * kTile * k_bytes;
  }
  __device__ __forceinline__ void place() {
    w.a_cur = lane_a + slot_off(k0);      w.b_cur = lane_b + slot_off(k0 + 1u);
    w.a_nxt = lane_a + slot_off(k0 + 2u); w.b_nxt = lane_b + slot_off(k0 + 3u);
    w.dst_b = dst_wave + slot_off(k0);        // B rows two slabs ahead take over the current A slot
    w.dst_a = dst_wave + slot_off(k0 + 1u);   // A rows three slabs ahead take over the current B slot
  }
  // Move a stream to its next slab: 128 bytes along K, or on to the first slab of the workgroup's next
  // tile (after the last tile: of its first tile again, a fetch nobody reads).
  __device__ __forceinline__ void next_a() {
    if (--a_left == 0u) {
      a_round = a_round + 1u == grid.mine ? 0u : a_round + 1u;
      w.ga = a_rows(a_round);
      a_left = steps;
    } else {
      w.ga += kRowBytes;
    }
  }
  __device__ __forceinline__ void next_b() {
    if (--b_left == 0u) {
      b_round = b_round + 1u == grid.mine ? 0u : b_round + 1u;
      w.gb = b_rows(b_round);
      b_left = steps;
    } else {
      w.gb += kRowBytes;
    }
  }
  __device__ __forceinline__ void fetch(uint64_t rows, uint32_t slot) const {
#pragma unroll
    for (uint32_t q = 0; q < kLoads; q++) MI355_LOAD_LDS(w.voff, rows + (uint64_t)q * w.row8, dst_wave + slot_off(slot) + q * 1024u);
  }
  // Fill the ring (A and B rows of slabs 0 and 1, A rows of slab 2), wait for it, and stand on slab 0.
  __device__ __forceinline__ void start(const uint8_t *A, const uint8_t *B, uint32_t k_bytes_, uint32_t lds_base,
                                        uint32_t wave, uint32_t lane, const TileGrid &g) {
    const uint32_t wm = wave / WAVES_N, wn = wave % WAVES_N;
    grid = g;
    k_bytes = k_bytes_;
    steps = k_bytes / kRowBytes;
    a_origin = (uint64_t)(uintptr_t)(A + (size_t)wave * kLoadRows * k_bytes);
    b_origin = (uint64_t)(uintptr_t)(B + (size_t)wave * kLoadRows * k_bytes);
    // global -> LDS: instruction q of a wave fills rows [(wave*kLoads+q)*8, +8) of a slab; lane i is position
    // i%8 of row i/8, which holds logical chunk (i%8) ^ (row & 7) = (i%8) ^ (i/8).
    const uint32_t lchunk = (lane % 8u) ^ (lane / 8u);
    w.voff = (lane / 8u) * k_bytes + lchunk * 16u;
    w.row8 = 8u * k_bytes;
    dst_wave = __builtin_amdgcn_readfirstlane(lds_base + wave * kLoadRows * (uint32_t)kRowBytes);
    // LDS -> fragments: row (lane%16) of the wave's sub-tile, logical chunk lane/16 (+4 for the second K
    // half, i.e. the address with bit 6 flipped), swizzled with row&7 = lane&7.
    const uint32_t swz0 = ((lane / 16u) ^ (lane & 7u)) << 4;
    lane_a = lds_base + (wm * kWaveRows + lane % 16u) * kRowBytes + swz0;
    lane_b = lds_base + (wn * kWaveCols + lane % 16u) * kRowBytes + swz0;

    a_round = b_round = 0;
    a_left = b_left = steps;
    w.ga = a_rows(0);
    w.gb = b_rows(0);
    fetch(w.ga, 0); next_a();
    fetch(w.gb, 1); next_b();
    fetch(w.ga, 2); next_a();
    fetch(w.gb, 3); next_b();
    fetch(w.ga, 4); next_a();
    asm volatile("s_waitcnt vmcnt(0)\n s_barrier" ::: "memory");
    k0 = 0;
    place();
  }
  __device__ __forceinline__ void advance() {
    k0 = k0 + 2u >= 5u ? k0 + 2u - 5u : k0 + 2u;
    place();
    next_a();
    next_b();
  }
};

// What every wave does once its last tile is stored: the fetches that ran ahead of it still write LDS.
#define MI355_DRAIN_RING() asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory")

constexpr size_t kRingBytes = 5 * (size_t)kSlabBytes;   // five 32 KiB slots: all 160 KiB of a CU

// A kernel that takes the whole LDS must be allowed to, once per device handle (the attribute belongs to
// the function on the handle's device).  `bit` names the kernel within mi355_dev::full_lds_allowed.
enum { kLdsF32 = 0 /* gemm_quad.h: kLdsQuad0 + the operand kind of gemm_quad_kernel */ };
template <typename Kernel>
inline int allow_full_lds(mi355_dev *dev, Kernel kernel, unsigned bit) {
  if (dev->full_lds_allowed & (1u << bit)) return MI355_OK;
  MI355_HIP(dev, hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)kRingBytes));
  dev->full_lds_allowed |= 1u << bit;
  return MI355_OK;
}

// One persistent workgroup per CU (a workgroup takes the whole LDS of one), never more than tiles.
inline uint32_t gemm_workgroups(const mi355_dev *dev, uint32_t tiles) {
  const uint32_t cus = dev->props.num_cus > 0 ? (uint32_t)dev->props.num_cus : 1u;
  return tiles < cus ? tiles : cus;
}

