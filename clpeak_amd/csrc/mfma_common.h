// Operand layouts of the gfx950 matrix instructions, as used by every MFMA/SMFMAC
// kernel of this backend.  Lanes are numbered 0..63 within a wavefront.
//
// 16x16xK shapes (K = 32 f16/bf16, 64 i8, 128 f8f6f4):
//   A operand: lane l holds row (l % 16), K elements [ (l/16)*K/4 , (l/16+1)*K/4 ), low
//              element in the low bits of the first register.
//   B operand: lane l holds column (l % 16), same K range.
//   C/D:       register r of lane l is element (row 4*(l/16) + r, column l % 16).
// 32x32x16 f16/bf16:
//   A operand: lane l holds row (l % 32), K elements [ (l/32)*8, (l/32)*8 + 8 ).
//   B operand: lane l holds column (l % 32), same K range.
//   C/D:       register r (0..15) of lane l is element
//              (row 8*(r/4) + 4*(l/32) + r%4, column l % 32).
// 16x16x4 f32 / f64 (one element per lane and operand): lane l holds row (l % 16), k = l / 16.  C/D of
//   the f32 shape as above; of the f64 shape register r (a pair) of lane l is element
//   (row 4*r + l/16, column l % 16): rows interleave over the lane groups.
// f8f6f4, 16x16x128.  6-bit and 4-bit codes follow the rule above (lane l holds the 32
//   consecutive K elements of block l/16).  8-bit codes do not: the 32 bytes of lane l
//   are K elements [ 16*(l/16), +16 ) followed by [ 64 + 16*(l/16), +16 ), i.e. two
//   K=64 operands back to back.  In every case the E8M0 scale of 32-element block b of
//   row/column r is taken from lane (r + 16*b), from the byte of the scale register
//   that op_sel names.
// SMFMAC 16x16xK (K = 64 for 16-bit, 128 for 8-bit data):
//   A holds the K/2 kept values of row (l % 16): lane l has kept values
//     [ (l/16)*K/8, (l/16+1)*K/8 ), i.e. the kept values of dense K range
//     [ (l/16)*K/4, (l/16+1)*K/4 ).
//   B is laid out as two dense half-K operands back to back: the first half of lane
//     l's registers holds K elements [ (l/16)*K/8, (l/16+1)*K/8 ) of column (l % 16), the
//     second half holds [ K/2 + (l/16)*K/8, K/2 + (l/16+1)*K/8 ).  In bytes both kinds
//     read 16 bytes at row offset 16*(l/16) and 16 bytes at 64 + 16*(l/16).
//   The index register carries two 2-bit positions per group of four, the first kept
//     value in the lower bits, groups in K order from bit 0 (16 index bits for 16-bit
//     data, ABID picks the half of the register; 32 bits for 8-bit data).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef _Float16 half8v  __attribute__((ext_vector_type(8)));
typedef _Float16 half16v __attribute__((ext_vector_type(16)));
typedef __bf16   bf16x8v  __attribute__((ext_vector_type(8)));
typedef __bf16   bf16x16v __attribute__((ext_vector_type(16)));
typedef float    f32x4v  __attribute__((ext_vector_type(4)));
typedef float    f32x16v __attribute__((ext_vector_type(16)));
typedef int      i32x2v  __attribute__((ext_vector_type(2)));
typedef int      i32x4v  __attribute__((ext_vector_type(4)));
typedef int      i32x8v  __attribute__((ext_vector_type(8)));
typedef int      i32x16v __attribute__((ext_vector_type(16)));

// f8f6f4 format selectors (cbsz for A, blgp for B).
#define MI355_F8F6F4_E4M3 0
#define MI355_F8F6F4_E5M2 1
#define MI355_F8F6F4_E2M3 2
#define MI355_F8F6F4_E3M2 3
#define MI355_F8F6F4_E2M1 4

// Unaligned-safe vector loads from byte addresses (operands are only element aligned).
template <typename V>
__device__ inline V load_bytes(const uint8_t *p) {
  V v;
  __builtin_memcpy(&v, p, sizeof(V));
  return v;
}

// Two fp32 values rounded to nearest even and packed, `lo` in bits 0..15: one instruction each on
// gfx950 (v_cvt_pk_bf16_f32, v_cvt_pk_f16_f32).  Same results as the bit-level routines of
// numeric_formats.h for every finite input (bf16: every fp32 value; f16: gradual underflow, overflow
// to infinity), which cost ten instructions and a branch per value.
typedef float f32x2v __attribute__((ext_vector_type(2)));
__device__ inline uint32_t mi355_pack_bf16x2(float lo, float hi) {
  typedef __bf16 bf16x2v __attribute__((ext_vector_type(2)));
  const bf16x2v r = __builtin_convertvector((f32x2v){lo, hi}, bf16x2v);
  uint32_t u;
  __builtin_memcpy(&u, &r, sizeof(u));
  return u;
}
__device__ inline uint32_t mi355_pack_f16x2(float lo, float hi) {
  typedef _Float16 half2v __attribute__((ext_vector_type(2)));
  const half2v r = __builtin_convertvector((f32x2v){lo, hi}, half2v);
  uint32_t u;
  __builtin_memcpy(&u, &r, sizeof(u));
  return u;
}
