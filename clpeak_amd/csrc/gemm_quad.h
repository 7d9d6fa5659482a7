// gemm_quad.hip: the four-wave GEMM kernel behind mi355_gemm_bf16 / _f16 / _i8 / _fp8_e4m3 / _fp8_e5m2.
#pragma once
#include "internal.h"

enum { kQuadE4m3 = 0, kQuadE5m2 = 1, kQuadBf16 = 2, kQuadF16 = 3, kQuadI8 = 4, kQuadMx = 5 };
enum { kLdsQuad0 = 8 };   // first bit of mi355_dev::full_lds_allowed used by the instantiations of gemm_quad_kernel
enum { kLdsSmall0 = 16 };  // the same for gemm_small_kernel (gemm_small.hip)

// Shapes have been checked by the caller (multiples of 256 x 256, K a multiple of 128 bytes, 16-byte aligned buffers).
int mi355_launch_gemm_quad(mi355_dev *dev, int op, const char *what, const void *A, const void *B, void *C, uint32_t M, uint32_t N,
                           uint32_t k_bytes, float scale);
// The block-scaled e2m1 product (scale bytes already in per-lane order, blocks of 128 rows for both operands).
int mi355_launch_gemm_quad_mx(mi355_dev *dev, const uint8_t *A, const uint8_t *B, const uint8_t *scales_a, const uint8_t *scales_b,
                              uint16_t *C, uint32_t M, uint32_t N, uint32_t K);
// gemm_small.hip: the same products (not the block-scaled one) on 128x128 tiles, one workgroup per tile.
int mi355_launch_gemm_small(mi355_dev *dev, int op, const char *what, const void *A, const void *B, void *C, uint32_t M, uint32_t N,
                            uint32_t k_bytes, float scale);
