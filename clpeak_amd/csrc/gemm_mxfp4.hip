// Block-scaled FP4 GEMM (OCP MXFP4):  C[M][N] (bf16) = sum_k (A[m][k] * 2^(SA[m][k/32]-127)) * (B[n][k] * 2^(SB[n][k/32]-127)).
// A and B hold e2m1 codes, two per byte, K contiguous; SA / SB hold one E8M0 byte per 32 elements.
//
// The product runs on the four-wave kernel of gemm_quad.hip (operand kind kQuadMx): the same tile walk, LDS slots,
// swizzle and direct-to-LDS loads as the other kinds, K in steps of 128 bytes per row (256 codes, 8 scale blocks).  A
// K=128 instruction takes 16 bytes per lane, one 16-byte chunk of a row, which is exactly one scale block; the
// two instructions of a slot take chunks g and g+4 (g = lane / 16) like the two bf16 instructions of a slot.
//
// Scales do not pass through LDS (it is full).  Lane r+16g of a fragment must hold the scale byte of row r,
// block g.  The pre-pass below rewrites scale_a / scale_b into that shape once per call: for every block of
// 128 rows (what one wave multiplies, of either operand) and every K step, 64 lanes x 16 bytes, byte
// 2i+h of lane (r,g) being the scale of row 16i+r, block 8s+4h+g (fragment i, K half h).  The main loop then
// fetches the scales of a step with ONE load per operand, fully coalesced, a whole step ahead, and the matrix
// instruction picks byte 2(i%2)+h of register i/2 with its op_sel fields.  (Fetching the bytes from the
// row-major arrays inside the loop, one gather per fragment and half, more than doubled the run time.)
// Two waves of a workgroup share each block of rows, so every scale byte is loaded twice per workgroup: 8 KiB per
// step on top of the 64 KiB of the slab.
#include "internal.h"
#include "gemm_ring.h"
#include "gemm_quad.h"

namespace {

// Pre-pass: scales from row-major [rows][k32] to the per-lane order the main loop loads, both operands in one
// launch.  One workgroup per (block of rows, 16 K steps): blocks of 128 rows (8 fragments of 16 rows, 16
// bytes per lane and step) for both operands.  16 steps are 128 scale bytes of a
// row, one cache line: the rows are read once, 8 bytes per thread and fully coalesced, into LDS (row stride 136
// bytes, so that the 16 rows of a fragment fall into 16 different banks), and each wave then builds the words
// of every fourth step from byte reads of LDS.  (Gathering the bytes straight from global memory, two per row
// and lane, took 9.5 us per call at 8192^3, 4 % of the product.)
constexpr uint32_t kLayoutSteps = 16, kLayoutStride = 136, kLayoutFrags = 8;

__global__ void __launch_bounds__(256)
mx_scale_layout_kernel(const uint8_t *__restrict__ SA, const uint8_t *__restrict__ SB, uint8_t *__restrict__ out_a,
                       uint8_t *__restrict__ out_b, uint32_t k32, uint32_t steps, uint32_t groups_a, uint32_t groups_b) {
  __shared__ __attribute__((aligned(16))) uint8_t rows[128 * kLayoutStride];
  const uint32_t chunks = (steps + kLayoutSteps - 1) / kLayoutSteps;   // groups of 16 steps per block of rows
  uint32_t grp = blockIdx.x;
  if (grp >= groups_a + groups_b) return;
  const uint8_t *S = SA;
  uint8_t *out = out_a;
  constexpr uint32_t frags = kLayoutFrags;
  if (grp >= groups_a) { grp -= groups_a; S = SB; out = out_b; }
  const uint32_t rb = grp / chunks, s0 = (grp % chunks) * kLayoutSteps;
  const uint32_t ns = steps - s0 < kLayoutSteps ? steps - s0 : kLayoutSteps, nrows = 16u * frags;
  for (uint32_t u = threadIdx.x; u < nrows * ns; u += blockDim.x) {
    const uint32_t row = u / ns, st = u % ns;
    *reinterpret_cast<uint2 *>(rows + row * kLayoutStride + st * 8u) =
        *reinterpret_cast<const uint2 *>(S + (size_t)(rb * nrows + row) * k32 + (size_t)(s0 + st) * 8u);
  }
  __syncthreads();
  const uint32_t wave = threadIdx.x / 64u, lane = threadIdx.x % 64u, r = lane % 16u, g = lane / 16u;
  for (uint32_t st = wave; st < ns; st += blockDim.x / 64u) {
    uint32_t word[4] = {0, 0, 0, 0};
#pragma unroll
    for (uint32_t i = 0; i < frags; i++) {
      const uint8_t *p = rows + (16u * i + r) * kLayoutStride + st * 8u + g;
      const uint32_t pair = (uint32_t)p[0] | ((uint32_t)p[4] << 8);   // K halves 0 and 1 of fragment i
      if (i % 2 == 0) word[i / 2] = pair;
      else word[i / 2] |= pair << 16;
    }
    const size_t unit = (size_t)rb * steps + s0 + st;
    *reinterpret_cast<uint4 *>(out + (unit * 64u + lane) * 16u) = make_uint4(word[0], word[1], word[2], word[3]);
  }
}

// A lane's offsets within its wave's 64 rows of a slab are 32-bit: a row of K (K/2 bytes) may be at most 64 MiB long.
constexpr uint32_t kMaxRowBytes = 64u << 20;

// Shape and alignment checks shared by the entry points; nothing is allocated or launched before they pass.
int check_mx_shapes(mi355_dev *dev, const void *A, const void *B, const void *C, uint32_t M, uint32_t N, uint32_t K) {
  MI355_REQUIRE(dev, A && B && C, "gemm_mxfp4: null buffer");
  MI355_REQUIRE(dev, M > 0 && N > 0 && K > 0, "gemm_mxfp4: empty problem");
  MI355_REQUIRE(dev, M % kTile == 0 && N % kTile == 0, "gemm_mxfp4: M (%u) and N (%u) must be multiples of 256", M, N);
  MI355_REQUIRE(dev, K % 256 == 0, "gemm_mxfp4: K (%u) must be a multiple of 256", K);
  MI355_REQUIRE(dev, K / 2u <= kMaxRowBytes, "gemm_mxfp4: a row of K is %u bytes, the kernel takes at most %u", K / 2u, kMaxRowBytes);
  MI355_REQUIRE(dev, (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15u) == 0, "gemm_mxfp4: buffers must be 16-byte aligned");
  return MI355_OK;
}
int check_mx_scales(mi355_dev *dev, const void *scale_a, const void *scale_b) {
  MI355_REQUIRE(dev, scale_a && scale_b, "gemm_mxfp4: null buffer");
  MI355_REQUIRE(dev, (((uintptr_t)scale_a | (uintptr_t)scale_b) & 7u) == 0, "gemm_mxfp4: scale arrays must be 8-byte aligned");
  return MI355_OK;
}

// The pre-pass: scale_a / scale_b into `lane_scales` (M*K/32 bytes for A, then N*K/32 for B), on the handle's stream.
int lay_out_scales(mi355_dev *dev, const uint8_t *scale_a, const uint8_t *scale_b, uint32_t M, uint32_t N, uint32_t K, uint8_t *lane_scales) {
  const uint32_t k32 = K / 32u, steps = K / 256u;
  uint8_t *sal = lane_scales, *sbl = sal + (size_t)M * k32;
  const uint32_t chunks = (steps + kLayoutSteps - 1) / kLayoutSteps;
  const uint32_t groups_a = M / 128u * chunks, groups_b = N / 128u * chunks;
  mx_scale_layout_kernel<<<groups_a + groups_b, 256, 0, dev->stream>>>(scale_a, scale_b, sal, sbl, k32, steps, groups_a, groups_b);
  MI355_LAUNCH_CHECK(dev, "mx_scale_layout");
  return MI355_OK;
}

// The product on scales already in per-lane order.
int multiply_mx(mi355_dev *dev, const uint8_t *A, const uint8_t *B, const uint8_t *lane_scales, uint16_t *C, uint32_t M, uint32_t N, uint32_t K) {
  return mi355_launch_gemm_quad_mx(dev, A, B, lane_scales, lane_scales + (size_t)M * (K / 32u), C, M, N, K);
}

}  // namespace

// Scratch of the entry point that allocates nothing: the lane-ordered scales of one call.  4 MiB hold the
// scales of the 8192^3 product (2 x 8192 x 8192 / 32 bytes).  Every GPU the library runs on holds its own copy
// of this array, at its own address, until the process ends.
constexpr size_t kStaticScaleBytes = 4u << 20;
static __device__ __align__(256) uint8_t scratch[kStaticScaleBytes];

// Called by mi355_open with the handle's device current: the device address of `scratch` on that device.  (In
// host code the array's name is only a stand-in for the symbol; kernels and copies must be given this address.)
int mi355_mx_resolve_static_scratch(mi355_dev *dev) {
  void *ptr = nullptr;
  MI355_HIP(dev, hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
  if (!ptr) return mi355_fail(dev, MI355_ERR_HIP, "gemm_mxfp4: the static scratch array has no device address");
  dev->mx_static_scratch = ptr;
  return MI355_OK;
}

extern "C" int mi355_gemm_mxfp4(mi355_dev *dev, const uint8_t *A, const uint8_t *B, const uint8_t *scale_a,
                                const uint8_t *scale_b, uint16_t *C, uint32_t M, uint32_t N, uint32_t K) {
  MI355_ENTER(dev);
  if (int rc = check_mx_shapes(dev, A, B, C, M, N, K)) return rc;
  if (int rc = check_mx_scales(dev, scale_a, scale_b)) return rc;
  // lane-ordered copies of the scales live in a scratch buffer the handle keeps (same size as the scales)
  const size_t need = ((size_t)M + N) * (K / 32u);
  if (dev->mx_scratch_bytes < need) {
    MI355_HIP(dev, hipStreamSynchronize(dev->stream));
    if (dev->mx_scratch) MI355_HIP(dev, hipFree(dev->mx_scratch));
    dev->mx_scratch = nullptr;
    dev->mx_scratch_bytes = 0;
    const hipError_t e = hipMalloc(&dev->mx_scratch, need);
    if (e != hipSuccess) return mi355_fail(dev, e == hipErrorOutOfMemory ? MI355_ERR_OOM : MI355_ERR_HIP,
                                           "gemm_mxfp4: scratch of %zu bytes: %s", need, hipGetErrorString(e));
    dev->mx_scratch_bytes = need;
  }
  uint8_t *lane_scales = static_cast<uint8_t *>(dev->mx_scratch);
  if (int rc = lay_out_scales(dev, scale_a, scale_b, M, N, K, lane_scales)) return rc;
  return multiply_mx(dev, A, B, lane_scales, C, M, N, K);
}

extern "C" int mi355_gemm_mxfp4_prepare_scales(mi355_dev *dev, const uint8_t *scale_a, const uint8_t *scale_b, uint32_t M, uint32_t N,
                                               uint32_t K, uint8_t *prepared) {
  MI355_ENTER(dev);
  MI355_REQUIRE(dev, prepared != nullptr && ((uintptr_t)prepared & 15u) == 0, "gemm_mxfp4_prepare_scales: the prepared buffer must be 16-byte aligned");
  MI355_REQUIRE(dev, M > 0 && N > 0 && K > 0 && M % kTile == 0 && N % kTile == 0 && K % 256 == 0,
                "gemm_mxfp4_prepare_scales: M (%u) and N (%u) must be multiples of 256 and K (%u) a multiple of 256", M, N, K);
  if (int rc = check_mx_scales(dev, scale_a, scale_b)) return rc;
  return lay_out_scales(dev, scale_a, scale_b, M, N, K, prepared);
}

extern "C" int mi355_gemm_mxfp4_prepared(mi355_dev *dev, const uint8_t *A, const uint8_t *B, const uint8_t *prepared, uint16_t *C,
                                         uint32_t M, uint32_t N, uint32_t K) {
  MI355_ENTER(dev);
  if (int rc = check_mx_shapes(dev, A, B, C, M, N, K)) return rc;
  MI355_REQUIRE(dev, prepared != nullptr && ((uintptr_t)prepared & 15u) == 0, "gemm_mxfp4_prepared: the prepared scales must be 16-byte aligned");
  return multiply_mx(dev, A, B, prepared, C, M, N, K);
}

extern "C" int mi355_gemm_mxfp4_static(mi355_dev *dev, const uint8_t *A, const uint8_t *B, const uint8_t *scale_a,
                                       const uint8_t *scale_b, uint16_t *C, uint32_t M, uint32_t N, uint32_t K) {
  MI355_ENTER(dev);
  if (int rc = check_mx_shapes(dev, A, B, C, M, N, K)) return rc;
  if (int rc = check_mx_scales(dev, scale_a, scale_b)) return rc;
  const size_t need = ((size_t)M + N) * (K / 32u);
  MI355_REQUIRE(dev, need <= kStaticScaleBytes,
                "gemm_mxfp4_static: (M + N) * K / 32 = %zu scale bytes exceed the static scratch of %zu bytes "
                "(use mi355_gemm_mxfp4 for larger problems)", need, kStaticScaleBytes);
  MI355_REQUIRE(dev, dev->mx_static_scratch != nullptr, "gemm_mxfp4_static: the static scratch was not resolved when the device was opened");
  // The pre-pass overwrites every byte the product reads, so nothing of the previous call's contents has to be cleared.
  uint8_t *lane_scales = static_cast<uint8_t *>(dev->mx_static_scratch);
  if (int rc = lay_out_scales(dev, scale_a, scale_b, M, N, K, lane_scales)) return rc;
  return multiply_mx(dev, A, B, lane_scales, C, M, N, K);
}

extern "C" int mi355_scratch_bytes(mi355_dev *dev, size_t *handle_bytes) {
  if (!dev || !handle_bytes) return mi355_fail(dev, MI355_ERR_ARG, "scratch_bytes: null argument");
  *handle_bytes = dev->mx_scratch_bytes;
  return MI355_OK;
}
