// Seeded fills: every element is a pure function of (seed, stream, index), produced
// on the device so that multi-GiB inputs never cross PCIe.
#include "internal.h"
#include "seeded_rng.h"
#include "numeric_formats.h"

namespace {

constexpr uint32_t kFillBlock = 256;

__device__ inline float draw(uint64_t seed, uint32_t stream, uint64_t i, int dist) {
  const uint64_t z = mi355_rng_word(seed, stream, i);
  return dist == MI355_DIST_U01 ? mi355_rng_u01(z) : mi355_rng_upm1(z);
}

__global__ void fill_f32_kernel(float *dst, uint64_t n, uint64_t seed, uint32_t stream, int dist) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    dst[i] = draw(seed, stream, i, dist);
}

__global__ void fill_f64_kernel(double *dst, uint64_t n, uint64_t seed, uint32_t stream, int dist) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    dst[i] = (double)draw(seed, stream, i, dist);
}

__global__ void fill_bf16_kernel(uint16_t *dst, uint64_t n, uint64_t seed, uint32_t stream, int dist) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    dst[i] = mi355_f32_to_bf16(draw(seed, stream, i, dist));
}

__global__ void fill_fp8_kernel(uint8_t *dst, uint64_t n, uint64_t seed, uint32_t stream, int dist,
                                float scale) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    dst[i] = mi355_f32_to_e4m3(draw(seed, stream, i, dist) * scale);
}

__global__ void fill_f16_kernel(uint16_t *dst, uint64_t n, uint64_t seed, uint32_t stream, int dist) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    dst[i] = mi355_f32_to_f16(draw(seed, stream, i, dist));
}

__global__ void fill_e5m2_kernel(uint8_t *dst, uint64_t n, uint64_t seed, uint32_t stream, int dist,
                                 float scale) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    dst[i] = mi355_f32_to_e5m2(draw(seed, stream, i, dist) * scale);
}

__global__ void fill_i8_kernel(int8_t *dst, uint64_t n, uint64_t seed, uint32_t stream) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    dst[i] = (int8_t)((int)(mi355_rng_word(seed, stream, i) >> 60) - 8);
}

__global__ void fill_bytes_kernel(uint8_t *dst, uint64_t n, uint64_t seed, uint32_t stream, uint32_t lo, uint32_t span) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    dst[i] = (uint8_t)(lo + mi355_rng_below(mi355_rng_word(seed, stream, i), span));
}

typedef int copy_vec __attribute__((ext_vector_type(4)));
__global__ void copy_kernel(copy_vec *__restrict__ dst, const copy_vec *__restrict__ src, uint64_t n) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}

uint32_t fill_grid(uint64_t n) {
  uint64_t blocks = (n + kFillBlock - 1) / kFillBlock;
  const uint64_t cap = 256u * 32u;  // 32 workgroups per CU is plenty for a store-bound fill
  return (uint32_t)(blocks < cap ? blocks : cap);
}

int check_fill(mi355_dev *dev, const void *dst, uint64_t n, int dist) {
  MI355_REQUIRE(dev, dst != nullptr, "fill: null destination");
  MI355_REQUIRE(dev, n > 0, "fill: zero elements");
  MI355_REQUIRE(dev, dist == MI355_DIST_U01 || dist == MI355_DIST_UPM1, "fill: unknown dist %d", dist);
  return MI355_OK;
}

}  // namespace

extern "C" int mi355_fill_f32(mi355_dev *dev, float *dst, uint64_t n, uint64_t seed, uint32_t stream,
                              int dist) {
  MI355_ENTER(dev);
  if (int rc = check_fill(dev, dst, n, dist)) return rc;
  fill_f32_kernel<<<fill_grid(n), kFillBlock, 0, dev->stream>>>(dst, n, seed, stream, dist);
  MI355_LAUNCH_CHECK(dev, "fill_f32");
  return MI355_OK;
}

extern "C" int mi355_fill_f64(mi355_dev *dev, double *dst, uint64_t n, uint64_t seed, uint32_t stream,
                              int dist) {
  MI355_ENTER(dev);
  if (int rc = check_fill(dev, dst, n, dist)) return rc;
  fill_f64_kernel<<<fill_grid(n), kFillBlock, 0, dev->stream>>>(dst, n, seed, stream, dist);
  MI355_LAUNCH_CHECK(dev, "fill_f64");
  return MI355_OK;
}

extern "C" int mi355_fill_bf16(mi355_dev *dev, uint16_t *dst, uint64_t n, uint64_t seed,
                               uint32_t stream, int dist) {
  MI355_ENTER(dev);
  if (int rc = check_fill(dev, dst, n, dist)) return rc;
  fill_bf16_kernel<<<fill_grid(n), kFillBlock, 0, dev->stream>>>(dst, n, seed, stream, dist);
  MI355_LAUNCH_CHECK(dev, "fill_bf16");
  return MI355_OK;
}

extern "C" int mi355_fill_fp8_e4m3(mi355_dev *dev, uint8_t *dst, uint64_t n, uint64_t seed,
                                   uint32_t stream, int dist, float scale) {
  MI355_ENTER(dev);
  if (int rc = check_fill(dev, dst, n, dist)) return rc;
  fill_fp8_kernel<<<fill_grid(n), kFillBlock, 0, dev->stream>>>(dst, n, seed, stream, dist, scale);
  MI355_LAUNCH_CHECK(dev, "fill_fp8_e4m3");
  return MI355_OK;
}

extern "C" int mi355_fill_f16(mi355_dev *dev, uint16_t *dst, uint64_t n, uint64_t seed, uint32_t stream,
                              int dist) {
  MI355_ENTER(dev);
  if (int rc = check_fill(dev, dst, n, dist)) return rc;
  fill_f16_kernel<<<fill_grid(n), kFillBlock, 0, dev->stream>>>(dst, n, seed, stream, dist);
  MI355_LAUNCH_CHECK(dev, "fill_f16");
  return MI355_OK;
}

extern "C" int mi355_fill_fp8_e5m2(mi355_dev *dev, uint8_t *dst, uint64_t n, uint64_t seed,
                                   uint32_t stream, int dist, float scale) {
  MI355_ENTER(dev);
  if (int rc = check_fill(dev, dst, n, dist)) return rc;
  fill_e5m2_kernel<<<fill_grid(n), kFillBlock, 0, dev->stream>>>(dst, n, seed, stream, dist, scale);
  MI355_LAUNCH_CHECK(dev, "fill_fp8_e5m2");
  return MI355_OK;
}

extern "C" int mi355_fill_i8(mi355_dev *dev, int8_t *dst, uint64_t n, uint64_t seed, uint32_t stream) {
  MI355_ENTER(dev);
  if (int rc = check_fill(dev, dst, n, MI355_DIST_U01)) return rc;
  fill_i8_kernel<<<fill_grid(n), kFillBlock, 0, dev->stream>>>(dst, n, seed, stream);
  MI355_LAUNCH_CHECK(dev, "fill_i8");
  return MI355_OK;
}

extern "C" int mi355_fill_bytes(mi355_dev *dev, uint8_t *dst, uint64_t n, uint64_t seed, uint32_t stream,
                                uint32_t lo, uint32_t span) {
  MI355_ENTER(dev);
  if (int rc = check_fill(dev, dst, n, MI355_DIST_U01)) return rc;
  MI355_REQUIRE(dev, span >= 1 && lo + span <= 256, "fill_bytes: [lo, lo+span) must lie within a byte");
  fill_bytes_kernel<<<fill_grid(n), kFillBlock, 0, dev->stream>>>(dst, n, seed, stream, lo, span);
  MI355_LAUNCH_CHECK(dev, "fill_bytes");
  return MI355_OK;
}

extern "C" int mi355_copy(mi355_dev *dev, void *dst, const void *src, size_t bytes) {
  MI355_ENTER(dev);
  MI355_REQUIRE(dev, dst && src, "copy: null pointer");
  MI355_REQUIRE(dev, bytes > 0 && bytes % 16 == 0, "copy: size must be a positive multiple of 16");
  MI355_REQUIRE(dev, (((uintptr_t)dst | (uintptr_t)src) & 15u) == 0, "copy: pointers must be 16-byte aligned");
  copy_kernel<<<fill_grid(bytes / 16), kFillBlock, 0, dev->stream>>>((copy_vec *)dst, (const copy_vec *)src, bytes / 16);
  MI355_LAUNCH_CHECK(dev, "copy");
  return MI355_OK;
}
