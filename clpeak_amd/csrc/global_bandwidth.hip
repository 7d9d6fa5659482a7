// Global-memory streaming read: float / float2 / float4 grid-stride read-reduce.
//
// T threads in total; thread t owns vector elements t, t+T, t+2T, ... so that at
// every step a wavefront reads 64 consecutive vectors (256 B / 512 B / 1 KiB
// contiguous) and the whole grid sweeps the buffer front to back.  The loop is
// unrolled so each thread keeps kUnroll independent loads in flight; the adds are
// then done in element order, which keeps every partial sum a fixed sequence of
// fp32 additions that a CPU can replay bit for bit.
//
// Tuning, measured on MI355X over a 4 GiB buffer: the loads of one unrolled group are
// T vectors apart, so a small grid (one or two 256-thread workgroups per CU) keeps the
// group inside a few 2 MiB pages and beats a large grid by ~15 %; about 96 bytes in
// flight per lane (6 float4, 12 float2, 24 float loads) is the sweet spot; the loads
// are nontemporal (streaming: +12 % over cached loads).
//
// HBM-bound: 4 bytes read per float, 4 bytes written per thread (negligible).
#include "internal.h"

namespace {

typedef float float2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));

template <typename V> struct Lanes;
template <> struct Lanes<float>   { static constexpr int n = 1; };
template <> struct Lanes<float2v> { static constexpr int n = 2; };
template <> struct Lanes<float4v> { static constexpr int n = 4; };

__device__ inline float hsum(float v)   { return v; }
__device__ inline float hsum(float2v v) { return v.x + v.y; }
__device__ inline float hsum(float4v v) { return ((v.x + v.y) + v.z) + v.w; }

template <typename V, int kUnroll>
__global__ void __launch_bounds__(1024)
global_bandwidth_kernel(const V *__restrict__ in, uint64_t nvec, float *__restrict__ out) {
  const uint64_t T = (uint64_t)gridDim.x * blockDim.x;
  const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  V acc = (V)(0.0f);
  uint64_t i = t;
  // Full groups of kUnroll strided loads.
  if (nvec >= (uint64_t)(kUnroll - 1) * T) {
    const uint64_t last_full = nvec - (uint64_t)(kUnroll - 1) * T;  // i < last_full => all kUnroll loads in range
    for (; i < last_full; i += (uint64_t)kUnroll * T) {
      V v[kUnroll];
#pragma unroll
      for (int k = 0; k < kUnroll; k++) v[k] = __builtin_nontemporal_load(in + i + (uint64_t)k * T);
#pragma unroll
      for (int k = 0; k < kUnroll; k++) acc += v[k];
    }
  }
  for (; i < nvec; i += T) acc += __builtin_nontemporal_load(in + i);
  out[t] = hsum(acc);
}

template <typename V>
int launch(mi355_dev *dev, const float *in, uint64_t n_floats, float *out, uint32_t blocks,
           uint32_t block_size) {
  const uint64_t nvec = n_floats / Lanes<V>::n;
  constexpr int kUnroll = 24 / Lanes<V>::n;  // 96 bytes in flight per lane
  global_bandwidth_kernel<V, kUnroll><<<blocks, block_size, 0, dev->stream>>>(
      reinterpret_cast<const V *>(in), nvec, out);
  MI355_LAUNCH_CHECK(dev, "global_bandwidth");
  return MI355_OK;
}

}  // namespace

extern "C" int mi355_global_bandwidth(mi355_dev *dev, int width, const float *in, uint64_t n_floats,
                                      float *out, uint32_t blocks, uint32_t block_size) {
  MI355_ENTER(dev);
  MI355_REQUIRE(dev, in && out, "global_bandwidth: null buffer");
  MI355_REQUIRE(dev, width == 1 || width == 2 || width == 4, "global_bandwidth: width %d not in {1,2,4}", width);
  MI355_REQUIRE(dev, n_floats % (uint64_t)width == 0, "global_bandwidth: n_floats not a multiple of width");
  MI355_REQUIRE(dev, ((uintptr_t)in & 15u) == 0, "global_bandwidth: input not 16-byte aligned");
  MI355_REQUIRE(dev, blocks > 0, "global_bandwidth: zero blocks");
  MI355_REQUIRE(dev, block_size == 64 || block_size == 128 || block_size == 256 || block_size == 512 ||
                         block_size == 1024,
                "global_bandwidth: block_size %u not in {64,128,256,512,1024}", block_size);
  switch (width) {
    case 1: return launch<float>(dev, in, n_floats, out, blocks, block_size);
    case 2: return launch<float2v>(dev, in, n_floats, out, blocks, block_size);
    default: return launch<float4v>(dev, in, n_floats, out, blocks, block_size);
  }
}
