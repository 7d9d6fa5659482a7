// LDS ping-pong: every thread stores its value to its own slot of the workgroup's LDS array,
// the workgroup synchronises, every thread loads its right-hand neighbour's slot, the workgroup
// synchronises again; `reps` times.  After the loop a thread holds the start value of the thread
// `reps` places to its right (cyclically within the workgroup), which makes the result a closed
// form of the indices.  One repetition moves 2 * width * 4 bytes per thread through LDS.
//
// The store and the load are each one LDS instruction per thread (ds_write_b32/b64/b128 and the
// matching read); a workgroup is 4 waves by default, so 8 of them fit a CU and overlap each
// other's barrier waits.
#include "internal.h"

namespace {

template <int W> struct Vec;
template <> struct Vec<1> { typedef float type; };
template <> struct Vec<2> { typedef float2 type; };
template <> struct Vec<4> { typedef float4 type; };

__device__ inline float start_value(uint32_t gid, float *) { return (float)gid; }
__device__ inline float2 start_value(uint32_t gid, float2 *) { return make_float2((float)gid, (float)(gid + 1u)); }
__device__ inline float4 start_value(uint32_t gid, float4 *) {
  return make_float4((float)gid, (float)(gid + 1u), (float)(gid + 2u), (float)(gid + 3u));
}
__device__ inline float total(float v) { return v; }
__device__ inline float total(float2 v) { return v.x + v.y; }
__device__ inline float total(float4 v) { return v.x + v.y + v.z + v.w; }

template <int W>
__global__ void __launch_bounds__(1024) local_bandwidth_kernel(float *__restrict__ out, uint32_t reps) {
  typedef typename Vec<W>::type V;
  extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
  V *slots = reinterpret_cast<V *>(lds_raw);
  const uint32_t lid = threadIdx.x, lsize = blockDim.x;
  const uint32_t gid = blockIdx.x * lsize + lid;
  const uint32_t next = lid + 1u == lsize ? 0u : lid + 1u;
  V v = start_value(gid, (V *)nullptr);
#pragma unroll 1
  for (uint32_t i = 0; i < reps; i++) {
    slots[lid] = v;
    __syncthreads();
    v = slots[next];
    __syncthreads();
  }
  out[gid] = total(v);
}

}  // namespace

extern "C" int mi355_local_bandwidth(mi355_dev *dev, int width, float *out, uint32_t blocks, uint32_t block_size,
                                     uint32_t reps) {
  MI355_ENTER(dev);
  MI355_REQUIRE(dev, out != nullptr, "local_bandwidth: null out buffer");
  MI355_REQUIRE(dev, width == 1 || width == 2 || width == 4, "local_bandwidth: width %d not in {1,2,4}", width);
  MI355_REQUIRE(dev, blocks > 0, "local_bandwidth: zero blocks");
  MI355_REQUIRE(dev, block_size >= 64 && block_size <= 1024 && block_size % 64 == 0,
                "local_bandwidth: block_size %u must be a multiple of 64 in [64,1024]", block_size);
  MI355_REQUIRE(dev, (uint64_t)blocks * block_size <= 0xffffffffull, "local_bandwidth: more than 2^32 threads");
  const size_t lds = (size_t)block_size * (size_t)width * sizeof(float);
  switch (width) {
  case 1: local_bandwidth_kernel<1><<<blocks, block_size, lds, dev->stream>>>(out, reps); break;
  case 2: local_bandwidth_kernel<2><<<blocks, block_size, lds, dev->stream>>>(out, reps); break;
  default: local_bandwidth_kernel<4><<<blocks, block_size, lds, dev->stream>>>(out, reps); break;
  }
  MI355_LAUNCH_CHECK(dev, "local_bandwidth");
  return MI355_OK;
}
