// Launch round-trip probe: an empty 1x1x1 kernel, launched and waited for one at a
// time, wall-clocked on the host.
#include "internal.h"
#include <chrono>

namespace {
__global__ void noop_kernel() {}
}  // namespace

extern "C" int mi355_launch_roundtrip(mi355_dev *dev, uint32_t warmup, uint32_t launches, double *mean_us) {
  MI355_ENTER(dev);
  MI355_REQUIRE(dev, mean_us != nullptr, "launch_roundtrip: null out pointer");
  MI355_REQUIRE(dev, launches > 0, "launch_roundtrip: zero launches");
  *mean_us = 0.0;
  for (uint32_t w = 0; w < warmup; w++) {
    noop_kernel<<<1, 1, 0, dev->stream>>>();
    MI355_LAUNCH_CHECK(dev, "noop");
    MI355_HIP(dev, hipStreamSynchronize(dev->stream));
  }
  double total_ns = 0.0;
  for (uint32_t i = 0; i < launches; i++) {
    const auto t0 = std::chrono::steady_clock::now();
    noop_kernel<<<1, 1, 0, dev->stream>>>();
    const hipError_t le = hipGetLastError();
    const hipError_t se = hipStreamSynchronize(dev->stream);
    const auto t1 = std::chrono::steady_clock::now();
    if (le != hipSuccess) return mi355_fail(dev, MI355_ERR_HIP, "launch noop: %s", hipGetErrorString(le));
    if (se != hipSuccess) return mi355_fail(dev, MI355_ERR_HIP, "hipStreamSynchronize: %s", hipGetErrorString(se));
    total_ns += (double)std::chrono::duration_cast<std::chrono::nanoseconds>(t1 - t0).count();
  }
  *mean_us = total_ns / 1000.0 / (double)launches;
  return MI355_OK;
}
