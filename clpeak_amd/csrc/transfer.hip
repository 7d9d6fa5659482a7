// Pinned host memory and asynchronous host<->device copies on the handle's stream: the pieces the
// PCIe transfer test is made of.  The copies are enqueued without waiting, so that a batch of them
// can sit between the two timer events like a batch of kernel launches.
#include "internal.h"

extern "C" int mi355_host_alloc(mi355_dev *dev, size_t bytes, void **hptr) {
  MI355_ENTER(dev);
  MI355_REQUIRE(dev, hptr != nullptr && bytes > 0, "host_alloc: null out pointer or zero size");
  *hptr = nullptr;
  const hipError_t e = hipHostMalloc(hptr, bytes, hipHostMallocDefault);
  if (e == hipErrorOutOfMemory)
    return mi355_fail(dev, MI355_ERR_OOM, "hipHostMalloc(%zu bytes): out of pinned host memory", bytes);
  if (e != hipSuccess)
    return mi355_fail(dev, MI355_ERR_HIP, "hipHostMalloc(%zu bytes): %s", bytes, hipGetErrorString(e));
  return MI355_OK;
}

extern "C" int mi355_host_free(mi355_dev *dev, void *hptr) {
  MI355_ENTER(dev);
  if (!hptr) return MI355_OK;
  MI355_HIP(dev, hipStreamSynchronize(dev->stream));
  MI355_HIP(dev, hipHostFree(hptr));
  return MI355_OK;
}

extern "C" int mi355_copy_async(mi355_dev *dev, void *dst, const void *src, size_t bytes, int direction) {
  MI355_ENTER(dev);
  MI355_REQUIRE(dev, dst && src, "copy_async: null pointer");
  MI355_REQUIRE(dev, direction == MI355_H2D || direction == MI355_D2H, "copy_async: direction %d", direction);
  if (bytes == 0) return MI355_OK;
  MI355_HIP(dev, hipMemcpyAsync(dst, src, bytes, direction == MI355_H2D ? hipMemcpyHostToDevice : hipMemcpyDeviceToHost,
                                dev->stream));
  return MI355_OK;
}
