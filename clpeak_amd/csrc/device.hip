// Device handle, memory and timing entry points of the C ABI.
#include "internal.h"
#include <cstdarg>

std::string &mi355_global_error() {
  static thread_local std::string s;
  return s;
}

int mi355_fail(mi355_dev *dev, int code, const char *fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  if (dev) dev->last_error = buf;
  else mi355_global_error() = buf;
  return code;
}

static void format_version(int v, char *dst, size_t n) {
  // HIP packs versions as major*10'000'000 + minor*100'000 + patch.
  snprintf(dst, n, "%d.%d.%d", v / 10000000, (v / 100000) % 100, v % 100000);
}

extern "C" int mi355_device_count(int *count) {
  if (!count) return mi355_fail(nullptr, MI355_ERR_ARG, "count is null");
  *count = 0;
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e == hipErrorNoDevice) return MI355_OK;
  if (e != hipSuccess)
    return mi355_fail(nullptr, MI355_ERR_HIP, "hipGetDeviceCount: %s", hipGetErrorString(e));
  *count = n;
  return MI355_OK;
}

extern "C" int mi355_open(int ordinal, mi355_dev **out) {
  if (!out) return mi355_fail(nullptr, MI355_ERR_ARG, "out is null");
  *out = nullptr;
  int n = 0;
  int rc = mi355_device_count(&n);
  if (rc != MI355_OK) return rc;
  if (ordinal < 0 || ordinal >= n)
    return mi355_fail(nullptr, MI355_ERR_NODEV, "no HIP device with ordinal %d (%d present)", ordinal, n);

  hipDeviceProp_t p;
  hipError_t e = hipGetDeviceProperties(&p, ordinal);
  if (e != hipSuccess)
    return mi355_fail(nullptr, MI355_ERR_HIP, "hipGetDeviceProperties: %s", hipGetErrorString(e));
  if (strncmp(p.gcnArchName, "gfx950", 6) != 0)
    return mi355_fail(nullptr, MI355_ERR_ARCH,
                      "device %d is %s; this backend holds gfx950 code only", ordinal, p.gcnArchName);

  e = hipSetDevice(ordinal);
  if (e != hipSuccess)
    return mi355_fail(nullptr, MI355_ERR_HIP, "hipSetDevice: %s", hipGetErrorString(e));

  mi355_dev *d = new mi355_dev();
  d->ordinal = ordinal;
  // Some driver stacks report an empty marketing name; rows need a device string.
  if (p.name[0]) snprintf(d->props.name, sizeof(d->props.name), "%s", p.name);
  else snprintf(d->props.name, sizeof(d->props.name), "AMD GPU %.6s", p.gcnArchName);
  snprintf(d->props.arch, sizeof(d->props.arch), "%s", p.gcnArchName);
  int drv = 0, rt = 0;
  (void)hipDriverGetVersion(&drv);
  (void)hipRuntimeGetVersion(&rt);
  format_version(drv, d->props.driver_version, sizeof(d->props.driver_version));
  format_version(rt, d->props.runtime_version, sizeof(d->props.runtime_version));
  d->props.num_cus = p.multiProcessorCount;
  d->props.wave_size = p.warpSize;
  d->props.max_threads_per_block = p.maxThreadsPerBlock;
  d->props.clock_khz = p.clockRate;
  d->props.total_mem = (uint64_t)p.totalGlobalMem;

  if ((e = hipStreamCreateWithFlags(&d->stream, hipStreamNonBlocking)) != hipSuccess ||
      (e = hipEventCreate(&d->ev_start)) != hipSuccess ||
      (e = hipEventCreate(&d->ev_stop)) != hipSuccess) {
    int code = mi355_fail(nullptr, MI355_ERR_HIP, "stream/event creation: %s", hipGetErrorString(e));
    mi355_close(d);
    return code;
  }
  // the one array of the library that lives in device memory from load to exit: its address on this device
  if (int code = mi355_mx_resolve_static_scratch(d)) {
    mi355_global_error() = d->last_error;
    mi355_close(d);
    return code;
  }
  *out = d;
  return MI355_OK;
}

extern "C" int mi355_close(mi355_dev *dev) {
  if (!dev) return MI355_OK;
  (void)hipSetDevice(dev->ordinal);
  if (dev->stream) (void)hipStreamSynchronize(dev->stream);
  if (dev->mx_scratch) (void)hipFree(dev->mx_scratch);
  if (dev->ev_start) (void)hipEventDestroy(dev->ev_start);
  if (dev->ev_stop) (void)hipEventDestroy(dev->ev_stop);
  if (dev->stream) (void)hipStreamDestroy(dev->stream);
  delete dev;
  return MI355_OK;
}

extern "C" int mi355_get_props(mi355_dev *dev, mi355_props_t *out) {
  if (!dev || !out) return mi355_fail(dev, MI355_ERR_ARG, "null argument");
  *out = dev->props;
  return MI355_OK;
}

extern "C" const char *mi355_last_error(mi355_dev *dev) {
  return dev ? dev->last_error.c_str() : mi355_global_error().c_str();
}

extern "C" int mi355_alloc(mi355_dev *dev, size_t bytes, void **dptr) {
  MI355_ENTER(dev);
  MI355_REQUIRE(dev, dptr != nullptr && bytes > 0, "alloc: null out pointer or zero size");
  *dptr = nullptr;
  hipError_t e = hipMalloc(dptr, bytes);
  if (e == hipErrorOutOfMemory)
    return mi355_fail(dev, MI355_ERR_OOM, "hipMalloc(%zu bytes): out of device memory", bytes);
  if (e != hipSuccess)
    return mi355_fail(dev, MI355_ERR_HIP, "hipMalloc(%zu bytes): %s", bytes, hipGetErrorString(e));
  return MI355_OK;
}

extern "C" int mi355_free(mi355_dev *dev, void *dptr) {
  MI355_ENTER(dev);
  if (!dptr) return MI355_OK;
  MI355_HIP(dev, hipStreamSynchronize(dev->stream));
  MI355_HIP(dev, hipFree(dptr));
  return MI355_OK;
}

extern "C" int mi355_upload(mi355_dev *dev, void *dst_dev, const void *src_host, size_t bytes) {
  MI355_ENTER(dev);
  MI355_REQUIRE(dev, dst_dev && src_host, "upload: null pointer");
  if (bytes == 0) return MI355_OK;
  MI355_HIP(dev, hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, dev->stream));
  MI355_HIP(dev, hipStreamSynchronize(dev->stream));
  return MI355_OK;
}

extern "C" int mi355_download(mi355_dev *dev, void *dst_host, const void *src_dev, size_t bytes) {
  MI355_ENTER(dev);
  MI355_REQUIRE(dev, dst_host && src_dev, "download: null pointer");
  if (bytes == 0) return MI355_OK;
  MI355_HIP(dev, hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, dev->stream));
  MI355_HIP(dev, hipStreamSynchronize(dev->stream));
  return MI355_OK;
}

extern "C" int mi355_memset(mi355_dev *dev, void *dptr, int byte, size_t bytes) {
  MI355_ENTER(dev);
  MI355_REQUIRE(dev, dptr != nullptr, "memset: null pointer");
  if (bytes == 0) return MI355_OK;
  MI355_HIP(dev, hipMemsetAsync(dptr, byte, bytes, dev->stream));
  return MI355_OK;
}

extern "C" int mi355_sync(mi355_dev *dev) {
  MI355_ENTER(dev);
  MI355_HIP(dev, hipStreamSynchronize(dev->stream));
  return MI355_OK;
}

extern "C" int mi355_timer_start(mi355_dev *dev) {
  MI355_ENTER(dev);
  MI355_HIP(dev, hipEventRecord(dev->ev_start, dev->stream));
  return MI355_OK;
}

extern "C" int mi355_timer_stop(mi355_dev *dev, float *elapsed_us) {
  MI355_ENTER(dev);
  MI355_REQUIRE(dev, elapsed_us != nullptr, "timer_stop: null out pointer");
  MI355_HIP(dev, hipEventRecord(dev->ev_stop, dev->stream));
  MI355_HIP(dev, hipEventSynchronize(dev->ev_stop));
  float ms = 0.0f;
  MI355_HIP(dev, hipEventElapsedTime(&ms, dev->ev_start, dev->ev_stop));
  *elapsed_us = ms * 1000.0f;
  return MI355_OK;
}
