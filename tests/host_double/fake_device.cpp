// TEST DOUBLE, never linked into the program or the library that ship: a pretend device behind
// the Mi355Api table, built only into tests/host_double/clpeak-mi355-double and
// libclpeak_host_double.so, where it takes the place of clpeak_amd/host/device_api.cpp.
// No GPU, no arithmetic.  Allocations are sizes
// only (nothing is dereferenced), every launch "takes" a fixed time, and environment
// variables can inject failures so that the backend's degrade paths can be tested:
//   CLPEAK_FAKE_DEVICES=n          number of devices (default 1)
//   CLPEAK_FAKE_FAIL=<entry>       that entry point fails (alloc, mfma_dense, gemm_bf16, ...)
#include <cstdlib>
#include <cstring>
#include <string>
#include "../../clpeak_amd/host/device_api.h"

struct mi355_dev {
  std::string error;
  unsigned launches = 0;
};

namespace {
bool fails(const char *what) {
  const char *f = getenv("CLPEAK_FAKE_FAIL");
  return f && strcmp(f, what) == 0;
}
int fail(mi355_dev *d, const char *what) {
  d->error = std::string("fake device: injected failure in ") + what;
  return MI355_ERR_HIP;
}
#define FAKE_ENTRY(dev, name) do { if (fails(name)) return fail(dev, name); (dev)->launches++; } while (0)

int f_device_count(int *n) {
  const char *e = getenv("CLPEAK_FAKE_DEVICES");
  *n = e ? atoi(e) : 1;
  return MI355_OK;
}
int f_open(int ordinal, mi355_dev **out) {
  int n = 0;
  f_device_count(&n);
  if (ordinal < 0 || ordinal >= n) return MI355_ERR_NODEV;
  *out = new mi355_dev();
  return MI355_OK;
}
int f_close(mi355_dev *d) { delete d; return MI355_OK; }
int f_get_props(mi355_dev *, mi355_props_t *p) {
  memset(p, 0, sizeof(*p));
  strcpy(p->name, "Fake MI355X");
  strcpy(p->arch, "gfx950:sramecc+:xnack-");
  strcpy(p->driver_version, "7.2.0");
  strcpy(p->runtime_version, "7.2.26015");
  p->num_cus = 256; p->wave_size = 64; p->max_threads_per_block = 1024; p->clock_khz = 2400000;
  p->total_mem = 288ull << 30;
  return MI355_OK;
}
const char *f_last_error(mi355_dev *d) { return d ? d->error.c_str() : "fake device: no such device"; }
int f_alloc(mi355_dev *d, size_t bytes, void **p) {
  FAKE_ENTRY(d, "alloc");
  *p = (void *)(uintptr_t)(0x1000 + bytes % 4096 * 0);   // never dereferenced
  *p = (void *)(uintptr_t)0x100000;
  return MI355_OK;
}
int f_free(mi355_dev *, void *) { return MI355_OK; }
int f_upload(mi355_dev *d, void *, const void *, size_t) { FAKE_ENTRY(d, "upload"); return MI355_OK; }
int f_download(mi355_dev *d, void *dst, const void *, size_t n) { FAKE_ENTRY(d, "download"); memset(dst, 0, n); return MI355_OK; }
int f_sync(mi355_dev *) { return MI355_OK; }
int f_timer_start(mi355_dev *d) { d->launches = 0; return MI355_OK; }
int f_timer_stop(mi355_dev *d, float *us) { *us = 100.0f * (float)(d->launches ? d->launches : 1); return MI355_OK; }
int f_fill_f32(mi355_dev *d, float *, uint64_t, uint64_t, uint32_t, int) { FAKE_ENTRY(d, "fill_f32"); return MI355_OK; }
int f_fill_bf16(mi355_dev *d, uint16_t *, uint64_t, uint64_t, uint32_t, int) { FAKE_ENTRY(d, "fill_bf16"); return MI355_OK; }
int f_fill_fp8(mi355_dev *d, uint8_t *, uint64_t, uint64_t, uint32_t, int, float) { FAKE_ENTRY(d, "fill_fp8_e4m3"); return MI355_OK; }
int f_global_bandwidth(mi355_dev *d, int, const float *, uint64_t, float *, uint32_t, uint32_t) { FAKE_ENTRY(d, "global_bandwidth"); return MI355_OK; }
int f_compute_mad(mi355_dev *d, int, int, uint64_t, uint64_t, uint32_t, void *, uint32_t) { FAKE_ENTRY(d, "compute_mad"); return MI355_OK; }
int f_launch_roundtrip(mi355_dev *d, uint32_t, uint32_t, double *us) { FAKE_ENTRY(d, "launch_roundtrip"); *us = 9.5; return MI355_OK; }
int f_mfma_dense(mi355_dev *d, int, const void *, const void *, const uint8_t *, const uint8_t *, void *, uint32_t, uint32_t, uint64_t *) { FAKE_ENTRY(d, "mfma_dense"); return MI355_OK; }
int f_smfmac(mi355_dev *d, int, const void *, const uint8_t *, const void *, void *, uint32_t, uint32_t, uint64_t *) { FAKE_ENTRY(d, "smfmac"); return MI355_OK; }
int f_gemm_bf16(mi355_dev *d, const uint16_t *, const uint16_t *, uint16_t *, uint32_t, uint32_t, uint32_t) { FAKE_ENTRY(d, "gemm_bf16"); return MI355_OK; }
int f_gemm_fp8(mi355_dev *d, const uint8_t *, const uint8_t *, uint16_t *, uint32_t, uint32_t, uint32_t, float, float) { FAKE_ENTRY(d, "gemm_fp8_e4m3"); return MI355_OK; }
int f_local_bandwidth(mi355_dev *d, int, float *, uint32_t, uint32_t, uint32_t) { FAKE_ENTRY(d, "local_bandwidth"); return MI355_OK; }
int f_host_alloc(mi355_dev *d, size_t bytes, void **p) {
  FAKE_ENTRY(d, "host_alloc");
  *p = malloc(bytes);
  return *p ? MI355_OK : MI355_ERR_OOM;
}
int f_host_free(mi355_dev *, void *p) { free(p); return MI355_OK; }
int f_copy_async(mi355_dev *d, void *, const void *, size_t, int) { FAKE_ENTRY(d, "copy_async"); return MI355_OK; }
int f_fill_f16(mi355_dev *d, uint16_t *, uint64_t, uint64_t, uint32_t, int) { FAKE_ENTRY(d, "fill_f16"); return MI355_OK; }
int f_fill_e5m2(mi355_dev *d, uint8_t *, uint64_t, uint64_t, uint32_t, int, float) { FAKE_ENTRY(d, "fill_fp8_e5m2"); return MI355_OK; }
int f_fill_i8(mi355_dev *d, int8_t *, uint64_t, uint64_t, uint32_t) { FAKE_ENTRY(d, "fill_i8"); return MI355_OK; }
int f_gemm_f16(mi355_dev *d, const uint16_t *, const uint16_t *, uint16_t *, uint32_t, uint32_t, uint32_t) { FAKE_ENTRY(d, "gemm_f16"); return MI355_OK; }
int f_gemm_i8(mi355_dev *d, const int8_t *, const int8_t *, int32_t *, uint32_t, uint32_t, uint32_t) { FAKE_ENTRY(d, "gemm_i8"); return MI355_OK; }
int f_gemm_e5m2(mi355_dev *d, const uint8_t *, const uint8_t *, uint16_t *, uint32_t, uint32_t, uint32_t, float, float) { FAKE_ENTRY(d, "gemm_fp8_e5m2"); return MI355_OK; }
int f_gemm_mxfp4(mi355_dev *d, const uint8_t *, const uint8_t *, const uint8_t *, const uint8_t *, uint16_t *, uint32_t, uint32_t, uint32_t) { FAKE_ENTRY(d, "gemm_mxfp4"); return MI355_OK; }
int f_mx_prepare(mi355_dev *d, const uint8_t *, const uint8_t *, uint32_t, uint32_t, uint32_t, uint8_t *) { FAKE_ENTRY(d, "gemm_mxfp4_prepare_scales"); return MI355_OK; }
int f_mx_prepared(mi355_dev *d, const uint8_t *, const uint8_t *, const uint8_t *, uint16_t *, uint32_t, uint32_t, uint32_t) { FAKE_ENTRY(d, "gemm_mxfp4"); return MI355_OK; }
int f_fill_bytes(mi355_dev *d, uint8_t *, uint64_t, uint64_t, uint32_t, uint32_t, uint32_t) { FAKE_ENTRY(d, "fill_bytes"); return MI355_OK; }
int f_fill_f64(mi355_dev *d, double *, uint64_t, uint64_t, uint32_t, int) { FAKE_ENTRY(d, "fill_f64"); return MI355_OK; }
int f_gemm_f32(mi355_dev *d, const float *, const float *, float *, uint32_t, uint32_t, uint32_t) { FAKE_ENTRY(d, "gemm_f32"); return MI355_OK; }
int f_gemm_f64(mi355_dev *d, const double *, const double *, double *, uint32_t, uint32_t, uint32_t) { FAKE_ENTRY(d, "gemm_f64"); return MI355_OK; }
}  // namespace

const Mi355Api &mi355_api() {
  static const Mi355Api api = {
      f_device_count, f_open, f_close, f_get_props, f_last_error, f_alloc, f_free, f_upload, f_download, f_sync,
      f_timer_start, f_timer_stop, f_fill_f32, f_fill_bf16, f_fill_fp8, f_global_bandwidth, f_compute_mad,
      f_launch_roundtrip, f_mfma_dense, f_smfmac, f_gemm_bf16, f_gemm_fp8,
      f_local_bandwidth, f_host_alloc, f_host_free, f_copy_async,
      f_fill_f16, f_fill_e5m2, f_fill_i8, f_gemm_f16, f_gemm_i8, f_gemm_e5m2,
      f_gemm_mxfp4, f_fill_bytes, f_fill_f64, f_gemm_f32, f_gemm_f64, f_mx_prepare, f_mx_prepared};
  return api;
}
