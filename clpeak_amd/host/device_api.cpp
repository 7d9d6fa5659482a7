#include "device_api.h"

// The entry points of libclpeak_mi355.so.
const Mi355Api &mi355_api() {
  static const Mi355Api api = {
      mi355_device_count, mi355_open, mi355_close, mi355_get_props, mi355_last_error, mi355_alloc, mi355_free,
      mi355_upload, mi355_download, mi355_sync, mi355_timer_start, mi355_timer_stop, mi355_fill_f32,
      mi355_fill_bf16, mi355_fill_fp8_e4m3, mi355_global_bandwidth, mi355_compute_mad, mi355_launch_roundtrip,
      mi355_mfma_dense, mi355_smfmac, mi355_gemm_bf16, mi355_gemm_fp8_e4m3,
      mi355_local_bandwidth, mi355_host_alloc, mi355_host_free, mi355_copy_async,
      mi355_fill_f16, mi355_fill_fp8_e5m2, mi355_fill_i8, mi355_gemm_f16, mi355_gemm_i8, mi355_gemm_fp8_e5m2,
      mi355_gemm_mxfp4, mi355_fill_bytes, mi355_fill_f64, mi355_gemm_f32, mi355_gemm_f64,
      mi355_gemm_mxfp4_prepare_scales, mi355_gemm_mxfp4_prepared};
  return api;
}
