// The C ABI of libclpeak_mi355.so as a table of function pointers.  The backend class talks
// to the GPU only through such a table.  The program and the library that ship bind the entry
// points of libclpeak_mi355.so (device_api.cpp) and nothing else; the host-logic tests link the
// same classes against a table of their own instead of device_api.cpp.
#pragma once
#include "../../include/clpeak_mi355.h"

struct Mi355Api {
  decltype(&mi355_device_count) device_count;
  decltype(&mi355_open) open;
  decltype(&mi355_close) close;
  decltype(&mi355_get_props) get_props;
  decltype(&mi355_last_error) last_error;
  decltype(&mi355_alloc) alloc;
  decltype(&mi355_free) free;
  decltype(&mi355_upload) upload;
  decltype(&mi355_download) download;
  decltype(&mi355_sync) sync;
  decltype(&mi355_timer_start) timer_start;
  decltype(&mi355_timer_stop) timer_stop;
  decltype(&mi355_fill_f32) fill_f32;
  decltype(&mi355_fill_bf16) fill_bf16;
  decltype(&mi355_fill_fp8_e4m3) fill_fp8_e4m3;
  decltype(&mi355_global_bandwidth) global_bandwidth;
  decltype(&mi355_compute_mad) compute_mad;
  decltype(&mi355_launch_roundtrip) launch_roundtrip;
  decltype(&mi355_mfma_dense) mfma_dense;
  decltype(&mi355_smfmac) smfmac;
  decltype(&mi355_gemm_bf16) gemm_bf16;
  decltype(&mi355_gemm_fp8_e4m3) gemm_fp8_e4m3;
  decltype(&mi355_local_bandwidth) local_bandwidth;
  decltype(&mi355_host_alloc) host_alloc;
  decltype(&mi355_host_free) host_free;
  decltype(&mi355_copy_async) copy_async;
  decltype(&mi355_fill_f16) fill_f16;
  decltype(&mi355_fill_fp8_e5m2) fill_fp8_e5m2;
  decltype(&mi355_fill_i8) fill_i8;
  decltype(&mi355_gemm_f16) gemm_f16;
  decltype(&mi355_gemm_i8) gemm_i8;
  decltype(&mi355_gemm_fp8_e5m2) gemm_fp8_e5m2;
  decltype(&mi355_gemm_mxfp4) gemm_mxfp4;
  decltype(&mi355_fill_bytes) fill_bytes;
  decltype(&mi355_fill_f64) fill_f64;
  decltype(&mi355_gemm_f32) gemm_f32;
  decltype(&mi355_gemm_f64) gemm_f64;
  decltype(&mi355_gemm_mxfp4_prepare_scales) gemm_mxfp4_prepare_scales;
  decltype(&mi355_gemm_mxfp4_prepared) gemm_mxfp4_prepared;
};

const Mi355Api &mi355_api();   // the table this binary is linked with
