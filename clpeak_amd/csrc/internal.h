// Shared by the translation units of libclpeak_mi355.so.  Not installed.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstring>
#include <string>
#include "../../include/clpeak_mi355.h"

struct mi355_dev {
  int          ordinal   = -1;
  hipStream_t  stream    = nullptr;
  hipEvent_t   ev_start  = nullptr;
  hipEvent_t   ev_stop   = nullptr;
  mi355_props_t props{};
  std::string  last_error;
  // scratch owned by the handle: scale bytes of the block-scaled GEMM laid out per lane (grown on demand)
  void        *mx_scratch = nullptr;
  size_t       mx_scratch_bytes = 0;
  // device address, on this handle's device, of the static array behind mi355_gemm_mxfp4_static (set by mi355_open)
  void        *mx_static_scratch = nullptr;
  // GEMM kernels that have been allowed the whole LDS of a CU on this device (one bit per kernel)
  uint32_t     full_lds_allowed = 0;
  // which tiling the 4-, 8- and 16-bit GEMM entry points take (MI355_GEMM_TILING_*; set by mi355_gemm_tiling)
  int          gemm_tiling = 0;
};

// Error text for failures that have no handle to hang on (open, device_count).
std::string &mi355_global_error();

int mi355_fail(mi355_dev *dev, int code, const char *fmt, ...) __attribute__((format(printf, 3, 4)));

// gemm_mxfp4.hip: look up the device address of its static scratch array (the handle's device is current).
int mi355_mx_resolve_static_scratch(mi355_dev *dev);

// Wrap a HIP runtime call: on failure record "<call>: <hip error>" and return MI355_ERR_HIP.
#define MI355_HIP(dev, call)                                                            \
  do {                                                                                  \
    hipError_t e_ = (call);                                                             \
    if (e_ != hipSuccess)                                                               \
      return mi355_fail((dev), MI355_ERR_HIP, "%s: %s", #call, hipGetErrorString(e_));  \
  } while (0)

// After a <<<>>> launch: pick up launch-time errors (bad grid, missing code object).
#define MI355_LAUNCH_CHECK(dev, what)                                                   \
  do {                                                                                  \
    hipError_t e_ = hipGetLastError();                                                  \
    if (e_ != hipSuccess)                                                               \
      return mi355_fail((dev), MI355_ERR_HIP, "launch %s: %s", (what), hipGetErrorString(e_)); \
  } while (0)

#define MI355_REQUIRE(dev, cond, ...)                                                   \
  do {                                                                                  \
    if (!(cond)) return mi355_fail((dev), MI355_ERR_ARG, __VA_ARGS__);                  \
  } while (0)

// Every entry point that touches the device starts with this: validates the handle
// and makes its device current on the calling thread.
#define MI355_ENTER(dev)                                                                \
  do {                                                                                  \
    if (!(dev)) return mi355_fail(nullptr, MI355_ERR_ARG, "null device handle");        \
    MI355_HIP((dev), hipSetDevice((dev)->ordinal));                                     \
  } while (0)
