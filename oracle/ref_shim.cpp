// C entry points into the reference's own code, for tests (test infrastructure).
//
// Built only where the reference checkout is present, by ref.mk, together with the two reference
// source files it calls into, compiled where they lie:
//   src/common/common.cpp   -- pickIters, benchmark_config_t::forDevice, populate, cancel flag
//   src/cpu/thread_pool.cpp -- CpuThreadPool
//   src/cpu/cpu_kernels_tu.cpp -- the CPU backend's kernel table, once per ISA (AVX2 and AVX-512),
//                                 with the flags its CMakeLists gives that file
//                                 (src/cpu/CMakeLists.txt:94-102,142-152,338,383-388)
// Nothing else of the reference builds without its build system (result_store.cpp, options.cpp and
// clpeak_ffi.cpp include a generated version.h; the device kernels are embedded by generated code),
// so the timing discipline above the pool (CpuPeak::runWorkload) and the backends are compared by
// reading, not by running.
#include <atomic>
#include <cstdint>
#include <functional>
#include <vector>

#include <common/common.h>
#include <cpu/cpu_peak.h>

#include "cpu_kernels.h"   // src/cpu, on the include path

extern "C" const clpeak_cpu::CpuKernelTable *clpeak_table_avx2();
extern "C" const clpeak_cpu::CpuKernelTable *clpeak_table_avx512();

extern "C" {

unsigned ref_pick_iters(double per_iter_us, unsigned target_us, unsigned forced, unsigned max_iters) {
  return pickIters(per_iter_us, target_us, forced, max_iters);
}

unsigned long long ref_target_global_threads(unsigned num_cus) { return targetGlobalThreads(num_cus); }

// fields of benchmark_config_t::forDevice(type): type 1 = CPU, 2 = GPU
void ref_config_for_device(unsigned type, unsigned long long out[6]) {
  const benchmark_config_t c = benchmark_config_t::forDevice((DeviceType)type);
  out[0] = c.globalBWMaxSize; out[1] = c.computeWgsPerCU; out[2] = c.computeDPWgsPerCU;
  out[3] = c.transferBWMaxSize; out[4] = c.targetTimeUs; out[5] = c.kernelLatencyIters;
}

void ref_populate(float *dst, unsigned long long n) { populate(dst, n); }

unsigned ref_lmem_reps(void) { return LMEM_REPS; }

// CpuThreadPool: every worker 0..n-1 adds (tid+1)*iters to counts[tid]; the calling convention of
// the harness's own count hook.
void *ref_pool_create(int max_threads) { return new CpuThreadPool(max_threads); }
void ref_pool_destroy(void *p) { delete static_cast<CpuThreadPool *>(p); }
int ref_pool_max_threads(void *p) { return static_cast<CpuThreadPool *>(p)->maxThreads(); }
void ref_pool_count(void *p, int n, unsigned long long iters, unsigned long long *counts) {
  static_cast<CpuThreadPool *>(p)->run(n, [&](int tid) { counts[tid] += (unsigned long long)(tid + 1) * iters; });
}

void ref_request_cancel(void) { clpeak::requestCancel(); }
void ref_reset_cancel(void) { clpeak::resetCancel(); }
int ref_cancel_requested(void) { return clpeak::cancelRequested() ? 1 : 0; }

// --- the CPU backend's kernels: isa 0 = AVX2 table, 1 = AVX-512 table ---------------------------
// (calling into the AVX-512 table on a host without AVX-512 is the caller's mistake)
static const clpeak_cpu::CpuKernelTable *table(int isa) { return isa == 1 ? clpeak_table_avx512() : clpeak_table_avx2(); }
const char *ref_isa_name(int isa) { return table(isa)->isaName; }
// runFp32Chain (src/cpu/kernels/base_compute.h:78-102) and its flop count per outer iteration
void *ref_fp32_chain_fn(int isa) { return (void *)table(isa)->fp32.fn; }
double ref_fp32_chain_ops(int isa) { return table(isa)->fp32.opsPerIter; }
// readBufferChecksum (src/cpu/kernels/base_compute.h:301-433), the DRAM read kernel
void *ref_readsum_fn(int isa) { return (void *)table(isa)->readsum; }
}
