// The auxiliary C entry points of libclpeak_host.so (include/clpeak_host.h): the seeded operand
// generator, the calibration helpers, the result-file converter and the cancel flag.
#include <cstring>
#include "../../include/clpeak_host.h"
#include <sstream>
#include "mi355_peak.h"
#include "results.h"
#include "seeded_inputs.h"

extern "C" {

unsigned clpeak_host_pick_iters(double per_iter_us, unsigned target_us, unsigned forced, unsigned max_iters) {
  return pickIters(per_iter_us, target_us, forced, max_iters);
}

unsigned long long clpeak_host_target_global_threads(unsigned num_cus) { return targetGlobalThreads(num_cus); }

// fmt: 0 f16, 1 bf16, 2 e4m3, 3 e5m2, 4 e2m3, 5 e3m2, 6 e2m1, 7 int8.  Returns the number of bytes written.
size_t clpeak_host_seeded_operand(int fmt, double sigma, unsigned long long seed, unsigned stream, unsigned long long n,
                                  unsigned char *out, size_t cap) {
  const std::vector<uint8_t> v = seeded_operand((OperandFormat)fmt, sigma, seed, stream, n);
  if (v.size() > cap) return 0;
  memcpy(out, v.data(), v.size());
  return v.size();
}

// The same formats: n elements of the constant the reference's kernel of the format multiplies.
size_t clpeak_host_reference_operand(int fmt, unsigned long long n, unsigned char *out, size_t cap) {
  const std::vector<uint8_t> v = reference_operand((OperandFormat)fmt, n);
  if (v.size() > cap) return 0;
  memcpy(out, v.data(), v.size());
  return v.size();
}

size_t clpeak_host_seeded_bytes(int what, unsigned long long seed, unsigned stream, unsigned long long n, unsigned char *out) {
  const std::vector<uint8_t> v = what == 0 ? seeded_e8m0(seed, stream, n) : seeded_sparse_meta(seed, stream, n);
  memcpy(out, v.data(), v.size());
  return v.size();
}

// fields of benchmark_config_t::forDevice(type): type 1 = CPU, 2 = GPU
void clpeak_host_config_for_device(unsigned type, unsigned long long out[6]) {
  const benchmark_config_t c = benchmark_config_t::forDevice((DeviceType)type);
  out[0] = c.globalBWMaxSize; out[1] = c.computeWgsPerCU; out[2] = c.computeDPWgsPerCU;
  out[3] = c.transferBWMaxSize; out[4] = c.targetTimeUs; out[5] = c.kernelLatencyIters;
}

// Load a result file (any of the three formats, by extension) and write it out again as `fmt`
// (0 XML, 1 JSON, 2 CSV).  Returns the number of rows loaded, or -1 when saving failed.
int clpeak_host_resave(const char *in_path, const char *out_path, int fmt) {
  DeviceInfoStore devices;
  const ResultStore store = loadResultFile(in_path, &devices);
  const bool ok = fmt == 0 ? saveXml(store, out_path, devices) : fmt == 1 ? saveJson(store, out_path, devices) : saveCsv(store, out_path);
  return ok ? (int)store.size() : -1;
}

int clpeak_host_cancel_requested(void) { return clpeak::cancelRequested() ? 1 : 0; }
void clpeak_host_request_cancel(void) { clpeak::requestCancel(); }
void clpeak_host_reset_cancel(void) { clpeak::resetCancel(); }
}
