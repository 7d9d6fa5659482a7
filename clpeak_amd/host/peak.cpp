#include "peak.h"
#include <atomic>

unsigned pickIters(double per_iter_us, unsigned target_us, unsigned forced, unsigned max_iters) {
  if (forced) return forced;
  const double budget = target_us ? (double)target_us : 5e6;
  double n = budget / (per_iter_us < 1.0 ? 1.0 : per_iter_us);
  if (n > (double)max_iters) n = (double)max_iters;
  return n < 1.0 ? 1u : (unsigned)n;
}

benchmark_config_t benchmark_config_t::forDevice(DeviceType type) {
  const bool cpu = type == DeviceType::Cpu;
  benchmark_config_t c;
  c.globalBWMaxSize = cpu ? (1ull << 27) : (1ull << 29);
  c.transferBWMaxSize = c.globalBWMaxSize;
  c.computeWgsPerCU = cpu ? 512 : 2048;
  c.computeDPWgsPerCU = cpu ? 256 : 512;
  c.targetTimeUs = DEFAULT_TARGET_TIME_US;
  c.kernelLatencyIters = 2000;
  return c;
}

namespace clpeak {
namespace {
std::atomic<bool> cancelFlag{false};
bool verboseFlag = false;
}  // namespace
void requestCancel() { cancelFlag.store(true, std::memory_order_relaxed); }
bool cancelRequested() { return cancelFlag.load(std::memory_order_relaxed); }
void resetCancel() { cancelFlag.store(false, std::memory_order_relaxed); }
bool verboseEnabled() { return verboseFlag; }
void setVerbose(bool on) { verboseFlag = on; }
}  // namespace clpeak

void Peak::applyOptions(const CliOptions &opts) {
  forceIters = opts.forceIters;
  specifiedIters = opts.iters;
  warmupCount = opts.warmupCount;
  targetTimeUs = opts.targetTimeUs;
  enabledTests = opts.enabledTests;
  enabledCategories = opts.enabledCategories;
  clpeak::setVerbose(opts.verbose);
}
