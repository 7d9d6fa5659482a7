// What every clpeak backend derives from and is configured with.
//
// Peak mirrors the reference's abstract backend (include/common/peak.h:12-62,
// src/common/peak.cpp:5-14): public knobs the front end sets, bit sets that gate tests and
// categories, isAllowed / isAllowedAs, applyOptions, runAll.  The calibration helpers and the
// cancel flag are those of include/common/common.h:142-219 and src/common/common.cpp:10-45.
#pragma once
#include <bitset>
#include <cstdint>
#include <memory>
#include <string>
#include <vector>
#include "clpeak_types.h"
#include "run_log.h"

static const unsigned DEFAULT_TARGET_TIME_US = 500000;       // --max-time default: 500 ms per timed batch
static const unsigned DEFAULT_CPU_TARGET_TIME_US = 2000000;  // --max-time-cpu default
static const unsigned MAX_WG_SIZE = 256;

// Launch width the reference aims for: max(32 Mi, CUs * 2048 * 256) work-items.
inline uint64_t targetGlobalThreads(uint32_t numCUs) {
  const uint64_t scaled = (uint64_t)numCUs * 2048ull * MAX_WG_SIZE;
  return scaled > (32ull << 20) ? scaled : (32ull << 20);
}

// Iterations that make a timed batch last about target_us given one iteration's time;
// `forced` (the --iters flag) wins; 0 target means the legacy 5 s; result in [1, max_iters].
unsigned pickIters(double per_iter_us, unsigned target_us, unsigned forced, unsigned max_iters = 10000);

struct benchmark_config_t {
  uint64_t globalBWMaxSize;
  unsigned computeWgsPerCU, computeDPWgsPerCU;
  unsigned targetTimeUs;
  unsigned kernelLatencyIters;
  uint64_t transferBWMaxSize;
  static benchmark_config_t forDevice(DeviceType type);
};

namespace clpeak {
void requestCancel();     // any thread
bool cancelRequested();
void resetCancel();
bool verboseEnabled();
void setVerbose(bool on);
}  // namespace clpeak

// The subset of the CLI options a ROCm backend consumes (include/common/options.h:13-83).
struct CliOptions {
  bool skipRocm = false;
  std::vector<int> rocmDeviceIndices;   // empty = all devices
  bool forceIters = false;
  unsigned iters = 0;
  unsigned warmupCount = 2;
  unsigned targetTimeUs = DEFAULT_TARGET_TIME_US;
  unsigned targetTimeUsCpu = DEFAULT_CPU_TARGET_TIME_US;
  std::bitset<static_cast<size_t>(Benchmark::COUNT)> enabledTests;
  std::bitset<static_cast<size_t>(Category::Unknown)> enabledCategories;
  bool enableXml = false, enableJson = false, enableCsv = false;
  std::string xmlFile, jsonFile, csvFile, compareFile;
  bool listDevices = false, describe = false, verbose = false;
  CliOptions() { enabledTests.set(); enabledCategories.set(); }
};

class Peak {
 public:
  std::unique_ptr<logger> log;
  unsigned warmupCount = 2;
  unsigned specifiedIters = 0;
  unsigned targetTimeUs = DEFAULT_TARGET_TIME_US;
  bool forceIters = false;
  std::bitset<static_cast<size_t>(Benchmark::COUNT)> enabledTests;
  std::bitset<static_cast<size_t>(Category::Unknown)> enabledCategories;

  Peak() { enabledTests.set(); enabledCategories.set(); }
  virtual ~Peak() = default;

  bool isTestEnabled(Benchmark b) const { return enabledTests.test(static_cast<size_t>(b)); }
  bool isCategoryEnabled(Category c) const {
    return c != Category::Unknown && enabledCategories.test(static_cast<size_t>(c));
  }
  // A requested cancellation turns every remaining test off.
  bool isAllowed(Benchmark b) const {
    return !clpeak::cancelRequested() && isCategoryEnabled(categoryOf(b)) && isTestEnabled(b);
  }
  bool isAllowedAs(Benchmark b, Category c) const {
    return !clpeak::cancelRequested() && isCategoryEnabled(c) && isTestEnabled(b);
  }

  virtual void applyOptions(const CliOptions &opts);   // derived classes call this first
  virtual int runAll() = 0;                            // 0 = ok (also when no device is present)
};
