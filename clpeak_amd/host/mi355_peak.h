// The MI355X backend behind clpeak's Peak interface.
//
// Takes the place of the reference's RocmPeak (include/rocm/rocm_peak.h:119-169,
// src/rocm/rocm_peak.cpp:117-229): same backend name ("ROCm"), same device properties, same
// test tags / metric names / units in the same order, the same degrade-to-a-skip-row error
// handling -- but every measured row runs a hand-written gfx950 kernel on seeded inputs
// through the C ABI in include/clpeak_mi355.h, never HIP directly.
#pragma once
#include <functional>
#include <vector>
#include "device_api.h"
#include "inventory.h"
#include "peak.h"

class Mi355Peak : public Peak {
 public:
  std::vector<int> deviceIndices;   // empty = run every device

  explicit Mi355Peak(const Mi355Api &api = mi355_api());
  void applyOptions(const CliOptions &opts) override;
  int runAll() override;

  // What the front ends call for --list-devices and the backend catalog
  // (RocmPeak::enumerate / printInventory, src/rocm/rocm_peak.cpp:231-278).
  static BackendInventory enumerate(const Mi355Api &api = mi355_api());
  static void printInventory(const BackendInventory &inv, std::ostream &os);

  // Shapes of the seeded workloads.  Defaults are the configured ones; tests shrink them.
  struct Workload {
    uint64_t seed = 0x5EEDC1BEA4D355ull;
    uint64_t madItems = 1ull << 20;       // work-items of the MAD tests
    uint32_t madSteps = 4096;             // dependent steps per accumulator
    uint64_t bwFloats = 1ull << 30;       // 4 GiB bandwidth buffer
    uint32_t bwBlocksPerCU = 1;           // 256-thread workgroups per CU
    uint32_t mfmaWavesPerCU = 8;          // 2048 waves on 256 CUs
    uint32_t mfmaIters = 4096;
    uint32_t gemmDim = 8192;
    uint32_t latencyLaunches = 10000;
    uint64_t ldsThreads = 0;              // 0: the reference's rule, max(32M, CUs * 2048 * 256)
    uint64_t transferBytes = 1ull << 29;  // pinned staging buffer of the transfer test
    // The matrix rows on the constants the reference's kernels and GEMM tests run on instead of seeded
    // operands (--reference-operands): like for like with the reference's readings.
    bool referenceOperands = false;
  } workload;

 private:
  const Mi355Api &api_;
  mi355_dev *dev_ = nullptr;
  mi355_props_t props_{};
  logger::DeviceScope *device_ = nullptr;

  // RocmPeak::runKernel (src/rocm/rocm_peak.cpp:51-115): warm-ups, one-launch probe, pickIters,
  // timed batch between two events; microseconds per launch, or -1 on any failure.
  float runKernel(const std::function<int()> &launch, unsigned targetTimeUs, unsigned forcedIters);

  struct Buffer;   // RAII device allocation
  double heldClockMhz(const void *clocks);
  void runDevice(int ordinal, logger::BackendScope &backend);
  void runComputeMad(const struct MadTest &t);
  void runUnsupportedMatrixRows(Category phase, bool wmma);
  void runMfma(Category phase);
  void runSparseMfma(Category phase);
  void runGemmRow(logger::TestScope &test, const char *metric, const char *note, size_t elemBytes, size_t outBytes,
                  uint8_t referenceByte, double peak, const std::function<int(void *, void *)> &fill, const std::function<int(void *, void *, void *)> &launch);
  void runGemmFp();
  void runGemmFp8();
  void runGemmInt();
  void runGlobalBandwidth();
  void runLocalBandwidth();
  void runTransferBandwidth();
  void runNotBuilt(const char *tag, const char *display, std::initializer_list<std::string> metrics, const char *why,
                   ResultStatus status);
  void runKernelLatency(const benchmark_config_t &cfg);
};
