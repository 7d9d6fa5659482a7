// Enumerations every clpeak backend and front end share.  The names and the meaning of
// each value follow the reference (include/common/benchmark_enums.h:8-147,
// include/common/result_store.h:26-40); only the tests a ROCm device can run are listed.
#pragma once
#include <string>

enum class DeviceType : unsigned { Unknown = 0, Cpu = 1, Gpu = 2, Accelerator = 4 };

// One bit per selectable test (the `--<test>` flags of the CLI).
enum class Benchmark : unsigned {
  GlobalBW, LocalBW, ImageBW, TransferBW,
  ComputeHP, ComputeMP, ComputeSP, ComputeDP, ComputeBF16,
  ComputeInt, ComputeInt8DP,
  Wmma, Rocwmma, Mfma, Rocblas,
  KernelLatency,
  COUNT
};

// Run-order phases; Unknown is the "derive it from the unit" sentinel and never enabled.
enum class Category { FpCompute, IntCompute, Crypto, String, Bandwidth, Latency, Unknown };

enum class ResultStatus { Ok, Unsupported, Skipped, Error };

// Primary category of a test.  The matrix tests (Wmma, Rocwmma, Mfma, Rocblas) are listed
// under fp_compute and run a second time in the int_compute phase for their integer rows.
inline Category categoryOf(Benchmark b) {
  switch (b) {
    case Benchmark::GlobalBW: case Benchmark::LocalBW: case Benchmark::ImageBW: case Benchmark::TransferBW:
      return Category::Bandwidth;
    case Benchmark::ComputeInt: case Benchmark::ComputeInt8DP:
      return Category::IntCompute;
    case Benchmark::KernelLatency:
      return Category::Latency;
    case Benchmark::COUNT:
      return Category::Unknown;
    default:
      return Category::FpCompute;
  }
}

const char *categoryString(Category c);
const char *statusString(ResultStatus s);
Category categoryFromString(const std::string &s);
ResultStatus statusFromString(const std::string &s);
// gflops/tflops -> fp_compute, gops/tops -> int_compute, gbps -> bandwidth, us -> latency.
Category categoryFromUnit(const std::string &unit);
