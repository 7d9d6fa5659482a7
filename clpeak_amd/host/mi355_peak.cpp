#include "mi355_peak.h"
#include <algorithm>
#include <cstdio>
#include <ostream>
#include "../csrc/seeded_rng.h"
#include "seeded_inputs.h"

// ---- small helpers ----------------------------------------------------------------------------
struct Mi355Peak::Buffer {
  const Mi355Api &api;
  mi355_dev *dev;
  void *ptr = nullptr;
  Buffer(const Mi355Api &a, mi355_dev *d, size_t bytes) : api(a), dev(d) {
    if (api.alloc(dev, bytes, &ptr) != MI355_OK) ptr = nullptr;
  }
  ~Buffer() { if (ptr) api.free(dev, ptr); }
  Buffer(const Buffer &) = delete;
  Buffer &operator=(const Buffer &) = delete;
  explicit operator bool() const { return ptr != nullptr; }
  bool upload(const std::vector<uint8_t> &host) { return ptr && api.upload(dev, ptr, host.data(), host.size()) == MI355_OK; }
};

// What the width of a reading means, per test family.
static const char *chainWidthNote(int width) {
  switch (width) {
    case 1: return "One value per lane at a time.";
    case 2: return "The 16 accumulators of a work-item grouped as 2-wide vectors.";
    case 4: return "The 16 accumulators of a work-item grouped as 4-wide vectors.";
    default: return "";
  }
}
static const char *loadWidthNote(int width) {
  switch (width) {
    case 1: return "One float (4 bytes) per lane and load instruction.";
    case 2: return "Two floats (8 bytes) per lane and load instruction.";
    case 4: return "Four floats (16 bytes) per lane and load instruction.";
    default: return "";
  }
}
static const char *ldsWidthNote(int width) {
  switch (width) {
    case 1: return "One float (4 bytes) per lane in every LDS store and load.";
    case 2: return "Two floats (8 bytes) per lane in every LDS store and load.";
    case 4: return "Four floats (16 bytes) per lane in every LDS store and load.";
    default: return "";
  }
}

// MI355X datasheet peaks, in the unit of the row they are compared with (dense; the 2:4 sparse
// peaks are twice the dense ones).  The reference quotes the datasheet beside its readings the
// same way (src/rocm/mfma.cpp:9-10, src/rocm/sparse_mfma.cpp:8-11).
namespace peaks {
constexpr double kVectorFp32Gflops = 157300.0, kVectorFp64Gflops = 78600.0;
constexpr double kMatrixFp32 = 157.3, kMatrixFp64 = 78.6, kMatrix16 = 2500.0, kMatrix8 = 5000.0, kMatrix6and4 = 10100.0;
constexpr double kHbmGbps = 8000.0;
}  // namespace peaks

// "<note> NN.N % of the MI355X datasheet peak (<peak> <what>)[; shader clock held: NNNN MHz]."
// The note a reading carries (EmitOptions::description, include/common/logger.h:121-128) is the one
// place of the row format that takes free text, so the fraction of peak travels there.
static std::string withPeak(const std::string &note, double value, double peak, const char *what, double heldMhz = 0.0) {
  std::string out = note;
  char buf[160];
  if (peak > 0.0) {
    snprintf(buf, sizeof buf, "%s%.1f %% of the MI355X datasheet peak (%g %s)", out.empty() ? "" : " ", 100.0 * value / peak, peak, what);
    out += buf;
    if (heldMhz > 0.0) {
      snprintf(buf, sizeof buf, "; shader clock held: %.0f MHz", heldMhz);
      out += buf;
    }
    out += ".";
  }
  return out;
}

Mi355Peak::Mi355Peak(const Mi355Api &api) : api_(api) {}

void Mi355Peak::applyOptions(const CliOptions &opts) {
  Peak::applyOptions(opts);
  deviceIndices = opts.rocmDeviceIndices;
}

BackendInventory Mi355Peak::enumerate(const Mi355Api &api) {
  BackendInventory inv;
  inv.backend = "ROCm";
  int n = 0;
  if (api.device_count(&n) != MI355_OK || n == 0) return inv;
  inv.available = true;
  InventoryPlatform plat;
  plat.index = 0;
  plat.name = "ROCm/HIP";
  for (int i = 0; i < n; i++) {
    mi355_dev *d = nullptr;
    if (api.open(i, &d) != MI355_OK) continue;   // not a gfx950 part: not this backend's device
    mi355_props_t p;
    api.get_props(d, &p);
    api.close(d);
    InventoryDevice dev;
    dev.index = i;
    dev.name = p.name;
    dev.typeStr = "GPU";
    dev.driverVersion = p.driver_version;
    dev.numComputeUnits = (unsigned)p.num_cus;
    dev.maxClockMHz = (unsigned)(p.clock_khz / 1000);
    dev.globalMemBytes = p.total_mem;
    dev.hasFp16 = dev.hasFp64 = true;
    plat.devices.push_back(dev);
  }
  inv.platforms.push_back(plat);
  return inv;
}

void Mi355Peak::printInventory(const BackendInventory &inv, std::ostream &os) {
  os << "\n=== ROCm backend ===\n";
  if (!inv.available) {
    os << "ROCm: runtime init failed or no devices found\n";
    return;
  }
  for (const InventoryPlatform &plat : inv.platforms)
    for (const InventoryDevice &d : plat.devices) {
      os << "  ROCm Device " << d.index << ": " << d.name;
      if (!d.typeStr.empty()) os << " [" << d.typeStr << "]";
      os << "\n";
    }
}

float Mi355Peak::runKernel(const std::function<int()> &launch, unsigned targetUs, unsigned forcedIters) {
  for (unsigned w = 0; w < warmupCount; w++)
    if (launch() != MI355_OK || api_.sync(dev_) != MI355_OK) return -1.0f;
  auto batch = [&](unsigned n) -> float {
    if (api_.timer_start(dev_) != MI355_OK) return -1.0f;
    for (unsigned i = 0; i < n; i++)
      if (launch() != MI355_OK) {
        if (clpeak::verboseEnabled()) fprintf(stderr, "launch failed: %s\n", api_.last_error(dev_));
        return -1.0f;
      }
    float us = 0.0f;
    if (api_.timer_stop(dev_, &us) != MI355_OK) return -1.0f;
    return us;
  };
  const float probe = batch(1);
  if (probe <= 0.0f) return -1.0f;
  const unsigned iters = pickIters(probe, targetUs, forcedIters);
  const float total = batch(iters);
  return total > 0.0f ? total / (float)iters : -1.0f;
}

// ---- run order ------------------------------------------------------------------------------------
int Mi355Peak::runAll() {
  int count = 0;
  if (api_.device_count(&count) != MI355_OK) {
    log->note("ROCm: runtime init failed\n");
    return -1;
  }
  if (count == 0) {
    log->note("ROCm: no devices found\n");
    return 0;
  }
  auto backend = log->beginBackend("ROCm");
  for (int i = 0; i < count; i++) {
    if (clpeak::cancelRequested()) break;
    if (!deviceIndices.empty() && std::find(deviceIndices.begin(), deviceIndices.end(), i) == deviceIndices.end()) continue;
    runDevice(i, backend);
  }
  return 0;
}

struct MadTest {
  Benchmark bench;
  const char *tag, *display, *unit, *description;
  int kind, elemBytes;
  int opsPerStep;   // operations one accumulator step counts for
  double peak;      // datasheet peak in the row's unit, 0 where the datasheet has no line
  const char *peakWhat;
  struct Variant { const char *metric; int width; const char *note; } variants[4];
};

void Mi355Peak::runDevice(int ordinal, logger::BackendScope &backend) {
  if (api_.open(ordinal, &dev_) != MI355_OK) {
    log->note("ROCm: failed to init device " + std::to_string(ordinal) + ": " + api_.last_error(nullptr) + "\n");
    dev_ = nullptr;
    return;
  }
  api_.get_props(dev_, &props_);
  benchmark_config_t cfg = benchmark_config_t::forDevice(DeviceType::Gpu);
  cfg.targetTimeUs = targetTimeUs;
  cfg.kernelLatencyIters = forceIters ? specifiedIters : workload.latencyLaunches;

  auto device = backend.beginDevice({props_.name, "", props_.driver_version,
                                     {{"Arch", props_.arch},
                                      {"HIP", props_.runtime_version},
                                      {"CUs", std::to_string(props_.num_cus)},
                                      {"Wave", std::to_string(props_.wave_size)},
                                      {"VRAM", std::to_string(props_.total_mem / (1024 * 1024)) + " MB"}},
                                     -1, ordinal});
  device_ = &device;

  static const MadTest sp = {Benchmark::ComputeSP, "single_precision_compute", "Single-precision compute", "gflops",
      "Vector-ALU rate on 32-bit floats: 2^20 work-items, each advancing 16 independent fused multiply-add chains, "
      "nothing but registers involved.", MI355_MAD_F32, 4, 2, peaks::kVectorFp32Gflops, "GFLOPS vector fp32",
      {{"float", 1, chainWidthNote(1)}, {"float2", 2, chainWidthNote(2)}, {"float4", 4, chainWidthNote(4)}, {nullptr, 0, nullptr}}};
  static const MadTest hp = {Benchmark::ComputeHP, "half_precision_compute", "Half-precision compute", "gflops",
      "The same chains in IEEE half precision; the packed form does two lanes per instruction.", MI355_MAD_F16, 2, 2, 0.0, "",
      {{"half", 1, "One scalar half-precision multiply-add per step and accumulator (the scalar instruction issues at half the rate of the packed one)."}, {"half2", 2, "Packed: two half-precision multiply-adds per lane and instruction."}, {nullptr, 0, nullptr}, {nullptr, 0, nullptr}}};
  static const MadTest dp = {Benchmark::ComputeDP, "double_precision_compute", "Double-precision compute", "gflops",
      "The same chains on 64-bit floats.", MI355_MAD_F64, 8, 2, peaks::kVectorFp64Gflops, "GFLOPS vector fp64",
      {{"double", 1, chainWidthNote(1)}, {"double2", 2, chainWidthNote(2)}, {"double4", 4, chainWidthNote(4)}, {nullptr, 0, nullptr}}};
  static const MadTest mp = {Benchmark::ComputeMP, "mixed_precision_compute", "Mixed-precision compute fp16xfp16+fp32", "gflops",
      "A 32-bit running value times a half-precision factor plus a half-precision addend, widened by the multiply-add "
      "itself; the running value passes through half precision once every 16 steps.", MI355_MAD_MP, 4, 2, 0.0, "",
      {{"mp", 1, nullptr}, {nullptr, 0, nullptr}, {nullptr, 0, nullptr}, {nullptr, 0, nullptr}}};
  static const MadTest bf = {Benchmark::ComputeBF16, "bfloat16_compute", "BF16 compute bf16xbf16+fp32", "gflops",
      "Two bfloat16 products added to a 32-bit running total per instruction; one factor is refreshed from the total "
      "once every 128 steps.", MI355_MAD_BF16, 4, 4, 0.0, "",
      {{"bf16", 1, "Counted as 4 operations per instruction (two products, two additions: a 2-element dot product); clpeak's own "
                   "row of this name counts a 2-operation multiply-add chain."}, {nullptr, 0, nullptr}, {nullptr, 0, nullptr}, {nullptr, 0, nullptr}}};
  static const MadTest i32 = {Benchmark::ComputeInt, "integer_compute", "Integer compute (32-bit IMAD)", "gops",
      "The same chains on 32-bit integers (multiply-add, wrapping).", MI355_MAD_I32, 4, 2, 0.0, "",
      {{"int", 1, chainWidthNote(1)}, {"int2", 2, chainWidthNote(2)}, {"int4", 4, chainWidthNote(4)}, {nullptr, 0, nullptr}}};
  static const MadTest i8 = {Benchmark::ComputeInt8DP, "integer_compute_int8_dp", "INT8 dot-product compute (DP4a)", "gops",
      "Four 8-bit multiply-adds per instruction, each result fed back into the next operand.", MI355_MAD_I8DP, 4, 8, 0.0, "",
      {{"int8_dp", 1, "One dependent chain."}, {"int8_dp2", 2, "Two independent chains."},
       {"int8_dp4", 4, "Four independent chains."}, {"int8_dp8", 8, "Eight independent chains."}}};

  // fp phase
  if (isAllowed(Benchmark::ComputeSP)) runComputeMad(sp);
  if (isAllowed(Benchmark::ComputeHP)) runComputeMad(hp);
  if (isAllowed(Benchmark::ComputeDP)) runComputeMad(dp);
  if (isAllowed(Benchmark::ComputeMP)) runComputeMad(mp);
  if (isAllowed(Benchmark::ComputeBF16)) runComputeMad(bf);
  if (isAllowedAs(Benchmark::Wmma, Category::FpCompute)) runUnsupportedMatrixRows(Category::FpCompute, true);
  if (isAllowedAs(Benchmark::Rocwmma, Category::FpCompute)) runUnsupportedMatrixRows(Category::FpCompute, false);
  if (isAllowedAs(Benchmark::Mfma, Category::FpCompute)) runMfma(Category::FpCompute);
  if (isAllowedAs(Benchmark::Mfma, Category::FpCompute)) runSparseMfma(Category::FpCompute);
  if (isAllowedAs(Benchmark::Rocblas, Category::FpCompute)) runGemmFp();
  if (isAllowedAs(Benchmark::Rocblas, Category::FpCompute)) runGemmFp8();
  // int phase
  if (isAllowed(Benchmark::ComputeInt)) runComputeMad(i32);
  if (isAllowed(Benchmark::ComputeInt8DP)) runComputeMad(i8);
  if (isAllowedAs(Benchmark::Wmma, Category::IntCompute)) runUnsupportedMatrixRows(Category::IntCompute, true);
  if (isAllowedAs(Benchmark::Rocwmma, Category::IntCompute)) runUnsupportedMatrixRows(Category::IntCompute, false);
  if (isAllowedAs(Benchmark::Mfma, Category::IntCompute)) runMfma(Category::IntCompute);
  if (isAllowedAs(Benchmark::Mfma, Category::IntCompute)) runSparseMfma(Category::IntCompute);
  if (isAllowedAs(Benchmark::Rocblas, Category::IntCompute)) runGemmInt();
  // bandwidth and latency
  if (isAllowed(Benchmark::GlobalBW)) runGlobalBandwidth();
  if (isAllowed(Benchmark::LocalBW)) runLocalBandwidth();
  if (isAllowed(Benchmark::ImageBW))
    runNotBuilt("image_memory_bandwidth", "Image memory bandwidth", {"float4"},
                "Device has no image/texture support", ResultStatus::Unsupported);
  if (isAllowed(Benchmark::TransferBW)) runTransferBandwidth();
  if (isAllowed(Benchmark::KernelLatency)) runKernelLatency(cfg);

  device_ = nullptr;
  device.end();
  api_.close(dev_);
  dev_ = nullptr;
}

// ---- vector MAD -----------------------------------------------------------------------------------------
void Mi355Peak::runComputeMad(const MadTest &t) {
  auto test = device_->beginTest({t.tag, t.display, t.unit, Category::Unknown, t.description});
  Buffer out(api_, dev_, workload.madItems * (size_t)t.elemBytes);
  for (const auto &v : t.variants) {
    if (!v.metric) break;
    const std::string note = v.note ? v.note : "";
    if (!out) {
      test.skip(v.metric, ResultStatus::Error, "Failed to allocate output buffer", note);
      continue;
    }
    const float us = runKernel(
        [&] { return api_.compute_mad(dev_, t.kind, v.width, workload.seed, workload.madItems, workload.madSteps, out.ptr, 256); },
        targetTimeUs, forceIters ? specifiedIters : 0);
    if (us <= 0.0f) {
      test.skip(v.metric, ResultStatus::Error, "kernel launch failed", note);
      continue;
    }
    // 16 accumulators per item (or `width` chains for the dot-product test)
    const double chains = t.kind == MI355_MAD_I8DP ? (double)v.width : 16.0;
    const double ops = (double)workload.madItems * chains * (double)workload.madSteps * (double)t.opsPerStep;
    const double giga = ops * 1e6 / us / 1e9;
    test.emit(v.metric, (float)giga, {false, withPeak(note, giga, t.peak, t.peakWhat)});
  }
}

// ---- rows that exist only on other AMD families ----------------------------------------------------------------
void Mi355Peak::runUnsupportedMatrixRows(Category phase, bool wmma) {
  struct Row { const char *tag, *display, *unit; };
  static const Row wmmaFp[] = {{"wmma_fp16", "WMMA fp16xfp16+fp32 16x16x16", "tflops"},
                               {"wmma_bf16", "WMMA bf16xbf16+fp32 16x16x16", "tflops"},
                               {"wmma_fp8_e4m3", "WMMA fp8(E4M3)xfp8(E4M3)+fp32 16x16x16", "tflops"},
                               {"wmma_fp8_e5m2", "WMMA fp8(E5M2)xfp8(E5M2)+fp32 16x16x16", "tflops"}};
  static const Row wmmaInt[] = {{"wmma_int8", "WMMA int8xint8+int32 16x16x16", "tops"}};
  const bool isInt = phase == Category::IntCompute;
  if (wmma) {
    const Row *rows = isInt ? wmmaInt : wmmaFp;
    const size_t n = isInt ? 1 : 4;
    for (size_t i = 0; i < n; i++) {
      auto test = device_->beginTest({rows[i].tag, rows[i].display, rows[i].unit, Category::Unknown, ""});
      test.skip(rows[i].tag, ResultStatus::Unsupported,
                "WMMA is an RDNA3+/RDNA4 (gfx11/gfx12) matrix-core feature; absent on this architecture");
    }
  } else {
    auto test = isInt ? device_->beginTest({"rocwmma-int", "rocWMMA int8xint8+int32 16x16x16", "tops", Category::Unknown, ""})
                      : device_->beginTest({"rocwmma-fp", "rocWMMA fp16xfp16+fp32 16x16x16", "tflops", Category::Unknown, ""});
    test.skip(isInt ? "rocwmma_int8" : "rocwmma_fp16", ResultStatus::Unsupported,
              "rocWMMA does not support this GPU architecture");
  }
}

// ---- dense MFMA ----------------------------------------------------------------------------------------------
// The matrix kernels leave two counters of their timed loop behind (shader cycles, ticks of the
// constant 100 MHz clock): the shader clock the part held under the load, in MHz; 0 when unknown.
double Mi355Peak::heldClockMhz(const void *clocks) {
  uint64_t c[2] = {0, 0};
  if (!clocks || api_.download(dev_, c, clocks, sizeof c) != MI355_OK || c[1] == 0) return 0.0;
  return (double)c[0] / (double)c[1] * 100.0;
}

static const char *operandsNote(bool reference) {
  return reference ? "Operands: the constants clpeak's own kernels multiply; one operand set per wave."
                   : "Operands: seeded random values; one operand set per wave, four accumulator chains.";
}

namespace {
struct MfmaRow {
  const char *tag, *display, *unit, *description;
  int kind, M, N, K;
  OperandFormat fmt;
  double sigma;
  bool scaled;
  double peak;   // dense datasheet peak of the operand type, TFLOPS / TOPS
};
const MfmaRow kMfmaFp[] = {
    {"mfma_fp16", "MFMA fp16xfp16+fp32 16x16x32", "tflops", "Matrix-core rate on half-precision inputs with a 32-bit accumulator.",
     MI355_MFMA_F16_16x16x32, 16, 16, 32, OperandFormat::F16, 0.01, false, peaks::kMatrix16},
    {"mfma_fp16_32x32x16", "MFMA fp16xfp16+fp32 32x32x16", "tflops", "The same on the 32x32 tile shape.",
     MI355_MFMA_F16_32x32x16, 32, 32, 16, OperandFormat::F16, 0.01, false, peaks::kMatrix16},
    {"mfma_bf16", "MFMA bf16xbf16+fp32 16x16x32", "tflops", "Matrix-core rate on bfloat16 inputs with a 32-bit accumulator.",
     MI355_MFMA_BF16_16x16x32, 16, 16, 32, OperandFormat::BF16, 0.01, false, peaks::kMatrix16},
    {"mfma_bf16_32x32x16", "MFMA bf16xbf16+fp32 32x32x16", "tflops", "The same on the 32x32 tile shape.",
     MI355_MFMA_BF16_32x32x16, 32, 32, 16, OperandFormat::BF16, 0.01, false, peaks::kMatrix16},
    {"mfma_fp8", "MFMA fp8xfp8+fp32 16x16x128", "tflops", "Matrix-core rate on OCP fp8 (E4M3) inputs.",
     MI355_MFMA_FP8_16x16x128, 16, 16, 128, OperandFormat::E4M3, 1.0, false, peaks::kMatrix8},
    {"mfma_bf8", "MFMA bf8xbf8+fp32 16x16x128", "tflops", "Matrix-core rate on OCP fp8 (E5M2) inputs.",
     MI355_MFMA_BF8_16x16x128, 16, 16, 128, OperandFormat::E5M2, 1.0, false, peaks::kMatrix8},
    {"mfma_mxfp6_e2m3", "MFMA mxfp6(e2m3)+fp32 16x16x128", "tflops", "6-bit MX inputs with one E8M0 scale per 32 elements.",
     MI355_MFMA_MXFP6_E2M3, 16, 16, 128, OperandFormat::E2M3, 1.0, true, peaks::kMatrix6and4},
    {"mfma_mxfp6_e3m2", "MFMA mxfp6(e3m2)+fp32 16x16x128", "tflops", "6-bit MX inputs, the wider-range variant.",
     MI355_MFMA_MXFP6_E3M2, 16, 16, 128, OperandFormat::E3M2, 1.0, true, peaks::kMatrix6and4},
    {"mfma_mxfp4", "MFMA mxfp4(e2m1)+fp32 16x16x128", "tflops", "4-bit MX inputs with one E8M0 scale per 32 elements.",
     MI355_MFMA_MXFP4_E2M1, 16, 16, 128, OperandFormat::E2M1, 1.0, true, peaks::kMatrix6and4},
};
const MfmaRow kMfmaInt[] = {
    {"mfma_int8", "MFMA int8xint8+int32 16x16x64", "tops", "Matrix-core rate on 8-bit integers with a 32-bit accumulator.",
     MI355_MFMA_I8_16x16x64, 16, 16, 64, OperandFormat::I8, 0.0, false, peaks::kMatrix8},
};
struct SparseRow {
  const char *tag, *display, *unit, *description;
  int kind, K;
  OperandFormat fmt;
  double sigma;
  double peak;   // 2:4 sparse datasheet peak (twice the dense one), TFLOPS / TOPS
};
const SparseRow kSparseFp[] = {
    {"smfmac_fp16", "Sparse MFMA fp16 2:4 16x16x64 (TFLOPS)", "tflops", "2:4 structured-sparse matrix-core rate, half-precision inputs.",
     MI355_SMFMAC_F16_16x16x64, 64, OperandFormat::F16, 0.01, 2 * peaks::kMatrix16},
    {"smfmac_bf16", "Sparse MFMA bf16 2:4 16x16x64 (TFLOPS)", "tflops", "2:4 structured-sparse matrix-core rate, bfloat16 inputs.",
     MI355_SMFMAC_BF16_16x16x64, 64, OperandFormat::BF16, 0.01, 2 * peaks::kMatrix16},
    {"smfmac_fp8", "Sparse MFMA fp8 2:4 16x16x128 (TFLOPS)", "tflops", "2:4 structured-sparse matrix-core rate, fp8 (E4M3) inputs.",
     MI355_SMFMAC_FP8_16x16x128, 128, OperandFormat::E4M3, 1.0, 2 * peaks::kMatrix8},
    {"smfmac_bf8", "Sparse MFMA bf8 2:4 16x16x128 (TFLOPS)", "tflops", "2:4 structured-sparse matrix-core rate, fp8 (E5M2) inputs.",
     MI355_SMFMAC_BF8_16x16x128, 128, OperandFormat::E5M2, 1.0, 2 * peaks::kMatrix8},
};
const SparseRow kSparseInt[] = {
    {"smfmac_int8", "Sparse MFMA int8 2:4 16x16x128 (TOPS)", "tops", "2:4 structured-sparse matrix-core rate, 8-bit integers.",
     MI355_SMFMAC_I8_16x16x128, 128, OperandFormat::I8, 0.0, 2 * peaks::kMatrix8},
};
}  // namespace

void Mi355Peak::runMfma(Category phase) {
  const bool isInt = phase == Category::IntCompute;
  const MfmaRow *rows = isInt ? kMfmaInt : kMfmaFp;
  const size_t n = isInt ? sizeof(kMfmaInt) / sizeof(kMfmaInt[0]) : sizeof(kMfmaFp) / sizeof(kMfmaFp[0]);
  const uint32_t waves = (uint32_t)props_.num_cus * workload.mfmaWavesPerCU;
  const uint64_t units = (uint64_t)waves * 4;
  for (size_t r = 0; r < n; r++) {
    const MfmaRow &m = rows[r];
    auto test = device_->beginTest({m.tag, m.display, m.unit, Category::Unknown, m.description});
    const bool ref = workload.referenceOperands;
    const std::vector<uint8_t> A = ref ? reference_operand(m.fmt, units * m.M * m.K)
                                       : seeded_operand(m.fmt, m.sigma, workload.seed, MI355_STREAM_MFMA_A, units * m.M * m.K);
    const std::vector<uint8_t> B = ref ? reference_operand(m.fmt, units * m.N * m.K)
                                       : seeded_operand(m.fmt, m.sigma, workload.seed, MI355_STREAM_MFMA_B, units * m.N * m.K);
    Buffer dA(api_, dev_, A.size()), dB(api_, dev_, B.size()), out(api_, dev_, units * m.M * m.N * 4);
    Buffer sA(api_, dev_, m.scaled ? units * m.M * (m.K / 32) : 16), sB(api_, dev_, m.scaled ? units * m.N * (m.K / 32) : 16);
    Buffer clk(api_, dev_, 16);
    bool ok = dA && dB && out && sA && sB && clk && dA.upload(A) && dB.upload(B);
    if (ok && m.scaled && ref)
      ok = sA.upload(std::vector<uint8_t>(units * m.M * (m.K / 32), kReferenceScale)) &&
           sB.upload(std::vector<uint8_t>(units * m.N * (m.K / 32), kReferenceScale));
    else if (ok && m.scaled)
      ok = sA.upload(seeded_e8m0(workload.seed, MI355_STREAM_SCALE_A, units * m.M * (m.K / 32))) &&
           sB.upload(seeded_e8m0(workload.seed, MI355_STREAM_SCALE_B, units * m.N * (m.K / 32)));
    if (!ok) {
      test.skip(m.tag, ResultStatus::Error, "Failed to allocate or upload operand buffers");
      continue;
    }
    const float us = runKernel(
        [&] {
          return api_.mfma_dense(dev_, m.kind | MI355_MFMA_ONE_OPERAND_SET, dA.ptr, dB.ptr, m.scaled ? (const uint8_t *)sA.ptr : nullptr,
                                 m.scaled ? (const uint8_t *)sB.ptr : nullptr, out.ptr, waves, workload.mfmaIters, (uint64_t *)clk.ptr);
        },
        targetTimeUs, forceIters ? specifiedIters : 0);
    if (us <= 0.0f) {
      test.skip(m.tag, ResultStatus::Error, "kernel launch failed");
      continue;
    }
    // every wave issues 4 * iters instructions of 2*M*N*K operations
    const double ops = (double)units * workload.mfmaIters * 2.0 * m.M * m.N * m.K;
    const double tera = ops * 1e6 / us / 1e12;
    test.emit(m.tag, (float)tera, {false, withPeak(operandsNote(workload.referenceOperands), tera, m.peak, isInt ? "TOPS dense" : "TFLOPS dense", heldClockMhz(clk.ptr))});
  }
}

void Mi355Peak::runSparseMfma(Category phase) {
  const bool isInt = phase == Category::IntCompute;
  const SparseRow *rows = isInt ? kSparseInt : kSparseFp;
  const size_t n = isInt ? sizeof(kSparseInt) / sizeof(kSparseInt[0]) : sizeof(kSparseFp) / sizeof(kSparseFp[0]);
  const uint32_t waves = (uint32_t)props_.num_cus * workload.mfmaWavesPerCU;
  const uint64_t units = (uint64_t)waves * 4;
  for (size_t r = 0; r < n; r++) {
    const SparseRow &m = rows[r];
    auto test = device_->beginTest({m.tag, m.display, m.unit, Category::Unknown, m.description});
    const bool ref = workload.referenceOperands;
    const std::vector<uint8_t> Ac = ref ? reference_operand(m.fmt, units * 16 * (m.K / 2))
                                        : seeded_operand(m.fmt, m.sigma, workload.seed, MI355_STREAM_MFMA_A, units * 16 * (m.K / 2));
    const std::vector<uint8_t> B = ref ? reference_operand(m.fmt, units * 16 * m.K)
                                       : seeded_operand(m.fmt, m.sigma, workload.seed, MI355_STREAM_MFMA_B, units * 16 * m.K);
    const std::vector<uint8_t> meta = ref ? std::vector<uint8_t>(units * 16 * (m.K / 4), kReferenceSparseMeta)
                                          : seeded_sparse_meta(workload.seed, MI355_STREAM_SPARSE, units * 16 * (m.K / 4));
    Buffer dA(api_, dev_, Ac.size()), dB(api_, dev_, B.size()), dM(api_, dev_, meta.size()), out(api_, dev_, units * 256 * 4);
    Buffer clk(api_, dev_, 16);
    if (!(dA && dB && dM && out && clk && dA.upload(Ac) && dB.upload(B) && dM.upload(meta))) {
      test.skip(m.tag, ResultStatus::Error, "Failed to allocate or upload operand buffers");
      continue;
    }
    const float us = runKernel(
        [&] { return api_.smfmac(dev_, m.kind | MI355_MFMA_ONE_OPERAND_SET, dA.ptr, (const uint8_t *)dM.ptr, dB.ptr, out.ptr, waves, workload.mfmaIters, (uint64_t *)clk.ptr); },
        targetTimeUs, forceIters ? specifiedIters : 0);
    if (us <= 0.0f) {
      test.skip(m.tag, ResultStatus::Error, "kernel launch failed");
      continue;
    }
    // counted with the dense-equivalent K, as the datasheet's sparse column is
    const double ops = (double)units * workload.mfmaIters * 2.0 * 16 * 16 * m.K;
    const double tera = ops * 1e6 / us / 1e12;
    test.emit(m.tag, (float)tera, {false, withPeak(operandsNote(workload.referenceOperands), tera, m.peak, isInt ? "TOPS 2:4 sparse" : "TFLOPS 2:4 sparse", heldClockMhz(clk.ptr))});
  }
}

// ---- GEMM (the slots of the vendor-library tests) ------------------------------------------------------------------
// One GEMM row: fill the operands on the device, time the launch like any kernel, emit 2*D^3 / time.
// With reference operands every byte of A and B is `referenceByte`, as the reference's tests set them
// (0x3f: src/rocm/rocblas.cpp:211-212; 0x38: src/rocm/hipblaslt_gemm.cpp:272-273).
void Mi355Peak::runGemmRow(logger::TestScope &test, const char *metric, const char *note, size_t elemBytes, size_t outBytes,
                           uint8_t referenceByte, double peak, const std::function<int(void *, void *)> &fill,
                           const std::function<int(void *, void *, void *)> &launch) {
  const uint32_t D = workload.gemmDim;
  const size_t abBytes = (size_t)D * D * elemBytes;
  Buffer A(api_, dev_, abBytes), B(api_, dev_, abBytes), C(api_, dev_, (size_t)D * D * outBytes);
  auto constantFill = [&](void *a, void *b) {
    const int rc = api_.fill_bytes(dev_, (uint8_t *)a, abBytes, workload.seed, MI355_STREAM_GEMM_A, referenceByte, 1);
    return rc != MI355_OK ? rc : api_.fill_bytes(dev_, (uint8_t *)b, abBytes, workload.seed, MI355_STREAM_GEMM_B, referenceByte, 1);
  };
  if (!(A && B && C) || (workload.referenceOperands ? constantFill(A.ptr, B.ptr) : fill(A.ptr, B.ptr)) != MI355_OK) {
    test.skip(metric, ResultStatus::Error, "Failed to allocate or fill GEMM buffers", note);
    return;
  }
  const float us = runKernel([&] { return launch(A.ptr, B.ptr, C.ptr); }, targetTimeUs, forceIters ? specifiedIters : 0);
  if (us <= 0.0f) test.skip(metric, ResultStatus::Error, "kernel launch failed", note);
  else {
    const double tera = 2.0 * D * D * D * 1e6 / us / 1e12;
    const char *what = peak == peaks::kMatrixFp32 ? "TFLOPS matrix fp32" : peak == peaks::kMatrixFp64 ? "TFLOPS matrix fp64"
                       : std::string(metric) == "int8" ? "TOPS dense" : "TFLOPS dense";
    test.emit(metric, (float)tera, {false, withPeak(note, tera, peak, what)});
  }
}

void Mi355Peak::runGemmFp() {
  auto test = device_->beginTest({"rocblas-fp", "rocBLAS GEMM peak", "tflops", Category::Unknown,
                                  "Square GEMM on this backend's hand-written MFMA kernels (LDS-tiled, K contiguous in both "
                                  "operands), not a vendor library."});
  const uint32_t D = workload.gemmDim;
  const uint64_t n = (uint64_t)D * D;
  runGemmRow(test, "fp32", "fp32 inputs, accumulation and output, on the fp32 matrix instruction; A row-major, B column-major.", 4, 4, 0x3f, peaks::kMatrixFp32,
             [&](void *a, void *b) {
               const int rc = api_.fill_f32(dev_, (float *)a, n, workload.seed, MI355_STREAM_GEMM_A, MI355_DIST_UPM1);
               return rc != MI355_OK ? rc : api_.fill_f32(dev_, (float *)b, n, workload.seed, MI355_STREAM_GEMM_B, MI355_DIST_UPM1);
             },
             [&](void *a, void *b, void *c) { return api_.gemm_f32(dev_, (const float *)a, (const float *)b, (float *)c, D, D, D); });
  runGemmRow(test, "fp64", "fp64 inputs, accumulation and output, on the fp64 matrix instruction; A row-major, B column-major.", 8, 8, 0x3f, peaks::kMatrixFp64,
             [&](void *a, void *b) {
               const int rc = api_.fill_f64(dev_, (double *)a, n, workload.seed, MI355_STREAM_GEMM_A, MI355_DIST_UPM1);
               return rc != MI355_OK ? rc : api_.fill_f64(dev_, (double *)b, n, workload.seed, MI355_STREAM_GEMM_B, MI355_DIST_UPM1);
             },
             [&](void *a, void *b, void *c) { return api_.gemm_f64(dev_, (const double *)a, (const double *)b, (double *)c, D, D, D); });
  runGemmRow(test, "fp16", "IEEE half inputs, fp32 accumulation, half output; A row-major, B column-major.", 2, 2, 0x3f, peaks::kMatrix16,
             [&](void *a, void *b) {
               const int rc = api_.fill_f16(dev_, (uint16_t *)a, n, workload.seed, MI355_STREAM_GEMM_A, MI355_DIST_UPM1);
               return rc != MI355_OK ? rc : api_.fill_f16(dev_, (uint16_t *)b, n, workload.seed, MI355_STREAM_GEMM_B, MI355_DIST_UPM1);
             },
             [&](void *a, void *b, void *c) { return api_.gemm_f16(dev_, (const uint16_t *)a, (const uint16_t *)b, (uint16_t *)c, D, D, D); });
  runGemmRow(test, "bf16", "bf16 inputs, fp32 accumulation, bf16 output; A row-major, B column-major.", 2, 2, 0x3f, peaks::kMatrix16,
             [&](void *a, void *b) {
               const int rc = api_.fill_bf16(dev_, (uint16_t *)a, n, workload.seed, MI355_STREAM_GEMM_A, MI355_DIST_UPM1);
               return rc != MI355_OK ? rc : api_.fill_bf16(dev_, (uint16_t *)b, n, workload.seed, MI355_STREAM_GEMM_B, MI355_DIST_UPM1);
             },
             [&](void *a, void *b, void *c) { return api_.gemm_bf16(dev_, (const uint16_t *)a, (const uint16_t *)b, (uint16_t *)c, D, D, D); });
}

void Mi355Peak::runGemmFp8() {
  auto test = device_->beginTest({"hipblaslt-fp8", "hipBLASLt FP8 GEMM peak", "tflops", Category::Unknown,
                                  "Square FP8 / FP4 GEMM with per-tensor or per-block scales: this backend's hand-written MFMA kernels, "
                                  "not a vendor library."});
  const uint32_t D = workload.gemmDim;
  const uint64_t n = (uint64_t)D * D;
  const float s43 = 448.0f, s52 = 57344.0f;   // uniform [-1,1) stretched over the range of the format
  runGemmRow(test, "fp8_e4m3", "OCP e4m3 inputs, per-tensor fp32 scales, fp32 accumulation, bf16 output.", 1, 2, 0x38, peaks::kMatrix8,
             [&](void *a, void *b) {
               const int rc = api_.fill_fp8_e4m3(dev_, (uint8_t *)a, n, workload.seed, MI355_STREAM_GEMM_A, MI355_DIST_UPM1, s43);
               return rc != MI355_OK ? rc : api_.fill_fp8_e4m3(dev_, (uint8_t *)b, n, workload.seed, MI355_STREAM_GEMM_B, MI355_DIST_UPM1, s43);
             },
             [&](void *a, void *b, void *c) {
               return api_.gemm_fp8_e4m3(dev_, (const uint8_t *)a, (const uint8_t *)b, (uint16_t *)c, D, D, D, 1.0f / s43, 1.0f / s43);
             });
  runGemmRow(test, "fp8_e5m2", "An OCP e5m2 A against an e4m3 B, per-tensor fp32 scales, fp32 accumulation, bf16 output.", 1, 2, 0x38, peaks::kMatrix8,
             [&](void *a, void *b) {
               const int rc = api_.fill_fp8_e5m2(dev_, (uint8_t *)a, n, workload.seed, MI355_STREAM_GEMM_A, MI355_DIST_UPM1, s52);
               return rc != MI355_OK ? rc : api_.fill_fp8_e4m3(dev_, (uint8_t *)b, n, workload.seed, MI355_STREAM_GEMM_B, MI355_DIST_UPM1, s43);
             },
             [&](void *a, void *b, void *c) {
               return api_.gemm_fp8_e5m2(dev_, (const uint8_t *)a, (const uint8_t *)b, (uint16_t *)c, D, D, D, 1.0f / s52, 1.0f / s43);
             });
  // block-scaled FP4: two e2m1 codes per byte, one E8M0 scale per 32 elements (2^-4 .. 2^4)
  const char *mxNote = "OCP MXFP4: e2m1 inputs with one E8M0 scale per 32 elements along K (laid out for the kernel once, before the timed launches), fp32 accumulation, bf16 output.";
  {
    // reference operands: bytes of 0x38 under scales of 0x7f (src/rocm/hipblaslt_gemm.cpp:272-273, 417-418)
    const bool ref = workload.referenceOperands;
    Buffer A(api_, dev_, (size_t)n / 2), B(api_, dev_, (size_t)n / 2), SA(api_, dev_, (size_t)n / 32), SB(api_, dev_, (size_t)n / 32),
        C(api_, dev_, (size_t)n * 2);
    const bool ok = A && B && SA && SB && C && D % 256 == 0 &&
                    api_.fill_bytes(dev_, (uint8_t *)A.ptr, n / 2, workload.seed, MI355_STREAM_GEMM_A, ref ? 0x38 : 0, ref ? 1 : 256) == MI355_OK &&
                    api_.fill_bytes(dev_, (uint8_t *)B.ptr, n / 2, workload.seed, MI355_STREAM_GEMM_B, ref ? 0x38 : 0, ref ? 1 : 256) == MI355_OK &&
                    api_.fill_bytes(dev_, (uint8_t *)SA.ptr, n / 32, workload.seed, MI355_STREAM_SCALE_A, ref ? 0x7f : 123, ref ? 1 : 9) == MI355_OK &&
                    api_.fill_bytes(dev_, (uint8_t *)SB.ptr, n / 32, workload.seed, MI355_STREAM_SCALE_B, ref ? 0x7f : 123, ref ? 1 : 9) == MI355_OK;
    // The scales of both operands stay what they are over the timed launches, as in the reference's loop (one set of
    // scale pointers for every product, src/rocm/hipblaslt_gemm.cpp:438-449, 487-505): laid out once for the kernel,
    // outside the timed batch.
    Buffer prepared(api_, dev_, (size_t)n / 32 * 2);
    const bool laidOut = ok && prepared &&
                         api_.gemm_mxfp4_prepare_scales(dev_, (const uint8_t *)SA.ptr, (const uint8_t *)SB.ptr, D, D, D, (uint8_t *)prepared.ptr) == MI355_OK;
    float us = -1.0f;
    if (laidOut)
      us = runKernel([&] { return api_.gemm_mxfp4_prepared(dev_, (const uint8_t *)A.ptr, (const uint8_t *)B.ptr, (const uint8_t *)prepared.ptr,
                                                            (uint16_t *)C.ptr, D, D, D); },
                     targetTimeUs, forceIters ? specifiedIters : 0);
    if (!laidOut) test.skip("mxf4_e2m1", ResultStatus::Error, "Failed to allocate or fill GEMM buffers", mxNote);
    else if (us <= 0.0f) test.skip("mxf4_e2m1", ResultStatus::Error, "kernel launch failed", mxNote);
    else {
      const double tera = 2.0 * D * D * D * 1e6 / us / 1e12;
      test.emit("mxf4_e2m1", (float)tera, {false, withPeak(mxNote, tera, peaks::kMatrix6and4, "TFLOPS dense")});
    }
  }
}

void Mi355Peak::runGemmInt() {
  auto test = device_->beginTest({"rocblas-int", "rocBLAS GEMM peak", "tops", Category::Unknown,
                                  "Square int8 GEMM with int32 accumulation and output: this backend's hand-written MFMA "
                                  "kernel, not a vendor library."});
  const uint32_t D = workload.gemmDim;
  const uint64_t n = (uint64_t)D * D;
  runGemmRow(test, "int8", "8-bit integers in [-8, 7], 32-bit totals; A row-major, B column-major.", 1, 4, 0x3f, peaks::kMatrix8,
             [&](void *a, void *b) {
               const int rc = api_.fill_i8(dev_, (int8_t *)a, n, workload.seed, MI355_STREAM_GEMM_A);
               return rc != MI355_OK ? rc : api_.fill_i8(dev_, (int8_t *)b, n, workload.seed, MI355_STREAM_GEMM_B);
             },
             [&](void *a, void *b, void *c) { return api_.gemm_i8(dev_, (const int8_t *)a, (const int8_t *)b, (int32_t *)c, D, D, D); });
}

// ---- bandwidth, latency ---------------------------------------------------------------------------------------------
void Mi355Peak::runGlobalBandwidth() {
  auto test = device_->beginTest({"global_memory_bandwidth", "Global memory bandwidth", "gbps", Category::Unknown,
                                  "Streaming read of a buffer far larger than every cache; each reading fetches a "
                                  "different number of floats per load instruction."});
  static const struct { const char *metric; int width; } variants[] = {{"float", 1}, {"float2", 2}, {"float4", 4}};
  uint64_t n = workload.bwFloats;
  const uint64_t cap = props_.total_mem / 4 / sizeof(float);   // never more than a quarter of VRAM
  if (n > cap) n = cap & ~3ull;
  const uint32_t blocks = (uint32_t)props_.num_cus * workload.bwBlocksPerCU, bs = 256;
  Buffer in(api_, dev_, n * sizeof(float)), out(api_, dev_, (size_t)blocks * bs * sizeof(float));
  const bool ok = in && out && api_.fill_f32(dev_, (float *)in.ptr, n, workload.seed, MI355_STREAM_BW, MI355_DIST_U01) == MI355_OK;
  for (const auto &v : variants) {
    if (!ok) {
      test.skip(v.metric, ResultStatus::Error, "Failed to allocate buffers", loadWidthNote(v.width));
      continue;
    }
    const float us = runKernel([&] { return api_.global_bandwidth(dev_, v.width, (const float *)in.ptr, n, (float *)out.ptr, blocks, bs); },
                               targetTimeUs, forceIters ? specifiedIters : 0);
    if (us <= 0.0f) test.skip(v.metric, ResultStatus::Error, "kernel launch failed", loadWidthNote(v.width));
    else {
      const double gbps = (double)n * sizeof(float) / us / 1e3;
      test.emit(v.metric, (float)gbps, {false, withPeak(loadWidthNote(v.width), gbps, peaks::kHbmGbps, "GB/s HBM3E")});
    }
  }
}

// LDS ping-pong, the reference's shape: 256 threads per workgroup, 64 repetitions, grid sized by
// targetGlobalThreads (include/common/common.h:142-147); bytes = reps * 2 * width * 4 * threads
// (src/rocm/local_bandwidth.cpp:63-65).
void Mi355Peak::runLocalBandwidth() {
  auto test = device_->beginTest({"local_memory_bandwidth", "Local memory bandwidth", "gbps", Category::Unknown,
                                  "How many bytes per second the GPU moves through shared local memory (LDS), the "
                                  "on-chip scratchpad a workgroup passes data through."});
  static const struct { const char *metric; int width; } variants[] = {{"float", 1}, {"float2", 2}, {"float4", 4}};
  const uint32_t bs = 256, reps = 64;
  uint64_t threads = workload.ldsThreads;
  if (threads == 0) threads = std::max<uint64_t>(32ull << 20, (uint64_t)props_.num_cus * 2048ull * 256ull);
  const uint32_t blocks = (uint32_t)(threads / bs);
  threads = (uint64_t)blocks * bs;
  Buffer out(api_, dev_, threads * sizeof(float));
  for (const auto &v : variants) {
    if (!out) {
      test.skip(v.metric, ResultStatus::Error, "Buffer alloc failed", ldsWidthNote(v.width));
      continue;
    }
    const float us = runKernel([&] { return api_.local_bandwidth(dev_, v.width, (float *)out.ptr, blocks, bs, reps); },
                               targetTimeUs, forceIters ? specifiedIters : 0);
    if (us <= 0.0f) test.skip(v.metric, ResultStatus::Error, "kernel launch failed", ldsWidthNote(v.width));
    else test.emit(v.metric, (float)((double)reps * 2.0 * v.width * sizeof(float) * (double)threads / us / 1e3), ldsWidthNote(v.width));
  }
}

// Pinned host buffer <-> device buffer over PCIe, both directions, each timed like a kernel: warm-up
// copies, a one-copy probe, a batch sized to the time budget between two events
// (src/rocm/transfer_bandwidth.cpp:42-103).
void Mi355Peak::runTransferBandwidth() {
  auto test = device_->beginTest({"transfer_bandwidth", "Transfer bandwidth", "gbps", Category::Unknown,
                                  "How fast data crosses between host memory and the card over the PCIe link; both "
                                  "readings use pinned host memory."});
  const char *h2dNote = "Host to device: sending data up to the card.";
  const char *d2hNote = "Device to host: reading results back down.";
  const size_t bytes = (size_t)workload.transferBytes;
  Buffer dbuf(api_, dev_, bytes);
  void *pinned = nullptr;
  if (!dbuf) {
    test.skip("h2d_pinned", ResultStatus::Error, "Failed to allocate device buffer", h2dNote);
    test.skip("d2h_pinned", ResultStatus::Error, "Failed to allocate device buffer", d2hNote);
    return;
  }
  if (api_.host_alloc(dev_, bytes, &pinned) != MI355_OK) {
    test.skip("h2d_pinned", ResultStatus::Error, "Failed to allocate pinned host buffer", h2dNote);
    test.skip("d2h_pinned", ResultStatus::Error, "Failed to allocate pinned host buffer", d2hNote);
    return;
  }
  seeded_uniform_f32((float *)pinned, bytes / sizeof(float), workload.seed, MI355_STREAM_BW);
  const unsigned forced = forceIters ? specifiedIters : 0;
  const float usH2D = runKernel([&] { return api_.copy_async(dev_, dbuf.ptr, pinned, bytes, MI355_H2D); }, targetTimeUs, forced);
  if (usH2D > 0.0f) test.emit("h2d_pinned", (float)((double)bytes / usH2D / 1e3), h2dNote);
  else test.skip("h2d_pinned", ResultStatus::Error, "transfer failed", h2dNote);
  const float usD2H = runKernel([&] { return api_.copy_async(dev_, pinned, dbuf.ptr, bytes, MI355_D2H); }, targetTimeUs, forced);
  if (usD2H > 0.0f) test.emit("d2h_pinned", (float)((double)bytes / usD2H / 1e3), d2hNote);
  else test.skip("d2h_pinned", ResultStatus::Error, "transfer failed", d2hNote);
  api_.host_free(dev_, pinned);
}

void Mi355Peak::runNotBuilt(const char *tag, const char *display, std::initializer_list<std::string> metrics, const char *why,
                            ResultStatus status) {
  auto test = device_->beginTest({tag, display, "gbps", Category::Unknown, ""});
  test.skipAll(metrics, status, why);
}

void Mi355Peak::runKernelLatency(const benchmark_config_t &cfg) {
  auto test = device_->beginTest({"kernel_launch_latency", "Kernel launch latency", "us", Category::Unknown,
                                  "What it costs to ask the GPU to do anything: an empty kernel, launched and waited for."});
  const char *dispatchNote = "Submit to start of execution; the host and the GPU share no clock through HIP.";
  const char *roundtripNote = "Submit, run, hear back: the mean wall-clock time of launch plus stream synchronisation.";
  test.skip("dispatch", ResultStatus::Unsupported, "Not measurable via HIP runtime/module API", dispatchNote);
  double us = 0.0;
  const unsigned n = cfg.kernelLatencyIters ? cfg.kernelLatencyIters : 1000;
  if (api_.launch_roundtrip(dev_, warmupCount, n, &us) != MI355_OK)
    test.skip("roundtrip", ResultStatus::Error, "launch/synchronize failed", roundtripNote);
  else
    test.emit("roundtrip", (float)us, roundtripNote);
}
