#include "options.h"
#include <cstdlib>
#include <cstring>
#include <ostream>

namespace {
struct Named { const char *flag; Benchmark b; };
const Named kTests[] = {
    {"global-memory-bandwidth", Benchmark::GlobalBW}, {"local-memory-bandwidth", Benchmark::LocalBW},
    {"image-memory-bandwidth", Benchmark::ImageBW},   {"transfer-bandwidth", Benchmark::TransferBW},
    {"half-precision-compute", Benchmark::ComputeHP}, {"mixed-precision-compute", Benchmark::ComputeMP},
    {"single-precision-compute", Benchmark::ComputeSP}, {"double-precision-compute", Benchmark::ComputeDP},
    {"bfloat16-compute", Benchmark::ComputeBF16},     {"integer-compute", Benchmark::ComputeInt},
    {"int8-dot-product-compute", Benchmark::ComputeInt8DP}, {"wmma", Benchmark::Wmma},
    {"rocwmma", Benchmark::Rocwmma},                  {"mfma", Benchmark::Mfma},
    {"rocblas", Benchmark::Rocblas},                  {"kernel-launch-latency", Benchmark::KernelLatency}};
struct NamedCat { const char *flag; Category c; };
const NamedCat kCats[] = {{"fp-compute", Category::FpCompute}, {"int-compute", Category::IntCompute},
                          {"crypto", Category::Crypto},         {"string", Category::String},
                          {"bandwidth", Category::Bandwidth},   {"latency", Category::Latency}};

// The rest of clpeak's grammar (src/common/options.cpp:194-264, 469-497, 552-639): flags that select tests, backends
// and devices this backend does not have.  A front end written against clpeak passes them (the GUI names every
// selected category and every deselected backend, app/lib/src/model/run_config.dart:98-144), so they parse here
// with the same effect they have on the ROCm backend there: tests of other backends select nothing of this one but
// still switch test selection to an allow-list, another backend named alone leaves this one out, device lists of
// other backends are checked and dropped.
const char *const kForeignTests[] = {
    "integer-compute-fast", "integer-compute-char", "integer-compute-short", "int16-dot-product-compute",
    "fp8-dot-product-compute", "divide-sqrt-compute", "integer-divide-compute", "coopmat", "simdgroup-matrix", "cublas",
    "mps-gemm", "mps-attention", "texture-sample", "joint-matrix", "onemkl", "amx", "accelerate", "aes", "sha256",
    "sha512", "crc32c", "string-scan", "utf8-validate", "cache-bandwidth", "memory-latency", "atomics",
    "branch-penalty", "store-forward", "smt-scaling"};
const char *const kForeignBackends[] = {"opencl", "vulkan", "cuda", "metal", "oneapi", "cpu"};
const char *const kForeignDeviceLists[] = {"--cl-platform", "--cl-device", "--vk-device", "--cuda-device", "--mtl-device",
                                           "--oneapi-device"};

bool parseIntList(const char *s, std::vector<int> &out) {
  std::string tok;
  for (const char *p = s;; p++) {
    if (*p == ',' || *p == '\0') {
      if (tok.empty()) return false;
      char *end = nullptr;
      const long v = strtol(tok.c_str(), &end, 10);
      if (*end || v < 0) return false;
      out.push_back((int)v);
      tok.clear();
      if (!*p) return true;
    } else tok += *p;
  }
}

bool parseUnsigned(const char *s, unsigned &out, bool allowZero = true) {
  if (!s || !*s) return false;
  for (const char *p = s; *p; p++)
    if (*p < '0' || *p > '9') return false;
  char *end = nullptr;
  const unsigned long long v = strtoull(s, &end, 10);
  if (*end || v > 0xffffffffull || (!allowZero && v == 0)) return false;
  out = (unsigned)v;
  return true;
}
}  // namespace

void printUsage(std::ostream &os) {
  os << "clpeak-mi355 " CLPEAK_MI355_VERSION " -- clpeak compute backend for AMD Instinct MI355X (gfx950)\n"
        "  --rocm-device LIST      comma-separated device ordinals (default: all)\n"
        "  --<test> / --no-<test>  ";
  for (const Named &t : kTests) os << t.flag << " ";
  os << "\n  --<category> / --no-<category>  fp-compute int-compute bandwidth latency (crypto, string: none here)\n"
        "  flags of clpeak's other backends (--opencl, --no-cpu, --cuda-device LIST, --max-time-cpu MS, --aes, ...)\n"
        "                          are accepted with the meaning they have for the ROCm backend there\n"
        "  -i, --iters N           fixed iteration count per timed batch\n"
        "  -w, --warmup N          warm-up launches (default 2)\n"
        "  --max-time MS           time budget of a timed batch (default 500 ms)\n"
        "  --xml-file F | --json-file F | --csv-file F   dump results\n"
        "  --compare F             print the change against a previous dump\n"
        "  --describe              print what each test and reading means\n"
        "  --list-devices          list devices and exit\n"
        "  --verbose               diagnostics on stderr\n"
        "  --reference-operands    matrix rows on the constant operands clpeak's own kernels use, not seeded ones\n"
        "  -v, --version | -h, --help\n";
}

ParseResult parseCliCore(int argc, char **argv, CliOptions &opts, HostExtras &extras, std::string &error) {
  bool testsAllowList = false, catsAllowList = false;
  bool otherBackendNamed = false, rocmNamed = false;
  const char *value = nullptr;
  auto need = [&](int &i) -> bool {
    if (i + 1 >= argc) {
      error = std::string("clpeak: missing argument for ") + argv[i] + "\n";
      return false;
    }
    value = argv[++i];
    return true;
  };
  auto invalid = [&](const char *flag) {
    error = std::string("clpeak: invalid value for ") + flag + ": " + value + "\n";
    return ParseResult::Error;
  };
  for (int i = 1; i < argc; i++) {
    const std::string a = argv[i];
    if (a == "-h" || a == "--help") return ParseResult::Help;
    if (a == "-v" || a == "--version") return ParseResult::Version;
    if (a == "--rocm") { rocmNamed = true; continue; }
    if (a == "--no-rocm") { opts.skipRocm = true; continue; }
    bool foreign = false;
    for (const char *b : kForeignBackends) {
      if (a == std::string("--") + b) { otherBackendNamed = true; foreign = true; }
      if (a == std::string("--no-") + b) foreign = true;
    }
    if (a == "--use-event-timer") foreign = true;   // OpenCL's timer choice
    for (const char *f : kForeignDeviceLists)
      if (a == f) {
        std::vector<int> ignored;
        if (!need(i)) return ParseResult::Error;
        if (!parseIntList(value, ignored)) {
          error = std::string("clpeak: invalid device index list: ") + value + "\n";
          return ParseResult::Error;
        }
        foreign = true;
      }
    if (a == "--max-time-cpu") {
      unsigned ms = 0;
      if (!need(i)) return ParseResult::Error;
      if (!parseUnsigned(value, ms, false) || ms > 0xffffffffu / 1000u) return invalid("--max-time-cpu");
      foreign = true;
    }
    if (foreign) continue;
    if (a == "--rocm-device") {
      if (!need(i)) return ParseResult::Error;
      if (!parseIntList(value, opts.rocmDeviceIndices)) {
        error = std::string("clpeak: invalid device list: ") + value + "\n";
        return ParseResult::Error;
      }
    } else if (a == "-i" || a == "--iters") {
      if (!need(i)) return ParseResult::Error;
      if (!parseUnsigned(value, opts.iters, false)) return invalid(a.c_str());
      opts.forceIters = true;
    } else if (a == "-w" || a == "--warmup") {
      if (!need(i)) return ParseResult::Error;
      if (!parseUnsigned(value, opts.warmupCount)) return invalid(a.c_str());
    } else if (a == "--max-time") {
      unsigned ms = 0;
      if (!need(i)) return ParseResult::Error;
      if (!parseUnsigned(value, ms, false) || ms > 0xffffffffu / 1000u) return invalid("--max-time");
      opts.targetTimeUs = ms * 1000u;
    } else if (a == "--xml-file") { if (!need(i)) return ParseResult::Error; opts.xmlFile = value; opts.enableXml = true; }
    else if (a == "--json-file") { if (!need(i)) return ParseResult::Error; opts.jsonFile = value; opts.enableJson = true; }
    else if (a == "--csv-file") { if (!need(i)) return ParseResult::Error; opts.csvFile = value; opts.enableCsv = true; }
    else if (a == "--compare") { if (!need(i)) return ParseResult::Error; opts.compareFile = value; }
    else if (a == "--describe") opts.describe = true;
    else if (a == "--list-devices") opts.listDevices = true;
    else if (a == "--verbose") opts.verbose = true;
    else if (a == "--reference-operands") extras.shape.referenceOperands = true;
    else if (a == "--small-shapes") {
      Mi355Peak::Workload &s = extras.shape;
      s.madItems = 1 << 12; s.madSteps = 64; s.bwFloats = 1 << 22; s.mfmaWavesPerCU = 1;
      s.mfmaIters = 32; s.gemmDim = 512; s.latencyLaunches = 50;
      s.ldsThreads = 1 << 16; s.transferBytes = 1 << 22;
    } else if (a.compare(0, 2, "--") == 0) {
      const bool neg = a.compare(0, 5, "--no-") == 0;
      const std::string name = a.substr(neg ? 5 : 2);
      bool hit = false;
      for (const Named &t : kTests)
        if (name == t.flag) {
          if (!neg && !testsAllowList) { opts.enabledTests.reset(); testsAllowList = true; }
          opts.enabledTests.set((size_t)t.b, !neg);
          hit = true;
        }
      for (const NamedCat &c : kCats)
        if (name == c.flag) {
          if (!neg && !catsAllowList) { opts.enabledCategories.reset(); catsAllowList = true; }
          opts.enabledCategories.set((size_t)c.c, !neg);
          hit = true;
        }
      if (name == "integer-compute-int8-dp") {   // this program's earlier spelling of --int8-dot-product-compute
        if (!neg && !testsAllowList) { opts.enabledTests.reset(); testsAllowList = true; }
        opts.enabledTests.set((size_t)Benchmark::ComputeInt8DP, !neg);
        hit = true;
      }
      for (const char *t : kForeignTests)
        if (name == t) {
          if (!neg && !testsAllowList) { opts.enabledTests.reset(); testsAllowList = true; }
          hit = true;
        }
      if (!hit) {
        error = "clpeak: unknown option '" + a + "'\n";
        return ParseResult::Error;
      }
    } else {
      error = "clpeak: unknown option '" + a + "'\n";
      return ParseResult::Error;
    }
  }
  // any --<backend> flag means "only the listed backends" (src/common/options.cpp:685-697)
  if (otherBackendNamed && !rocmNamed) opts.skipRocm = true;
  return ParseResult::Ok;
}

bool parseCliOptionsNoExit(int argc, char **argv, CliOptions &opts, HostExtras &extras, std::string &error) {
  switch (parseCliCore(argc, argv, opts, extras, error)) {
    case ParseResult::Ok: return true;
    case ParseResult::Help: error = "clpeak: --help is not available in embedded mode\n"; return false;
    case ParseResult::Version: error = "clpeak: --version is not available in embedded mode\n"; return false;
    default: return false;
  }
}
