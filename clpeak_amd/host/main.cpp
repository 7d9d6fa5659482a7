// Command-line front end of the MI355X backend: the part of clpeak's CLI (src/cli/main.cpp:151-211,
// flag grammar of src/common/options.cpp:406-708) that concerns a ROCm device.
//
//   clpeak-mi355 [--rocm-device 0,2] [--<test>|--no-<test>]... [--<category>|--no-<category>]...
//                [-i N] [-w N] [--max-time ms] [--xml-file f] [--json-file f] [--csv-file f]
//                [--compare f] [--describe] [--list-devices] [--verbose]
// The first positive --<test> (or --<category>) flag switches that set to allow-list mode;
// --no-... always subtracts.  Exit status: 0 ok, the backend's status otherwise, 1 on bad arguments.
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <string>
#include "mi355_peak.h"

namespace {
struct Named { const char *flag; Benchmark b; };
const Named kTests[] = {
    {"global-memory-bandwidth", Benchmark::GlobalBW}, {"local-memory-bandwidth", Benchmark::LocalBW},
    {"image-memory-bandwidth", Benchmark::ImageBW},   {"transfer-bandwidth", Benchmark::TransferBW},
    {"half-precision-compute", Benchmark::ComputeHP}, {"mixed-precision-compute", Benchmark::ComputeMP},
    {"single-precision-compute", Benchmark::ComputeSP}, {"double-precision-compute", Benchmark::ComputeDP},
    {"bfloat16-compute", Benchmark::ComputeBF16},     {"integer-compute", Benchmark::ComputeInt},
    {"integer-compute-int8-dp", Benchmark::ComputeInt8DP}, {"wmma", Benchmark::Wmma},
    {"rocwmma", Benchmark::Rocwmma},                  {"mfma", Benchmark::Mfma},
    {"rocblas", Benchmark::Rocblas},                  {"kernel-launch-latency", Benchmark::KernelLatency}};
struct NamedCat { const char *flag; Category c; };
const NamedCat kCats[] = {{"fp-compute", Category::FpCompute}, {"int-compute", Category::IntCompute},
                          {"bandwidth", Category::Bandwidth}, {"latency", Category::Latency}};

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

void usage(std::ostream &os) {
  os << "clpeak-mi355 " CLPEAK_MI355_VERSION " -- clpeak compute backend for AMD Instinct MI355X (gfx950)\n"
        "  --rocm-device LIST      comma-separated device ordinals (default: all)\n"
        "  --<test> / --no-<test>  ";
  for (const Named &t : kTests) os << t.flag << " ";
  os << "\n  --<category> / --no-<category>  fp-compute int-compute bandwidth latency\n"
        "  -i, --iters N           fixed iteration count per timed batch\n"
        "  -w, --warmup N          warm-up launches (default 2)\n"
        "  --max-time MS           time budget of a timed batch (default 500 ms)\n"
        "  --xml-file F | --json-file F | --csv-file F   dump results\n"
        "  --compare F             print the change against a previous dump\n"
        "  --describe              print what each test and reading means\n"
        "  --list-devices          list devices and exit\n"
        "  --verbose               diagnostics on stderr\n";
}
}  // namespace

int main(int argc, char **argv) {
  CliOptions opts;
  bool testsAllowList = false, catsAllowList = false, fake = false;
  Mi355Peak::Workload shape;
  auto need = [&](int &i) -> const char * {
    if (i + 1 >= argc) { std::cerr << "clpeak: " << argv[i] << " needs a value\n"; exit(1); }
    return argv[++i];
  };
  for (int i = 1; i < argc; i++) {
    const std::string a = argv[i];
    if (a == "-h" || a == "--help") { usage(std::cout); return 0; }
    else if (a == "--rocm") {}
    else if (a == "--rocm-device") {
      if (!parseIntList(need(i), opts.rocmDeviceIndices)) { std::cerr << "clpeak: bad --rocm-device list\n"; return 1; }
    } else if (a == "-i" || a == "--iters") { opts.iters = (unsigned)atoi(need(i)); opts.forceIters = opts.iters > 0; }
    else if (a == "-w" || a == "--warmup") opts.warmupCount = (unsigned)atoi(need(i));
    else if (a == "--max-time") opts.targetTimeUs = (unsigned)atoi(need(i)) * 1000u;
    else if (a == "--xml-file") { opts.xmlFile = need(i); opts.enableXml = true; }
    else if (a == "--json-file") { opts.jsonFile = need(i); opts.enableJson = true; }
    else if (a == "--csv-file") { opts.csvFile = need(i); opts.enableCsv = true; }
    else if (a == "--compare") opts.compareFile = need(i);
    else if (a == "--describe") opts.describe = true;
    else if (a == "--list-devices") opts.listDevices = true;
    else if (a == "--verbose") opts.verbose = true;
    // not part of clpeak's grammar: stand-in device and reduced shapes, for tests of the host logic
    else if (a == "--fake-device") fake = true;
    else if (a == "--small-shapes") {
      shape.madItems = 1 << 12; shape.madSteps = 64; shape.bwFloats = 1 << 22; shape.mfmaWavesPerCU = 1;
      shape.mfmaIters = 32; shape.gemmDim = 512; shape.latencyLaunches = 50;
      shape.ldsThreads = 1 << 16; shape.transferBytes = 1 << 22;
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
      if (!hit) { std::cerr << "clpeak: unknown option " << a << "\n"; usage(std::cerr); return 1; }
    } else { std::cerr << "clpeak: unknown argument " << a << "\n"; return 1; }
  }

  const Mi355Api &api = fake ? mi355_fake_api() : mi355_real_api();
  if (opts.listDevices) {
    Mi355Peak::printInventory(Mi355Peak::enumerate(api), std::cout);
    return 0;
  }

  Mi355Peak peak(api);
  peak.workload = shape;
  peak.log.reset(new LoggerText(std::cout, opts.compareFile, opts.describe));
  peak.applyOptions(opts);
  const int status = peak.runAll();
  bool dumped = true;
  if (opts.enableXml) dumped &= saveXml(peak.log->results, opts.xmlFile, peak.log->devices);
  if (opts.enableJson) dumped &= saveJson(peak.log->results, opts.jsonFile, peak.log->devices);
  if (opts.enableCsv) dumped &= saveCsv(peak.log->results, opts.csvFile);
  return status ? status : (dumped ? 0 : 1);
}
