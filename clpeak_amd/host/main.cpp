// Command-line front end of the MI355X backend: the part of clpeak's CLI (src/cli/main.cpp:151-211,
// flag grammar of src/common/options.cpp:406-708) that concerns a ROCm device.
//
//   clpeak-mi355 [--rocm-device 0,2] [--<test>|--no-<test>]... [--<category>|--no-<category>]...
//                [-i N] [-w N] [--max-time ms] [--xml-file f] [--json-file f] [--csv-file f]
//                [--compare f] [--describe] [--list-devices] [--verbose]
// The first positive --<test> (or --<category>) flag switches that set to allow-list mode;
// --no-... always subtracts.  Exit status: 0 ok, the backend's status otherwise, 1 on bad arguments.
#include <iostream>
#include <string>
#include "options.h"

int main(int argc, char **argv) {
  CliOptions opts;
  HostExtras extras;
  std::string error;
  switch (parseCliCore(argc, argv, opts, extras, error)) {
    case ParseResult::Help: printUsage(std::cout); return 0;
    case ParseResult::Version: std::cout << "clpeak-mi355 " CLPEAK_MI355_VERSION "\n"; return 0;
    case ParseResult::Error: std::cerr << error; printUsage(std::cerr); return 1;
    case ParseResult::Ok: break;
  }
  clpeak::setVerbose(opts.verbose);

  const Mi355Api &api = mi355_api();
  if (opts.listDevices) {
    Mi355Peak::printInventory(Mi355Peak::enumerate(api), std::cout);
    return 0;
  }
  if (opts.skipRocm) return 0;

  Mi355Peak peak(api);
  peak.workload = extras.shape;
  peak.log.reset(new LoggerText(std::cout, opts.compareFile, opts.describe));
  peak.applyOptions(opts);
  const int status = peak.runAll();
  bool dumped = true;
  if (opts.enableXml) dumped &= saveXml(peak.log->results, opts.xmlFile, peak.log->devices);
  if (opts.enableJson) dumped &= saveJson(peak.log->results, opts.jsonFile, peak.log->devices);
  if (opts.enableCsv) dumped &= saveCsv(peak.log->results, opts.csvFile);
  return status ? status : (dumped ? 0 : 1);
}
