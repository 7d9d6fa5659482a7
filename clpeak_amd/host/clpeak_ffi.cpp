// The embedding C ABI (include/clpeak_ffi.h) on top of Mi355Peak: catalog, blocking launch with a
// streamed event callback, cooperative cancel, saved-result loading.  Protocol of the reference's
// src/ffi/clpeak_ffi.cpp:132-225: one launch at a time (a second caller gets BUSY and no events),
// the cancel flag resets when a launch starts, bad arguments produce a note and a done event, the
// result files are written after the run also when it was cancelled, done is always last.
#include "../../include/clpeak_ffi.h"
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <locale>
#include <sstream>
#include <vector>
#include "logger_ffi.h"
#include "options.h"
#include "results.h"

namespace {
char *copyString(const std::string &s) {
  char *out = static_cast<char *>(std::malloc(s.size() + 1));
  if (out) std::memcpy(out, s.c_str(), s.size() + 1);
  return out;
}

void deviceJson(std::ostream &os, const InventoryDevice &d) {
  os << "{\"index\":" << d.index << ",\"name\":\"" << jsonEscape(d.name) << "\",\"type\":\"" << jsonEscape(d.typeStr) << "\"";
  if (!d.driverVersion.empty()) os << ",\"driver\":\"" << jsonEscape(d.driverVersion) << "\"";
  if (!d.apiVersion.empty()) os << ",\"api\":\"" << jsonEscape(d.apiVersion) << "\"";
  if (d.numComputeUnits) os << ",\"computeUnits\":" << d.numComputeUnits;
  if (d.maxClockMHz) os << ",\"clockMHz\":" << d.maxClockMHz;
  if (d.globalMemBytes) os << ",\"globalMemBytes\":" << d.globalMemBytes;
  if (d.maxAllocBytes) os << ",\"maxAllocBytes\":" << d.maxAllocBytes;
  if (d.hasFp16) os << ",\"fp16\":true";
  if (d.hasFp64) os << ",\"fp64\":true";
  os << "}";
}

void emitNote(ClpeakEventCallback cb, void *ud, const std::string &msg) {
  LogEvent e;
  e.kind = LogEvent::Kind::Note;
  e.message = msg;
  ffiEmitJson(cb, ud, ffiEventToJson(e));
}

void emitDone(ClpeakEventCallback cb, void *ud, int status, bool cancelled) {
  ffiEmitJson(cb, ud, "{\"t\":\"done\",\"status\":" + std::to_string(status) + ",\"cancelled\":" + (cancelled ? "true" : "false") + "}");
}

std::atomic<bool> g_running{false};
}  // namespace

std::string inventoryToJson(const std::vector<BackendInventory> &inv) {
  std::ostringstream os;
  os.imbue(std::locale::classic());
  os << "{\"backends\":[";
  for (size_t i = 0; i < inv.size(); i++) {
    const BackendInventory &b = inv[i];
    os << (i ? "," : "") << "{\"name\":\"" << jsonEscape(b.backend) << "\",\"available\":" << (b.available ? "true" : "false")
       << ",\"platforms\":[";
    for (size_t p = 0; p < b.platforms.size(); p++) {
      const InventoryPlatform &plat = b.platforms[p];
      os << (p ? "," : "") << "{\"index\":" << plat.index << ",\"name\":\"" << jsonEscape(plat.name) << "\",\"devices\":[";
      for (size_t d = 0; d < plat.devices.size(); d++) {
        if (d) os << ",";
        deviceJson(os, plat.devices[d]);
      }
      os << "]}";
    }
    os << "]}";
  }
  os << "]}";
  return os.str();
}

extern "C" {

const char *clpeak_version(void) { return CLPEAK_MI355_VERSION; }

char *clpeak_copy_backend_catalog_json(void) {
  return copyString(inventoryToJson({Mi355Peak::enumerate(mi355_api())}));
}

void clpeak_free_string(char *s) { std::free(s); }

void clpeak_request_cancel(void) { clpeak::requestCancel(); }

char *clpeak_load_result_file_json(const char *path) {
  if (!path) return nullptr;
  DeviceInfoStore devices;
  const ResultStore store = loadResultFile(path, &devices);
  if (store.empty()) return nullptr;
  return copyString(resultsToJson(store, devices));
}

int clpeak_launch(int argc, const char **argv, ClpeakEventCallback on_event, void *user_data) {
  bool expected = false;
  if (!g_running.compare_exchange_strong(expected, true)) return CLPEAK_RUN_BUSY;   // the running launch owns the stream
  clpeak::resetCancel();

  std::vector<char *> args;
  for (int i = 0; i < argc; i++) args.push_back(const_cast<char *>(argv[i]));
  CliOptions opts;
  HostExtras extras;
  std::string error;
  if (argc < 0 || (argc > 0 && !argv) || !parseCliOptionsNoExit(argc, args.data(), opts, extras, error) || opts.listDevices) {
    if (error.empty()) error = opts.listDevices ? "clpeak: --list-devices is not available in embedded mode\n" : "clpeak: bad arguments\n";
    emitNote(on_event, user_data, error);
    emitDone(on_event, user_data, CLPEAK_RUN_BAD_ARGS, false);
    g_running.store(false);
    return CLPEAK_RUN_BAD_ARGS;
  }
  clpeak::setVerbose(opts.verbose);

  ResultStore combined;
  DeviceInfoStore combinedDevices;
  int status = 0;
  if (!opts.skipRocm && !clpeak::cancelRequested()) {
    Mi355Peak peak(mi355_api());
    peak.workload = extras.shape;
    peak.log.reset(new LoggerFfi(on_event, user_data));
    peak.applyOptions(opts);
    status |= peak.runAll();
    combined = peak.log->results;
    combinedDevices = peak.log->devices;
  }
  if (opts.enableJson && !saveJson(combined, opts.jsonFile, combinedDevices)) status |= 1;
  if (opts.enableCsv && !saveCsv(combined, opts.csvFile)) status |= 1;
  if (opts.enableXml && !saveXml(combined, opts.xmlFile, combinedDevices)) status |= 1;

  const bool cancelled = clpeak::cancelRequested();
  const int result = cancelled ? CLPEAK_RUN_CANCELLED : status;
  emitDone(on_event, user_data, result, cancelled);
  g_running.store(false);
  return result;
}

}  // extern "C"
