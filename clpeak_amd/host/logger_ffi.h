// Logger whose sink is the embedding callback: every event becomes one JSON document
// (reference: src/ffi/logger_ffi.h:12-34, src/ffi/logger_ffi.cpp:15-146).
#pragma once
#include <string>
#include "../../include/clpeak_ffi.h"
#include "run_log.h"

std::string ffiEventToJson(const LogEvent &e);
// malloc's a copy of `json` and hands it to the callback, which owns it from then on.
void ffiEmitJson(ClpeakEventCallback cb, void *userData, const std::string &json);

class LoggerFfi : public logger {
 public:
  LoggerFfi(ClpeakEventCallback cb, void *userData) : cb_(cb), userData_(userData) {}
 protected:
  void onEvent(const LogEvent &e) override { ffiEmitJson(cb_, userData_, ffiEventToJson(e)); }
 private:
  ClpeakEventCallback cb_;
  void *userData_;
};
