// Structured run log: what a backend reports through and what front ends render.
//
// The scope API (beginBackend -> beginDevice -> beginTest -> emit / skip / skipAll) and the
// event stream behind it are those of the reference (include/common/logger.h:38-285,
// src/common/logger.cpp:86-340): one LogEvent per observable moment, handles that close
// themselves, at most one test open at a time, rows accumulated in `results` and device
// facts in `devices`.  Output channels override onEvent(); LoggerText renders the CLI table
// (src/common/logger_text.cpp:106-247).
#pragma once
#include <initializer_list>
#include <iosfwd>
#include <string>
#include <vector>
#include "results.h"

struct LogEvent {
  enum class Kind { BackendBegin, DeviceBegin, TestBegin, Metric, TestSkippedAll, TestEnd, DeviceEnd, BackendEnd, Note };
  Kind kind = Kind::Note;
  // scope context at the time of the event (empty when that scope is not open)
  std::string backend, platform, device, driver, testTag, testDisplay, unit, testDescription;
  Category category = Category::Unknown;
  // DeviceBegin
  std::vector<DeviceProp> props;
  int platformIndex = -1, deviceIndex = -1;
  bool showPlatformLine = false;
  // Metric
  ResultEntry entry;
  bool subMetric = false;
  // TestSkippedAll
  std::vector<std::string> metricNames;
  ResultStatus status = ResultStatus::Ok;
  std::string reason;
  // Note
  std::string message;
};

class logger {
 public:
  using Prop = DeviceProp;
  struct DeviceSpec {
    std::string name, platform /* empty = backend name */, driver_version;
    std::vector<Prop> props;
    int platform_index = -1, device_index = -1;
  };
  struct TestSpec {
    std::string tag, display, unit;
    Category category = Category::Unknown;   // Unknown = derive from the unit
    std::string description;
  };
  struct EmitOptions {
    bool subMetric = false;
    std::string description;
  };
  class BackendScope;
  class DeviceScope;
  class TestScope;

  explicit logger(std::string compareFileName = "");
  virtual ~logger() = default;

  BackendScope beginBackend(const std::string &name);
  void note(const std::string &msg);

  bool compareEnabled = false;
  BaselineMap baseline;
  ResultStore results;
  DeviceInfoStore devices;

 protected:
  virtual void onEvent(const LogEvent &e) = 0;

 private:
  // depth 0 none, 1 backend, 2 device, 3 test
  int depth_ = 0;
  std::string backend_, platform_, device_, driver_, test_, display_, description_, unit_;
  Category category_ = Category::Unknown;
  unsigned long long testSerial_ = 0, openSerial_ = 0;

  LogEvent stamp(LogEvent::Kind kind) const;
  ResultEntry row(const std::string &metric, ResultStatus st, float value, const std::string &reason,
                  const std::string &note) const;
  void endOpenTest();
  friend class BackendScope;
  friend class DeviceScope;
  friend class TestScope;
};

class logger::BackendScope {
 public:
  BackendScope(logger *log, const std::string &name);
  ~BackendScope() { end(); }
  BackendScope(BackendScope &&o) noexcept : log_(o.log_), closed_(o.closed_) { o.closed_ = true; }
  BackendScope(const BackendScope &) = delete;
  BackendScope &operator=(const BackendScope &) = delete;
  DeviceScope beginDevice(const DeviceSpec &spec);
  void end();
 private:
  logger *log_;
  bool closed_ = false;
};

class logger::DeviceScope {
 public:
  DeviceScope(logger *log, const DeviceSpec &spec);
  ~DeviceScope() { end(); }
  DeviceScope(DeviceScope &&o) noexcept : log_(o.log_), closed_(o.closed_) { o.closed_ = true; }
  DeviceScope(const DeviceScope &) = delete;
  DeviceScope &operator=(const DeviceScope &) = delete;
  TestScope beginTest(const TestSpec &spec);
  void end();
 private:
  logger *log_;
  bool closed_ = false;
};

class logger::TestScope {
 public:
  TestScope(logger *log, const TestSpec &spec);
  ~TestScope() { end(); }
  TestScope(TestScope &&o) noexcept : log_(o.log_), closed_(o.closed_), serial_(o.serial_) { o.closed_ = true; }
  TestScope(const TestScope &) = delete;
  TestScope &operator=(const TestScope &) = delete;
  void emit(std::string metric, float value, EmitOptions opts = {});
  void emit(std::string metric, float value, const char *description);
  void skip(std::string metric, ResultStatus status, std::string reason, std::string description = "");
  void skipAll(std::initializer_list<std::string> metrics, ResultStatus status, std::string reason);
  void end();
 private:
  logger *log_;
  bool closed_ = false;
  unsigned long long serial_ = 0;   // equals logger::openSerial_ while this is the open test
};

// Indented text table: "<display> (<UNIT>)" then "<metric padded to >= 8> : <value %.2f>".
class LoggerText : public logger {
 public:
  explicit LoggerText(std::ostream &out, const std::string &compareFileName = "", bool describe = false);
 protected:
  void onEvent(const LogEvent &e) override;
 private:
  struct Pending { ResultEntry entry; bool sub; };
  std::ostream &out_;
  bool describe_;
  size_t deviceSteps_ = 1;   // indentation of the device line in steps of two spaces
  std::vector<Pending> pending_;   // rows of the open test, printed together so they align
  void flush();
};
