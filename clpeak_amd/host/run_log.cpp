#include "run_log.h"
#include <algorithm>
#include <cstdio>
#include <iostream>

namespace {
// descriptions travel in attributes and table cells: keep them on one line
std::string flatten(const std::string &s) {
  std::string o;
  bool space = false;
  for (char c : s) {
    if (c == '\n' || c == '\r' || c == '\t' || c == ' ') { space = !o.empty(); continue; }
    if (space) o += ' ';
    space = false;
    o += c;
  }
  return o;
}
}  // namespace

logger::logger(std::string compareFileName) {
  if (!compareFileName.empty()) {
    baseline = buildBaselineMap(loadResultFile(compareFileName));
    compareEnabled = !baseline.empty();
  }
}

LogEvent logger::stamp(LogEvent::Kind kind) const {
  LogEvent e;
  e.kind = kind;
  e.backend = backend_; e.platform = platform_; e.device = device_; e.driver = driver_;
  e.testTag = test_; e.testDisplay = display_; e.unit = unit_; e.testDescription = description_;
  e.category = category_;
  return e;
}

ResultEntry logger::row(const std::string &metric, ResultStatus st, float value, const std::string &reason,
                        const std::string &note) const {
  ResultEntry r;
  r.backend = backend_; r.platform = platform_; r.device = device_; r.driver = driver_;
  r.category = categoryString(category_);
  r.test = test_; r.metric = metric; r.unit = unit_;
  r.status = st; r.value = value; r.reason = reason;
  r.display = display_; r.description = description_; r.metricDescription = flatten(note);
  return r;
}

logger::BackendScope logger::beginBackend(const std::string &name) { return BackendScope(this, name); }

void logger::note(const std::string &msg) {
  LogEvent e = stamp(LogEvent::Kind::Note);
  e.message = msg;
  onEvent(e);
}

void logger::endOpenTest() {
  if (depth_ != 3) return;
  onEvent(stamp(LogEvent::Kind::TestEnd));
  test_.clear(); display_.clear(); description_.clear(); unit_.clear();
  category_ = Category::Unknown;
  depth_ = 2;
  openSerial_ = 0;
}

// ---- backend ------------------------------------------------------------------------------
logger::BackendScope::BackendScope(logger *log, const std::string &name) : log_(log) {
  log->backend_ = name;
  log->platform_.clear(); log->device_.clear(); log->driver_.clear();
  log->depth_ = 1;
  log->onEvent(log->stamp(LogEvent::Kind::BackendBegin));
}

void logger::BackendScope::end() {
  if (closed_) return;
  closed_ = true;
  log_->onEvent(log_->stamp(LogEvent::Kind::BackendEnd));
  log_->backend_.clear();
  log_->depth_ = 0;
}

logger::DeviceScope logger::BackendScope::beginDevice(const DeviceSpec &spec) { return DeviceScope(log_, spec); }

// ---- device -------------------------------------------------------------------------------
logger::DeviceScope::DeviceScope(logger *log, const DeviceSpec &spec) : log_(log) {
  log->platform_ = spec.platform.empty() ? log->backend_ : spec.platform;
  log->device_ = spec.name;
  log->driver_ = spec.driver_version;
  log->depth_ = 2;
  DeviceInfo info;
  info.backend = log->backend_; info.platform = log->platform_; info.device = log->device_; info.driver = log->driver_;
  info.props = spec.props;
  auto known = std::find_if(log->devices.begin(), log->devices.end(),
                            [&](const DeviceInfo &d) { return d.key() == info.key(); });
  if (known == log->devices.end()) log->devices.push_back(info);
  else known->props = info.props;
  LogEvent e = log->stamp(LogEvent::Kind::DeviceBegin);
  e.props = spec.props;
  e.platformIndex = spec.platform_index;
  e.deviceIndex = spec.device_index;
  e.showPlatformLine = log->platform_ != log->backend_;
  log->onEvent(e);
}

void logger::DeviceScope::end() {
  if (closed_) return;
  closed_ = true;
  log_->endOpenTest();
  log_->onEvent(log_->stamp(LogEvent::Kind::DeviceEnd));
  log_->device_.clear(); log_->driver_.clear(); log_->platform_.clear();
  log_->depth_ = 1;
}

logger::TestScope logger::DeviceScope::beginTest(const TestSpec &spec) {
  if (log_->depth_ == 3) {   // a sibling was left open: close it, say so, carry on
    const std::string prev = log_->test_;
    log_->endOpenTest();
    log_->note("logger: test '" + spec.tag + "' opened while '" + prev + "' was still open; closed it first");
  }
  return TestScope(log_, spec);
}

// ---- test ---------------------------------------------------------------------------------
logger::TestScope::TestScope(logger *log, const TestSpec &spec) : log_(log) {
  log->test_ = spec.tag;
  log->display_ = spec.display;
  log->description_ = flatten(spec.description);
  log->unit_ = spec.unit;
  log->category_ = spec.category != Category::Unknown ? spec.category : categoryFromUnit(spec.unit);
  log->depth_ = 3;
  serial_ = ++log->testSerial_;
  log->openSerial_ = serial_;
  log->onEvent(log->stamp(LogEvent::Kind::TestBegin));
}

void logger::TestScope::emit(std::string metric, float value, EmitOptions opts) {
  if (closed_ || log_->openSerial_ != serial_) return;
  LogEvent e = log_->stamp(LogEvent::Kind::Metric);
  e.entry = log_->row(metric, ResultStatus::Ok, value, "", opts.description);
  e.subMetric = opts.subMetric;
  log_->results.push_back(e.entry);
  log_->onEvent(e);
}

void logger::TestScope::emit(std::string metric, float value, const char *description) {
  EmitOptions o;
  if (description) o.description = description;
  emit(std::move(metric), value, std::move(o));
}

void logger::TestScope::skip(std::string metric, ResultStatus status, std::string reason, std::string description) {
  if (closed_ || log_->openSerial_ != serial_) return;
  LogEvent e = log_->stamp(LogEvent::Kind::Metric);
  e.entry = log_->row(metric, status, 0.0f, reason, description);
  log_->results.push_back(e.entry);
  log_->onEvent(e);
}

void logger::TestScope::skipAll(std::initializer_list<std::string> metrics, ResultStatus status, std::string reason) {
  if (closed_ || log_->openSerial_ != serial_) return;
  LogEvent e = log_->stamp(LogEvent::Kind::TestSkippedAll);
  e.status = status;
  e.reason = reason;
  for (const std::string &m : metrics) {
    log_->results.push_back(log_->row(m, status, 0.0f, reason, ""));
    e.metricNames.push_back(m);
  }
  log_->onEvent(e);
}

void logger::TestScope::end() {
  if (closed_) return;
  closed_ = true;
  if (log_->openSerial_ == serial_) log_->endOpenTest();   // a stale handle must not emit a second TestEnd
}

// ---- text renderer ----------------------------------------------------------------------------
LoggerText::LoggerText(std::ostream &out, const std::string &compareFileName, bool describe)
    : logger(compareFileName), out_(out), describe_(describe) {}

static std::string statusLabel(ResultStatus s) {
  switch (s) {
    case ResultStatus::Unsupported: return "unsupported";
    case ResultStatus::Skipped: return "skipped";
    case ResultStatus::Error: return "error";
    default: return "ok";
  }
}

// Word-wrap `text` to 80 columns behind `column` spaces, never narrower than 32 characters; a word longer than
// that overruns (the --describe layout of src/common/logger_text.cpp:266-299).
static void writeWrapped(std::ostream &out, size_t column, const std::string &text) {
  const std::string pad(column, ' ');
  const size_t width = column + 32 > 80 ? 32 : 80 - column;
  std::string line;
  size_t pos = 0;
  while (pos < text.size()) {
    const size_t end = text.find(' ', pos);
    const std::string word = text.substr(pos, end == std::string::npos ? std::string::npos : end - pos);
    pos = end == std::string::npos ? text.size() : end + 1;
    if (word.empty()) continue;
    if (!line.empty() && line.size() + 1 + word.size() > width) {
      out << pad << line << "\n";
      line.clear();
    }
    if (!line.empty()) line += ' ';
    line += word;
  }
  if (!line.empty()) out << pad << line << "\n";
}

// Layout (src/common/logger_text.cpp:48-247): the device line sits one step (two spaces) in, or two when a
// platform line precedes it; properties and test headers one step further, readings one more, sub-readings one
// more again.  Names are padded to the longest of the test (at least 8), sub-readings two less.
void LoggerText::flush() {
  size_t width = 8;
  for (const Pending &p : pending_) width = std::max(width, p.entry.metric.size());
  const size_t readingColumn = (deviceSteps_ + 2) * 2;
  for (const Pending &p : pending_) {
    const ResultEntry &e = p.entry;
    const size_t column = readingColumn + (p.sub ? 2 : 0);
    const size_t pad = std::max(p.sub ? width - 2 : width, (size_t)8);
    std::string name = e.metric;
    if (name.size() < pad) name.resize(pad, ' ');
    out_ << std::string(column, ' ') << name << " : ";
    if (e.status == ResultStatus::Ok) {
      char buf[64];
      snprintf(buf, sizeof buf, "%.2f", e.value);
      out_ << buf;
      if (compareEnabled) {
        auto it = baseline.find(e.key());
        if (it != baseline.end()) {
          const float base = it->second, delta = base != 0.0f ? 100.0f * (e.value - base) / base : 0.0f;
          snprintf(buf, sizeof buf, "  (was %.2f, %c%.1f%%)", base, delta >= 0.0f ? '+' : '-', delta < 0.0f ? -delta : delta);
          out_ << buf;
        }
      }
    } else {
      out_ << "[" << statusLabel(e.status) << "] " << e.reason;
    }
    out_ << "\n";
    // the reading's note below it, flush with the value column
    if (describe_ && !e.metricDescription.empty()) writeWrapped(out_, column + pad + 3, e.metricDescription);
  }
  pending_.clear();
  out_.flush();
}

void LoggerText::onEvent(const LogEvent &e) {
  const std::string propPad((deviceSteps_ + 1) * 2, ' ');
  switch (e.kind) {
    case LogEvent::Kind::BackendBegin:
      out_ << "Backend: " << e.backend << "\n";
      break;
    case LogEvent::Kind::DeviceBegin: {
      deviceSteps_ = e.showPlatformLine ? 2 : 1;
      if (e.showPlatformLine) {
        out_ << "  Platform";
        if (e.platformIndex >= 0) out_ << " " << e.platformIndex;
        out_ << ": " << e.platform << "\n";
      }
      out_ << std::string(deviceSteps_ * 2, ' ') << "Device";
      if (e.deviceIndex >= 0) out_ << " " << e.deviceIndex;
      out_ << ": " << e.device << "\n";
      const std::string pad((deviceSteps_ + 1) * 2, ' ');
      auto prop = [&](std::string key, const std::string &value) {
        if (key.size() < 17) key.resize(17, ' ');
        out_ << pad << key << ": " << value << "\n";
      };
      if (!e.driver.empty()) prop("Driver version", e.driver);
      for (const DeviceProp &p : e.props) prop(p.key, p.value);
      break;
    }
    case LogEvent::Kind::TestBegin: {
      flush();
      std::string unit = e.unit;
      for (char &c : unit) c = (char)toupper((unsigned char)c);
      out_ << "\n" << propPad << e.testDisplay;
      if (!unit.empty()) out_ << " (" << unit << ")";
      out_ << "\n";
      if (describe_ && !e.testDescription.empty()) {
        writeWrapped(out_, (deviceSteps_ + 2) * 2, e.testDescription);
        out_ << "\n";
      }
      break;
    }
    case LogEvent::Kind::Metric:
      pending_.push_back({e.entry, e.subMetric});
      break;
    case LogEvent::Kind::TestSkippedAll:
      out_ << std::string((deviceSteps_ + 2) * 2, ' ') << "[" << statusLabel(e.status) << "] " << e.reason << "\n";
      break;
    case LogEvent::Kind::TestEnd:
      flush();
      break;
    case LogEvent::Kind::DeviceEnd:
      flush();
      out_ << "\n";
      break;
    case LogEvent::Kind::BackendEnd:
      out_.flush();
      break;
    case LogEvent::Kind::Note:
      out_ << e.message;
      if (e.message.empty() || e.message.back() != '\n') out_ << "\n";
      break;
  }
}
