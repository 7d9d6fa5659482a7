#include "results.h"
#include <cstdio>
#include <cstring>
#include <fstream>
#include <iostream>
#include <locale>
#include <sstream>

// ---- enum <-> text ------------------------------------------------------------------
namespace {
const struct { Category c; const char *name; } kCategories[] = {
    {Category::FpCompute, "fp_compute"}, {Category::IntCompute, "int_compute"}, {Category::Crypto, "crypto"},
    {Category::String, "string"},        {Category::Bandwidth, "bandwidth"},    {Category::Latency, "latency"}};
const struct { ResultStatus s; const char *name; } kStatuses[] = {
    {ResultStatus::Ok, "ok"}, {ResultStatus::Unsupported, "unsupported"}, {ResultStatus::Skipped, "skipped"},
    {ResultStatus::Error, "error"}};
}  // namespace

const char *categoryString(Category c) {
  for (const auto &e : kCategories) if (e.c == c) return e.name;
  return "";
}
const char *statusString(ResultStatus s) {
  for (const auto &e : kStatuses) if (e.s == s) return e.name;
  return "ok";
}
Category categoryFromString(const std::string &s) {
  for (const auto &e : kCategories) if (s == e.name) return e.c;
  return Category::Unknown;
}
ResultStatus statusFromString(const std::string &s) {
  for (const auto &e : kStatuses) if (s == e.name) return e.s;
  return ResultStatus::Ok;
}
Category categoryFromUnit(const std::string &u) {
  if (u == "gflops" || u == "tflops") return Category::FpCompute;
  if (u == "gops" || u == "tops") return Category::IntCompute;
  if (u == "gbps") return Category::Bandwidth;
  if (u == "us") return Category::Latency;
  return Category::Unknown;
}

BaselineMap buildBaselineMap(const ResultStore &store) {
  BaselineMap m;
  for (const auto &e : store)
    if (e.status == ResultStatus::Ok) m[e.key()] = e.value;
  return m;
}

// ---- escaping and number formatting ------------------------------------------------------
std::string jsonEscape(const std::string &s) {
  std::string o;
  for (unsigned char ch : s) {
    switch (ch) {
      case '"': o += "\\\""; break;
      case '\\': o += "\\\\"; break;
      case '\n': o += "\\n"; break;
      case '\r': o += "\\r"; break;
      case '\t': o += "\\t"; break;
      default:
        if (ch < 0x20) { char b[8]; snprintf(b, sizeof b, "\\u%04x", ch); o += b; }
        else o += (char)ch;
    }
  }
  return o;
}

std::string xmlEscape(const std::string &s) {
  std::string o;
  for (char ch : s) {
    switch (ch) {
      case '&': o += "&amp;"; break;
      case '<': o += "&lt;"; break;
      case '>': o += "&gt;"; break;
      case '"': o += "&quot;"; break;
      case '\'': o += "&apos;"; break;
      default: o += ch;
    }
  }
  return o;
}

static std::string xmlUnescape(const std::string &s) {
  static const struct { const char *ent; char ch; } ents[] = {
      {"&amp;", '&'}, {"&lt;", '<'}, {"&gt;", '>'}, {"&quot;", '"'}, {"&apos;", '\''}};
  std::string o;
  for (size_t i = 0; i < s.size();) {
    bool hit = false;
    if (s[i] == '&')
      for (const auto &e : ents) {
        const size_t n = strlen(e.ent);
        if (s.compare(i, n, e.ent) == 0) { o += e.ch; i += n; hit = true; break; }
      }
    if (!hit) o += s[i++];
  }
  return o;
}

std::string formatValue(float v) {
  std::ostringstream ss;
  ss.imbue(std::locale::classic());
  ss.setf(std::ios::fixed);
  ss.precision(4);
  ss << v;
  return ss.str();
}

static bool parseValue(const std::string &s, float &out) {
  std::istringstream is(s);
  is.imbue(std::locale::classic());
  float v;
  if (!(is >> v)) return false;
  out = v;
  return true;
}

// ---- XML ---------------------------------------------------------------------------------------
// <clpeak format_version clpeak_version os> <run backend platform device driver> <prop name value/>*
//   <category name> <test name [display] unit [description]> <metric name [info]>value</metric> |
//   <metric name [info] status reason/>
// Rows arrive grouped run -> category -> test (the logger emits them in run order), so one pass
// that opens and closes elements on every change of the grouping keys is enough.
bool saveXml(const ResultStore &store, const std::string &filename, const DeviceInfoStore &devices) {
  std::ofstream f(filename);
  if (!f) {
    std::cerr << "clpeak: cannot open XML output file: " << filename << "\n";
    return false;
  }
  f.imbue(std::locale::classic());
  f << "<?xml version=\"1.0\" encoding=\"utf-8\"?>\n"
    << "<clpeak format_version=\"" << CLPEAK_RESULT_FORMAT_VERSION << "\" clpeak_version=\""
    << xmlEscape(CLPEAK_MI355_VERSION) << "\" os=\"Linux x64\">\n";
  std::string run, cat, test;          // keys of the currently open elements ("" = closed)
  auto close = [&](int depth) {        // close everything at `depth` and below: 3 test, 2 category, 1 run
    if (depth <= 3 && !test.empty()) { f << "      </test>\n"; test.clear(); }
    if (depth <= 2 && !cat.empty()) { f << "    </category>\n"; cat.clear(); }
    if (depth <= 1 && !run.empty()) { f << "  </run>\n"; run.clear(); }
  };
  for (const ResultEntry &e : store) {
    const std::string rkey = e.backend + "/" + e.platform + "/" + e.device + "/" + e.driver;
    if (rkey != run) {
      close(1);
      run = rkey;
      f << "  <run backend=\"" << xmlEscape(e.backend) << "\" platform=\"" << xmlEscape(e.platform)
        << "\" device=\"" << xmlEscape(e.device) << "\" driver=\"" << xmlEscape(e.driver) << "\">\n";
      for (const DeviceInfo &d : devices)
        if (d.key() == rkey)
          for (const DeviceProp &p : d.props)
            f << "    <prop name=\"" << xmlEscape(p.key) << "\" value=\"" << xmlEscape(p.value) << "\"/>\n";
    }
    if (e.category != cat || cat.empty()) {
      close(2);
      cat = e.category.empty() ? std::string(" ") : e.category;
      f << "    <category name=\"" << xmlEscape(e.category) << "\">\n";
    }
    const std::string tkey = e.test + "\x1f" + e.unit;
    if (tkey != test) {
      close(3);
      test = tkey;
      f << "      <test name=\"" << xmlEscape(e.test) << "\"";
      if (!e.display.empty()) f << " display=\"" << xmlEscape(e.display) << "\"";
      f << " unit=\"" << xmlEscape(e.unit) << "\"";
      if (!e.description.empty()) f << " description=\"" << xmlEscape(e.description) << "\"";
      f << ">\n";
    }
    f << "        <metric name=\"" << xmlEscape(e.metric) << "\"";
    if (!e.metricDescription.empty()) f << " info=\"" << xmlEscape(e.metricDescription) << "\"";
    if (e.status == ResultStatus::Ok) f << ">" << formatValue(e.value) << "</metric>\n";
    else f << " status=\"" << statusString(e.status) << "\" reason=\"" << xmlEscape(e.reason) << "\"/>\n";
  }
  close(1);
  f << "</clpeak>\n";
  return f.good();
}

// attribute `name` of the element text `tag` ("" when absent)
static std::string xmlAttr(const std::string &tag, const std::string &name) {
  const std::string pat = " " + name + "=\"";
  const size_t a = tag.find(pat);
  if (a == std::string::npos) return "";
  const size_t b = tag.find('"', a + pat.size());
  if (b == std::string::npos) return "";
  return xmlUnescape(tag.substr(a + pat.size(), b - a - pat.size()));
}

ResultStore loadXml(const std::string &filename, DeviceInfoStore *devices) {
  ResultStore out;
  std::ifstream f(filename);
  if (!f) return out;
  std::string line;
  ResultEntry cur;   // carries the run / category / test context
  bool versionOk = false;
  while (std::getline(f, line)) {
    const size_t lt = line.find('<');
    if (lt == std::string::npos) continue;
    const std::string t = line.substr(lt);
    if (t.compare(0, 7, "<clpeak") == 0) {
      versionOk = xmlAttr(t, "format_version") == std::to_string(CLPEAK_RESULT_FORMAT_VERSION);
      if (!versionOk) {
        std::cerr << "clpeak: " << filename << ": unsupported format_version\n";
        return ResultStore();
      }
    } else if (t.compare(0, 5, "<run ") == 0) {
      cur = ResultEntry();
      cur.backend = xmlAttr(t, "backend"); cur.platform = xmlAttr(t, "platform");
      cur.device = xmlAttr(t, "device"); cur.driver = xmlAttr(t, "driver");
      if (devices) {
        DeviceInfo d;
        d.backend = cur.backend; d.platform = cur.platform; d.device = cur.device; d.driver = cur.driver;
        devices->push_back(d);
      }
    } else if (t.compare(0, 6, "<prop ") == 0) {
      if (devices && !devices->empty()) devices->back().props.push_back({xmlAttr(t, "name"), xmlAttr(t, "value")});
    } else if (t.compare(0, 10, "<category ") == 0) {
      cur.category = xmlAttr(t, "name");
    } else if (t.compare(0, 6, "<test ") == 0) {
      cur.test = xmlAttr(t, "name"); cur.unit = xmlAttr(t, "unit");
      cur.display = xmlAttr(t, "display"); cur.description = xmlAttr(t, "description");
    } else if (t.compare(0, 8, "<metric ") == 0) {
      ResultEntry e = cur;
      e.metric = xmlAttr(t, "name");
      e.metricDescription = xmlAttr(t, "info");
      const std::string st = xmlAttr(t, "status");
      if (!st.empty()) {
        e.status = statusFromString(st);
        e.reason = xmlAttr(t, "reason");
      } else {
        const size_t gt = t.find('>');
        if (gt == std::string::npos || !parseValue(t.substr(gt + 1), e.value)) continue;
      }
      out.push_back(e);
    }
  }
  if (!versionOk) return ResultStore();
  return out;
}

// ---- JSON ----------------------------------------------------------------------------------------
// {"format_version":2,"clpeak_version":"..","os":"..",["devices":[ one object per line ],]"entries":[
//  one object per line ]}
static void jsonField(std::ostream &f, const char *k, const std::string &v, bool comma = true) {
  f << "\"" << k << "\":\"" << jsonEscape(v) << "\"";
  if (comma) f << ",";
}

static void writeJson(std::ostream &f, const ResultStore &store, const DeviceInfoStore &devices) {
  f.imbue(std::locale::classic());
  f << "{\"format_version\":" << CLPEAK_RESULT_FORMAT_VERSION << ",\"clpeak_version\":\""
    << jsonEscape(CLPEAK_MI355_VERSION) << "\",\"os\":\"Linux x64\"";
  if (!devices.empty()) {
    f << ",\"devices\":[\n";
    for (size_t i = 0; i < devices.size(); i++) {
      const DeviceInfo &d = devices[i];
      f << "{";
      jsonField(f, "backend", d.backend); jsonField(f, "platform", d.platform);
      jsonField(f, "device", d.device); jsonField(f, "driver", d.driver);
      f << "\"props\":[";
      for (size_t j = 0; j < d.props.size(); j++)
        f << (j ? "," : "") << "{\"k\":\"" << jsonEscape(d.props[j].key) << "\",\"v\":\""
          << jsonEscape(d.props[j].value) << "\"}";
      f << "]}" << (i + 1 < devices.size() ? "," : "") << "\n";
    }
    f << "]";
  }
  f << ",\"entries\":[\n";
  for (size_t i = 0; i < store.size(); i++) {
    const ResultEntry &e = store[i];
    f << "{";
    jsonField(f, "backend", e.backend); jsonField(f, "platform", e.platform); jsonField(f, "device", e.device);
    jsonField(f, "driver", e.driver); jsonField(f, "category", e.category); jsonField(f, "test", e.test);
    jsonField(f, "metric", e.metric); jsonField(f, "unit", e.unit, false);
    if (!e.display.empty()) { f << ","; jsonField(f, "display", e.display, false); }
    if (!e.description.empty()) { f << ","; jsonField(f, "description", e.description, false); }
    if (!e.metricDescription.empty()) { f << ","; jsonField(f, "metric_description", e.metricDescription, false); }
    if (e.status == ResultStatus::Ok) f << ",\"value\":" << formatValue(e.value);
    else { f << ",\"status\":\"" << statusString(e.status) << "\","; jsonField(f, "reason", e.reason, false); }
    f << "}" << (i + 1 < store.size() ? "," : "") << "\n";
  }
  f << "]}\n";
}

bool saveJson(const ResultStore &store, const std::string &filename, const DeviceInfoStore &devices) {
  std::ofstream f(filename);
  if (!f) {
    std::cerr << "clpeak: cannot open JSON output file: " << filename << "\n";
    return false;
  }
  writeJson(f, store, devices);
  return f.good();
}

std::string resultsToJson(const ResultStore &store, const DeviceInfoStore &devices) {
  std::ostringstream ss;
  writeJson(ss, store, devices);
  return ss.str();
}

// value of "key":"..." in a one-object line, unescaped ("" when absent)
static std::string jsonStr(const std::string &line, const std::string &key) {
  const std::string pat = "\"" + key + "\":\"";
  const size_t a = line.find(pat);
  if (a == std::string::npos) return "";
  std::string o;
  for (size_t i = a + pat.size(); i < line.size(); i++) {
    const char c = line[i];
    if (c == '"') break;
    if (c == '\\' && i + 1 < line.size()) {
      const char n = line[++i];
      if (n == 'n') o += '\n'; else if (n == 'r') o += '\r'; else if (n == 't') o += '\t';
      else if (n == 'u' && i + 4 < line.size()) { o += (char)strtol(line.substr(i + 1, 4).c_str(), nullptr, 16); i += 4; }
      else o += n;
    } else o += c;
  }
  return o;
}

ResultStore loadJson(const std::string &filename, DeviceInfoStore *devices) {
  ResultStore out;
  std::ifstream f(filename);
  if (!f) return out;
  std::string line;
  bool versionOk = false, inDevices = false;
  while (std::getline(f, line)) {
    if (line.find("\"format_version\":") != std::string::npos) {
      const size_t a = line.find("\"format_version\":") + 17;
      versionOk = atoi(line.c_str() + a) == CLPEAK_RESULT_FORMAT_VERSION;
      if (!versionOk) {
        std::cerr << "clpeak: " << filename << ": unsupported format_version\n";
        return ResultStore();
      }
      inDevices = line.find("\"devices\":[") != std::string::npos;
      continue;
    }
    if (line.find("\"entries\":[") != std::string::npos) { inDevices = false; continue; }
    if (line.empty() || line[0] != '{') continue;
    if (inDevices || line.find("\"metric\":") == std::string::npos) {
      if (devices && line.find("\"props\":") != std::string::npos) {
        DeviceInfo d;
        d.backend = jsonStr(line, "backend"); d.platform = jsonStr(line, "platform");
        d.device = jsonStr(line, "device"); d.driver = jsonStr(line, "driver");
        size_t p = line.find("\"props\":[");
        while ((p = line.find("{\"k\":\"", p)) != std::string::npos) {
          const std::string rest = line.substr(p);
          d.props.push_back({jsonStr(rest, "k"), jsonStr(rest, "v")});
          p += 6;
        }
        devices->push_back(d);
      }
      continue;
    }
    ResultEntry e;
    e.backend = jsonStr(line, "backend"); e.platform = jsonStr(line, "platform"); e.device = jsonStr(line, "device");
    e.driver = jsonStr(line, "driver"); e.category = jsonStr(line, "category"); e.test = jsonStr(line, "test");
    e.metric = jsonStr(line, "metric"); e.unit = jsonStr(line, "unit"); e.display = jsonStr(line, "display");
    e.description = jsonStr(line, "description"); e.metricDescription = jsonStr(line, "metric_description");
    e.status = statusFromString(jsonStr(line, "status"));
    if (e.status == ResultStatus::Ok) {
      const size_t v = line.find("\"value\":");
      if (v == std::string::npos || !parseValue(line.substr(v + 8), e.value)) continue;
    } else e.reason = jsonStr(line, "reason");
    out.push_back(e);
  }
  if (!versionOk) return ResultStore();
  return out;
}

// ---- CSV -----------------------------------------------------------------------------------------
// A header row, then one row per measurement; format_version repeats on every row so the file
// describes itself even when a tool drops the header.  Ok rows leave `reason` empty, other rows
// leave `value` empty.
static const char *kCsvHeader =
    "format_version,backend,platform,device,driver,category,test,metric,unit,status,value,reason,display,"
    "description,metric_description";

static std::string csvQuote(const std::string &s) {
  if (s.find_first_of(",\"\n\r") == std::string::npos) return s;
  std::string o = "\"";
  for (char c : s) { if (c == '"') o += '"'; o += c; }
  return o + "\"";
}

bool saveCsv(const ResultStore &store, const std::string &filename) {
  std::ofstream f(filename);
  if (!f) {
    std::cerr << "clpeak: cannot open CSV output file: " << filename << "\n";
    return false;
  }
  f.imbue(std::locale::classic());
  f << kCsvHeader << "\n";
  for (const ResultEntry &e : store) {
    f << CLPEAK_RESULT_FORMAT_VERSION << ",";
    const std::string *head[] = {&e.backend, &e.platform, &e.device, &e.driver, &e.category, &e.test, &e.metric, &e.unit};
    for (const std::string *c : head) f << csvQuote(*c) << ",";
    f << statusString(e.status) << "," << (e.status == ResultStatus::Ok ? formatValue(e.value) : "") << ","
      << csvQuote(e.reason) << "," << csvQuote(e.display) << "," << csvQuote(e.description) << ","
      << csvQuote(e.metricDescription) << "\n";
  }
  return f.good();
}

static std::vector<std::string> csvSplit(const std::string &line) {
  std::vector<std::string> cols(1);
  bool quoted = false;
  for (size_t i = 0; i < line.size(); i++) {
    const char c = line[i];
    if (quoted) {
      if (c == '"' && i + 1 < line.size() && line[i + 1] == '"') { cols.back() += '"'; i++; }
      else if (c == '"') quoted = false;
      else cols.back() += c;
    } else if (c == '"') quoted = true;
    else if (c == ',') cols.emplace_back();
    else cols.back() += c;
  }
  return cols;
}

ResultStore loadCsv(const std::string &filename) {
  ResultStore out;
  std::ifstream f(filename);
  if (!f) return out;
  std::string line;
  while (std::getline(f, line)) {
    if (line.empty() || line.compare(0, 15, "format_version,") == 0) continue;
    const std::vector<std::string> c = csvSplit(line);
    if (c.size() < 12 || atoi(c[0].c_str()) != CLPEAK_RESULT_FORMAT_VERSION) continue;
    ResultEntry e;
    e.backend = c[1]; e.platform = c[2]; e.device = c[3]; e.driver = c[4]; e.category = c[5]; e.test = c[6];
    e.metric = c[7]; e.unit = c[8]; e.status = statusFromString(c[9]); e.reason = c[11];
    if (c.size() > 12) e.display = c[12];
    if (c.size() > 13) e.description = c[13];
    if (c.size() > 14) e.metricDescription = c[14];
    if (e.status == ResultStatus::Ok && !parseValue(c[10], e.value)) continue;
    out.push_back(e);
  }
  return out;
}

ResultStore loadResultFile(const std::string &filename, DeviceInfoStore *devices) {
  const size_t dot = filename.rfind('.');
  const std::string ext = dot == std::string::npos ? "" : filename.substr(dot);
  if (ext == ".csv") return loadCsv(filename);
  if (ext == ".xml") return loadXml(filename, devices);
  return loadJson(filename, devices);
}
