// Result rows and their three dump formats (XML, JSON, CSV; format_version 2).
// Row identity, field set and file grammar follow the reference
// (include/common/result_store.h:42-149, src/common/result_store.cpp:120-448), so files
// written here load in the reference's CLI and GUI and vice versa.
#pragma once
#include <map>
#include <string>
#include <vector>
#include "clpeak_types.h"

#define CLPEAK_RESULT_FORMAT_VERSION 2
#define CLPEAK_MI355_VERSION "2.0.16-mi355"

struct ResultEntry {
  std::string backend, platform, device, driver;
  std::string category, test, metric, unit;
  ResultStatus status = ResultStatus::Ok;
  float value = 0.0f;            // every value is a float, printed with 4 decimals
  std::string reason;            // why, when status != Ok
  std::string display;           // human-readable test name
  std::string description;       // what the test measures
  std::string metricDescription; // what this one reading means

  // backend/platform/device/category/test/metric: the key --compare and the GUI match on.
  std::string key() const {
    return backend + "/" + platform + "/" + device + "/" + category + "/" + test + "/" + metric;
  }
};

struct DeviceProp { std::string key, value; };

struct DeviceInfo {
  std::string backend, platform, device, driver;
  std::vector<DeviceProp> props;
  std::string key() const { return backend + "/" + platform + "/" + device + "/" + driver; }
};

typedef std::vector<ResultEntry> ResultStore;
typedef std::vector<DeviceInfo> DeviceInfoStore;
typedef std::map<std::string, float> BaselineMap;

BaselineMap buildBaselineMap(const ResultStore &store);   // Ok rows only

bool saveXml(const ResultStore &store, const std::string &filename, const DeviceInfoStore &devices = {});
bool saveJson(const ResultStore &store, const std::string &filename, const DeviceInfoStore &devices = {});
bool saveCsv(const ResultStore &store, const std::string &filename);
std::string resultsToJson(const ResultStore &store, const DeviceInfoStore &devices = {});

// Loaders for files written by the functions above (or by the reference).  A file whose
// format_version is not 2 yields an empty store.
ResultStore loadXml(const std::string &filename, DeviceInfoStore *devices = nullptr);
ResultStore loadJson(const std::string &filename, DeviceInfoStore *devices = nullptr);
ResultStore loadCsv(const std::string &filename);
ResultStore loadResultFile(const std::string &filename, DeviceInfoStore *devices = nullptr);

std::string jsonEscape(const std::string &s);
std::string xmlEscape(const std::string &s);
std::string formatValue(float v);   // classic locale, fixed, 4 decimals
