// Device inventory a backend reports for --list-devices and for the GUI's backend catalog.
// Field set of the reference's include/common/inventory.h:14-41.
#pragma once
#include <cstdint>
#include <iosfwd>
#include <string>
#include <vector>

struct InventoryDevice {
  int index = -1;
  std::string name, typeStr, driverVersion, apiVersion;
  unsigned numComputeUnits = 0, maxClockMHz = 0;
  std::uint64_t globalMemBytes = 0, maxAllocBytes = 0;
  bool hasFp16 = false, hasFp64 = false;
};
struct InventoryPlatform {
  int index = -1;
  std::string name;
  std::vector<InventoryDevice> devices;
};
struct BackendInventory {
  std::string backend;
  bool available = false;
  std::vector<InventoryPlatform> platforms;
};
