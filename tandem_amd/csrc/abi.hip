// Library-level entry points: last error, ABI version, device facts.

#include <cstring>

#include "common.h"

namespace tandem_hip {

namespace {
thread_local std::string g_last_error;
}

void set_last_error(const std::string& message) { g_last_error = message; }

}  // namespace tandem_hip

using namespace tandem_hip;

extern "C" {

const char* tdm_last_error(void) { return g_last_error.c_str(); }

int tdm_abi_version(void) { return 1; }

int tdm_device_info(int device, char* name, int name_len, int* compute_units, int64_t* total_bytes) {
  return guard([&] {
    hipDeviceProp_t prop;
    check_hip(hipGetDeviceProperties(&prop, device), "hipGetDeviceProperties");
    if (name != nullptr && name_len > 0) {
      std::strncpy(name, prop.name, static_cast<size_t>(name_len) - 1);
      name[name_len - 1] = '\0';
    }
    if (compute_units != nullptr) *compute_units = prop.multiProcessorCount;
    if (total_bytes != nullptr) *total_bytes = static_cast<int64_t>(prop.totalGlobalMem);
  });
}

}  // extern "C"
