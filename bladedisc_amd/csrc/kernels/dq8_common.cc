// Thread-local error slot and library-level queries of the gfx950 kernel library.
#include "dq8_common.h"

#include "disc_q8.h"

namespace dq8 {
namespace {
thread_local std::string g_last_error;
}

int fail(const std::string& msg) {
  g_last_error = msg;
  return 1;
}

void clear_error() { g_last_error.clear(); }

}  // namespace dq8

extern "C" const char* dq8_last_error(void) { return dq8::g_last_error.c_str(); }

extern "C" int dq8_version(void) { return 100; }

extern "C" int dq8_device_info(int* compute_units, int* lds_bytes_per_cu,
                               int* clock_khz) {
  dq8::clear_error();
  int dev = 0;
  DQ8_HIP(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  DQ8_HIP(hipGetDeviceProperties(&prop, dev));
  if (compute_units) *compute_units = prop.multiProcessorCount;
  if (lds_bytes_per_cu) *lds_bytes_per_cu = (int)prop.maxSharedMemoryPerMultiProcessor;
  if (clock_khz) *clock_khz = prop.clockRate;
  return 0;
}
