// Shared host-side helpers of the gfx950 kernel library: error reporting and
// launch-argument checks.  Device code lives in the .hip files.
#ifndef DQ8_COMMON_H_
#define DQ8_COMMON_H_

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>
#include <cstdio>
#include <string>

namespace dq8 {

// Records `msg` as the calling thread's last error and returns a non-zero status.
int fail(const std::string& msg);
void clear_error();

inline int check_hip(hipError_t e, const char* what) {
  if (e == hipSuccess) return 0;
  // reported through the status; do not leave it in the thread's HIP error state as well,
  // where the caller's framework would find it at its next GPU call
  (void)hipGetLastError();
  return fail(std::string(what) + ": " + hipGetErrorString(e));
}

inline bool aligned(const void* p, size_t a) {
  return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0;
}

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// number of compute units of the current device (cached; 256 when no device answers)
int compute_units();

// Dynamic LDS above the default limit has to be allowed per kernel and per device.  `done`
// is the kernel's bit set of devices (by ordinal) on which that has happened; two threads
// racing on the first launch both set the attribute, which is harmless.
inline int allow_dynamic_lds(const void* kernel, int bytes, std::atomic<uint64_t>* done) {
  int dev = 0;
  if (int s = check_hip(hipGetDevice(&dev), "hipGetDevice")) return s;
  const uint64_t bit = 1ull << (dev & 63);
  if (done->load(std::memory_order_acquire) & bit) return 0;
  if (int s = check_hip(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                            bytes),
                        "hipFuncSetAttribute(MaxDynamicSharedMemorySize)"))
    return s;
  done->fetch_or(bit, std::memory_order_release);
  return 0;
}

}  // namespace dq8

#define DQ8_HIP(expr)                                   \
  do {                                                  \
    if (int _s = ::dq8::check_hip((expr), #expr)) return _s; \
  } while (0)

#define DQ8_REQUIRE(cond, msg)                 \
  do {                                         \
    if (!(cond)) return ::dq8::fail(msg);      \
  } while (0)

#endif  // DQ8_COMMON_H_
