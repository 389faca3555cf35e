// Shared host-side helpers of the gfx950 kernel library: error reporting and
// launch-argument checks.  Device code lives in the .hip files.
#ifndef DQ8_COMMON_H_
#define DQ8_COMMON_H_

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <string>

namespace dq8 {

// Records `msg` as the calling thread's last error and returns a non-zero status.
int fail(const std::string& msg);
void clear_error();

inline int check_hip(hipError_t e, const char* what) {
  if (e == hipSuccess) return 0;
  return fail(std::string(what) + ": " + hipGetErrorString(e));
}

inline bool aligned(const void* p, size_t a) {
  return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0;
}

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

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
