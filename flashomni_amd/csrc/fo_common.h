// Shared host-side helpers of the C-ABI library: error slot, argument checks, launch checks.
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/flashomni_hip.h"

namespace fo {

void set_error(const char* fmt, ...);

inline int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
inline int fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  set_error("%s", buf);
  return code;
}

inline int ceil_div(int64_t a, int64_t b) { return static_cast<int>((a + b - 1) / b); }

}  // namespace fo

#define FO_REQUIRE(cond, ...)                              \
  do {                                                     \
    if (!(cond)) return fo::fail(FO_ERR_INVALID, __VA_ARGS__); \
  } while (0)

#define FO_HIP_CALL(expr)                                                                   \
  do {                                                                                      \
    hipError_t e_ = (expr);                                                                 \
    if (e_ != hipSuccess)                                                                   \
      return fo::fail(FO_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_),    \
                      __FILE__, __LINE__);                                                  \
  } while (0)

#define FO_CHECK_LAUNCH() FO_HIP_CALL(hipGetLastError())
