// Thread-local error message slot and the small query entry points of the C ABI.
#include "fo_common.h"

namespace {
thread_local char g_error[512] = "";
}

namespace fo {
void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}
}  // namespace fo

extern "C" const char* fo_last_error(void) { return g_error; }

extern "C" int fo_abi_version(void) { return FO_ABI_VERSION; }

extern "C" int fo_num_cu(void) {
  // asked on every launch: the count of a device is looked up once
  static std::atomic<int> cached[64] = {};
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (dev >= 0 && dev < 64 && (n = cached[dev].load(std::memory_order_relaxed)) > 0) return n;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
  if (dev >= 0 && dev < 64) cached[dev].store(n, std::memory_order_relaxed);
  return n;
}
