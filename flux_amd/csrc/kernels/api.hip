// Library-wide pieces of the C-ABI: version, thread-local error text, device query.
#include "common.hpp"

namespace fluxmi {
namespace {
thread_local char g_last_error[512] = "";
}

void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
}
}  // namespace fluxmi

extern "C" int fluxmi_version(void) { return 111; }

extern "C" const char *fluxmi_last_error(void) { return fluxmi::g_last_error; }

extern "C" int fluxmi_device_cu_count(void) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return -1;
  static std::atomic<int> cached[64];  // CU count per device id, 0 = not queried yet
  if (dev >= 0 && dev < 64) {
    const int c = cached[dev].load(std::memory_order_relaxed);
    if (c > 0) return c;
  }
  int cus = 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return -1;
  if (dev >= 0 && dev < 64) cached[dev].store(cus, std::memory_order_relaxed);
  return cus;
}
