// Error reporting and device queries shared by all entry points.
#include "common.h"

#include <cstring>

namespace uvmi {
static thread_local char g_err[512] = "";
void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}
}  // namespace uvmi

extern "C" int uvmi_version(void) { return UVMI_ABI_VERSION; }
extern "C" const char* uvmi_last_error(void) { return uvmi::g_err; }

extern "C" int uvmi_device_cus(void) {
  static thread_local int cached_dev = -1, cached_cus = 0;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    uvmi::set_error("uvmi_device_cus: hipGetDevice failed");
    return UVMI_EHIP;
  }
  if (dev != cached_dev) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
      uvmi::set_error("uvmi_device_cus: hipDeviceGetAttribute failed");
      return UVMI_EHIP;
    }
    cached_dev = dev;
    cached_cus = n;
  }
  return cached_cus;
}
