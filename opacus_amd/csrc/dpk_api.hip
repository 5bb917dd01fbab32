// Error reporting and device queries of the dpk C ABI.
#include <stdarg.h>
#include <stdio.h>

#include "dpk_common.h"

static thread_local char g_last_error[512] = "";

int dpk_fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

extern "C" int dpk_abi_version(void) { return DPK_ABI_VERSION; }

extern "C" const char* dpk_last_error(void) { return g_last_error; }

extern "C" int dpk_device_cus(void) {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return dpk_fail(DPK_E_LAUNCH, "dpk_device_cus: no HIP device");
  if (dev < 0 || dev >= 64) dev = 0;
  if (cached[dev] == 0) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
      return dpk_fail(DPK_E_LAUNCH, "dpk_device_cus: attribute query failed");
    cached[dev] = cus;
  }
  return cached[dev];
}
