// Error reporting and device queries shared by all entry points.
#include "common.h"

#include <stdarg.h>
#include <string.h>

static thread_local char g_last_error[1024] = "";

void lmsf_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
}

extern "C" const char* lmsf_last_error() { return g_last_error; }

// ABI version of the entry points; the Python side refuses a library that reports another.
extern "C" int lmsf_abi_version() { return 23; }

// Compute units of the current device (asked once per device; 0 if the device cannot be asked).
int lmsf_compute_units() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) n = 0;
    cached[dev] = n;
  }
  return cached[dev];
}

// Name of the architecture the current device reports, e.g. "gfx950:sramecc+:xnack-".
extern "C" int lmsf_device_arch(char* out, int cap) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    lmsf_set_error("hipGetDevice failed");
    return 1;
  }
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, dev) != hipSuccess) {
    lmsf_set_error("hipGetDeviceProperties failed");
    return 1;
  }
  strncpy(out, prop.gcnArchName, cap - 1);
  out[cap - 1] = 0;
  return 0;
}
