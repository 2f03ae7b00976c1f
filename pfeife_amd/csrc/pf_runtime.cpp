// Library state of libpfeife_hip.so: per-thread error text, version, device check.
#include <stdarg.h>
#include <string.h>

#include "pf_common.h"

#define PF_ABI_VERSION 2

static thread_local char g_err[512] = "";

void pf_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

extern "C" const char* pf_last_error(void) { return g_err; }

extern "C" int pf_version(void) { return PF_ABI_VERSION; }

extern "C" int pf_init(int device) {
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess || n <= 0) {
    pf_set_error("pf_init: no HIP device (%s)", e == hipSuccess ? "count is 0" : hipGetErrorString(e));
    return PF_ERR_HIP;
  }
  PF_REQUIRE(device >= 0 && device < n, "pf_init: device %d outside [0, %d)", device, n);
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, device);
  if (e != hipSuccess) {
    pf_set_error("pf_init: hipGetDeviceProperties: %s", hipGetErrorString(e));
    return PF_ERR_HIP;
  }
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
    pf_set_error("pf_init: device %d is %s; this library carries gfx950 code only", device, prop.gcnArchName);
    return PF_ERR_UNSUPPORTED;
  }
  e = hipSetDevice(device);
  if (e != hipSuccess) {
    pf_set_error("pf_init: hipSetDevice: %s", hipGetErrorString(e));
    return PF_ERR_HIP;
  }
  return PF_OK;
}
