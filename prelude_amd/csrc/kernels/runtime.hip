// Host-side error channel shared by all entry points, and device queries.
#include "common.h"
#include "api.h"

#include <stdarg.h>
#include <stdio.h>

namespace {
thread_local char g_error[1024] = "";
}

extern "C" const char* pa_last_error() { return g_error; }

namespace pa {

int fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return 1;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail("%s: launch failed: %s", what, hipGetErrorString(e));
  return 0;
}

}  // namespace pa

// Name of the architecture the current device reports (e.g. "gfx950:sramecc+:xnack-").
extern "C" int pa_device_arch(char* out, int cap) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return pa::fail("hipGetDevice: %s", hipGetErrorString(e));
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) return pa::fail("hipGetDeviceProperties: %s", hipGetErrorString(e));
  snprintf(out, cap, "%s", prop.gcnArchName);
  return 0;
}

extern "C" int pa_num_compute_units() {
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
  return n;
}
