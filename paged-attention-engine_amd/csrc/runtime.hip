// Error reporting shared by the entry points, and a query of the device's name.
#include "common.h"
#include "api.h"
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

static thread_local char g_error[512] = "";

extern "C" const char* pae_last_error() { return g_error; }

int pae_fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return -1;
}

int pae_check_launch(const char* what) {
  const hipError_t err = hipGetLastError();
  if (err == hipSuccess) return 0;
  snprintf(g_error, sizeof(g_error), "%s: launch failed: %s", what, hipGetErrorString(err));
  return -2;
}

extern "C" int pae_device_arch(char* out, int cap) {
  int dev = 0;
  hipDeviceProp_t prop;
  if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess)
    return pae_fail("no HIP device");
  strncpy(out, prop.gcnArchName, cap - 1);
  out[cap - 1] = 0;
  return 0;
}
