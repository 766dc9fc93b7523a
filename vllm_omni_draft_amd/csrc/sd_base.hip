// What every part of the library needs: the per-thread error text, the version and the device
// query.  (Its own object, so that a build of a subset of the library links without the rest.)
#include <stdarg.h>
#include <string.h>

#include "sd_common.h"

namespace {
thread_local char g_err[512] = "";
}

void sd_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

extern "C" int sd_version(void) { return 100; }

extern "C" int sd_last_error(char* buf, size_t n) {
  if (!buf || n == 0) return SD_ERR_INVALID;
  strncpy(buf, g_err, n - 1);
  buf[n - 1] = '\0';
  return SD_OK;
}

extern "C" int sd_device_info(int* cu_count, char* name, size_t n) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    sd_set_error("sd_device_info: hipGetDevice: %s", hipGetErrorString(e));
    return SD_ERR_HIP;
  }
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) {
    sd_set_error("sd_device_info: hipGetDeviceProperties: %s", hipGetErrorString(e));
    return SD_ERR_HIP;
  }
  if (cu_count) *cu_count = prop.multiProcessorCount;
  if (name && n) {
    strncpy(name, prop.gcnArchName, n - 1);
    name[n - 1] = '\0';
  }
  return SD_OK;
}

