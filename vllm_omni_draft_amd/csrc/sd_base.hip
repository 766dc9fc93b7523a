// What every part of the library needs: the per-thread error text, the version, the device
// query, and the hipGraph capture helpers with which a step of fixed shape replays as one launch.  (Its own object, so that a build of a subset of the library links without the rest.)
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


// ------------------------------------------------------------------ stream capture
struct sd_graph {
  hipGraph_t graph;
  hipGraphExec_t exec;
};

extern "C" int sd_graph_begin(sd_stream_t stream) {
  hipError_t e = hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeRelaxed);
  if (e != hipSuccess) {
    sd_set_error("sd_graph_begin: %s", hipGetErrorString(e));
    return SD_ERR_HIP;
  }
  return SD_OK;
}

extern "C" int sd_graph_end(sd_stream_t stream, sd_graph** out) {
  SD_REQUIRE(out, SD_ERR_INVALID, "sd_graph_end: null out");
  hipGraph_t g = nullptr;
  hipError_t e = hipStreamEndCapture((hipStream_t)stream, &g);
  if (e != hipSuccess || !g) {
    sd_set_error("sd_graph_end: capture failed: %s", hipGetErrorString(e));
    return SD_ERR_HIP;
  }
  hipGraphExec_t ex = nullptr;
  e = hipGraphInstantiate(&ex, g, nullptr, nullptr, 0);
  if (e != hipSuccess) {
    (void)hipGraphDestroy(g);
    sd_set_error("sd_graph_end: instantiate failed: %s", hipGetErrorString(e));
    return SD_ERR_HIP;
  }
  *out = new sd_graph{g, ex};
  return SD_OK;
}

extern "C" int sd_graph_launch(sd_graph* g, sd_stream_t stream) {
  SD_REQUIRE(g, SD_ERR_INVALID, "sd_graph_launch: null graph");
  hipError_t e = hipGraphLaunch(g->exec, (hipStream_t)stream);
  if (e != hipSuccess) {
    sd_set_error("sd_graph_launch: %s", hipGetErrorString(e));
    return SD_ERR_HIP;
  }
  return SD_OK;
}

extern "C" void sd_graph_destroy(sd_graph* g) {
  if (!g) return;
  (void)hipGraphExecDestroy(g->exec);   // nothing to report to: the handle is gone either way
  (void)hipGraphDestroy(g->graph);
  delete g;
}

