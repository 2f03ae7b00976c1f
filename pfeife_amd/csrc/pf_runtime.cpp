// Library state of libpfeife_hip.so: per-thread error text, version, device check.
#include <stdarg.h>
#include <string.h>

#include "pf_common.h"

int pf_norm_init_device();   // pf_norm.hip

#define PF_ABI_VERSION 4

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
  return pf_norm_init_device();   // device addresses of the library's built-in scratch arrays
}

// ---- hipGraph capture of launch lists ---------------------------------------------
// A stage job is a fixed list of kernel launches on fixed buffers, so it is captured once
// (stream capture around the ordinary entry points) and replayed with one call per job.
extern "C" int pf_graph_capture_begin(void* stream) {
  PF_REQUIRE(stream != nullptr, "pf_graph_capture_begin: the legacy default stream cannot be captured");
  hipError_t e = hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeRelaxed);
  if (e != hipSuccess) {
    pf_set_error("pf_graph_capture_begin: %s", hipGetErrorString(e));
    return PF_ERR_HIP;
  }
  return PF_OK;
}

extern "C" int pf_graph_capture_end(void* stream, void** graph_exec_out) {
  PF_REQUIRE(stream != nullptr && graph_exec_out != nullptr, "pf_graph_capture_end: bad arguments");
  hipGraph_t graph = nullptr;
  hipError_t e = hipStreamEndCapture((hipStream_t)stream, &graph);
  if (e != hipSuccess || graph == nullptr) {
    pf_set_error("pf_graph_capture_end: %s", hipGetErrorString(e));
    return PF_ERR_HIP;
  }
  hipGraphExec_t exec = nullptr;
  e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  if (e != hipSuccess) {
    pf_set_error("pf_graph_capture_end: instantiate: %s", hipGetErrorString(e));
    return PF_ERR_HIP;
  }
  *graph_exec_out = (void*)exec;
  return PF_OK;
}

extern "C" int pf_graph_launch(void* graph_exec, void* stream) {
  PF_REQUIRE(graph_exec != nullptr, "pf_graph_launch: null graph");
  hipError_t e = hipGraphLaunch((hipGraphExec_t)graph_exec, (hipStream_t)stream);
  if (e != hipSuccess) {
    pf_set_error("pf_graph_launch: %s", hipGetErrorString(e));
    return PF_ERR_HIP;
  }
  return PF_OK;
}

extern "C" int pf_graph_destroy(void* graph_exec) {
  if (graph_exec) (void)hipGraphExecDestroy((hipGraphExec_t)graph_exec);
  return PF_OK;
}
