// Error reporting, device queries and HIP graph capture for the kernel library.
#include "common.h"

#include <stdarg.h>
#include <stdio.h>
#include <string.h>

static thread_local char g_error[1024] = "";

int lrs_fail(const char* fmt, ...) {
  va_list args;
  va_start(args, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, args);
  va_end(args);
  return 1;
}

int lrs_check_launch(const char* what) {
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return lrs_fail("%s: launch failed: %s", what, hipGetErrorString(err));
  return 0;
}

LRS_API const char* lrs_last_error() { return g_error; }

// Writes the architecture name (for example "gfx950:sramecc+:xnack-") of `device` into `out`.
LRS_API int lrs_device_arch(int device, char* out, int out_len, int* compute_units) {
  hipDeviceProp_t prop;
  hipError_t err = hipGetDeviceProperties(&prop, device);
  if (err != hipSuccess) return lrs_fail("hipGetDeviceProperties: %s", hipGetErrorString(err));
  snprintf(out, out_len, "%s", prop.gcnArchName);
  if (compute_units) *compute_units = prop.multiProcessorCount;
  return 0;
}

// ---- HIP graphs: capture whatever is launched on `stream` between begin and end, replay later.
// No memset node may be recorded (clear buffers with fill kernels); the library launches none.
LRS_API int lrs_graph_begin(void* stream) {
  hipError_t err = hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal);
  if (err != hipSuccess) return lrs_fail("hipStreamBeginCapture: %s", hipGetErrorString(err));
  return 0;
}

LRS_API int lrs_graph_end(void* stream, void** exec_out) {
  hipGraph_t graph = nullptr;
  hipError_t err = hipStreamEndCapture((hipStream_t)stream, &graph);
  if (err != hipSuccess) return lrs_fail("hipStreamEndCapture: %s", hipGetErrorString(err));
  hipGraphExec_t exec = nullptr;
  err = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  hipGraphDestroy(graph);
  if (err != hipSuccess) return lrs_fail("hipGraphInstantiate: %s", hipGetErrorString(err));
  *exec_out = (void*)exec;
  return 0;
}

LRS_API int lrs_graph_launch(void* exec, void* stream) {
  hipError_t err = hipGraphLaunch((hipGraphExec_t)exec, (hipStream_t)stream);
  if (err != hipSuccess) return lrs_fail("hipGraphLaunch: %s", hipGetErrorString(err));
  return 0;
}

LRS_API int lrs_graph_destroy(void* exec) {
  if (exec) hipGraphExecDestroy((hipGraphExec_t)exec);
  return 0;
}

// Asynchronous copy of step metadata from pinned host memory to the device.
LRS_API int lrs_copy_h2d(void* dst, const void* src, int64_t bytes, void* stream) {
  hipError_t err = hipMemcpyAsync(dst, src, (size_t)bytes, hipMemcpyHostToDevice, (hipStream_t)stream);
  if (err != hipSuccess) return lrs_fail("hipMemcpyAsync: %s", hipGetErrorString(err));
  return 0;
}
