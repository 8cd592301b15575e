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

// The address under which kernels see pinned host memory (hipHostMalloc): results of a few bytes
// (the chosen tokens) are written there directly, which spares a copy back and its latency.
LRS_API int lrs_host_device_pointer(void* host, void** device) {
  hipError_t err = hipHostGetDevicePointer(device, host, 0);
  if (err != hipSuccess) return lrs_fail("hipHostGetDevicePointer: %s (is the memory pinned?)", hipGetErrorString(err));
  return 0;
}

// Asynchronous copy of step metadata from pinned host memory to the device.  Small copies (a decode
// step's few KB) are done by a kernel that reads the pinned memory through its device address:
// launching it costs the host a fraction of what the runtime's copy path does, and it orders with
// the step's kernels like any other.  `src` must be pinned (hipHostMalloc) memory.
__global__ void copy_from_host_kernel(int4* __restrict__ dst, const int4* __restrict__ src, int64_t chunks) {   // either side may be pinned host memory
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < chunks; i += (int64_t)gridDim.x * blockDim.x) dst[i] = src[i];
}

// A few bytes of results from the device into pinned host memory, written by a kernel through the
// memory's device address (can be recorded in a graph, unlike a copy that may use a copy engine).
LRS_API int lrs_copy_to_pinned(void* dst_host, const void* src, int64_t bytes, void* stream) {
  LRS_REQUIRE(bytes > 0 && bytes % 16 == 0 && (uintptr_t)dst_host % 16 == 0 && (uintptr_t)src % 16 == 0,
              "copy_to_pinned: %lld bytes and both addresses must be multiples of 16", (long long)bytes);
  void* device_dst = nullptr;
  hipError_t err = hipHostGetDevicePointer(&device_dst, dst_host, 0);
  if (err != hipSuccess) return lrs_fail("hipHostGetDevicePointer: %s (is the memory pinned?)", hipGetErrorString(err));
  const int64_t chunks = bytes / 16;
  const int blocks = (int)((chunks + 255) / 256 < 64 ? (chunks + 255) / 256 : 64);
  copy_from_host_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>((int4*)device_dst, (const int4*)src, chunks);
  return lrs_check_launch("copy_to_pinned");
}

// A step's metadata from pinned host memory to the device and, in the same launch, the block table entries that
// changed since the last step written into the device's tables: `count` (offset, value) pairs lie in the pinned buffer
// from byte `pairs_at` on (they need not be part of what is copied); the workgroups behind those that copy read them
// there and scatter them.  One launch where a copy and a scatter kernel would be two, each with its wait for the host.
__global__ void copy_and_scatter_kernel(int4* __restrict__ dst, const int4* __restrict__ src, int64_t chunks, int copy_blocks,
                                        int* __restrict__ tables, const int* __restrict__ pairs, int count) {
  if ((int)blockIdx.x < copy_blocks) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < chunks; i += (int64_t)copy_blocks * blockDim.x) dst[i] = src[i];
  } else {
    const int i = ((int)blockIdx.x - copy_blocks) * blockDim.x + threadIdx.x;
    if (i < count) tables[pairs[2 * i]] = pairs[2 * i + 1];
  }
}

LRS_API int lrs_copy_h2d_scatter(void* dst, const void* src, int64_t bytes, int* tables, int64_t pairs_at, int count, void* stream) {
  LRS_REQUIRE(bytes >= 0 && bytes % 16 == 0 && (uintptr_t)dst % 16 == 0 && (uintptr_t)src % 16 == 0 && bytes <= (256 << 10),
              "copy_h2d_scatter: %lld bytes (at most 256 KB; 0: nothing is copied) and both addresses must be multiples of 16", (long long)bytes);
  LRS_REQUIRE(count > 0 && tables && pairs_at >= 0 && pairs_at % 8 == 0, "copy_h2d_scatter: needs pairs to scatter at a multiple of 8 bytes");
  void* device_src = nullptr;
  hipError_t err = hipHostGetDevicePointer(&device_src, const_cast<void*>(src), 0);
  if (err != hipSuccess) return lrs_fail("hipHostGetDevicePointer: %s (is the memory pinned?)", hipGetErrorString(err));
  const int64_t chunks = bytes / 16;
  const int copy_blocks = (int)((chunks + 255) / 256 < 64 ? (chunks + 255) / 256 : 64);
  copy_and_scatter_kernel<<<copy_blocks + (count + 255) / 256, 256, 0, (hipStream_t)stream>>>(
      (int4*)dst, (const int4*)device_src, chunks, copy_blocks, tables, (const int*)((const char*)device_src + pairs_at), count);
  return lrs_check_launch("copy_h2d_scatter");
}

LRS_API int lrs_copy_h2d(void* dst, const void* src, int64_t bytes, void* stream) {
  hipStream_t s = (hipStream_t)stream;
  if (bytes <= (256 << 10) && bytes % 16 == 0 && (uintptr_t)dst % 16 == 0 && (uintptr_t)src % 16 == 0) {
    void* device_src = nullptr;
    if (hipHostGetDevicePointer(&device_src, const_cast<void*>(src), 0) != hipSuccess) {
      (void)hipGetLastError();      // not pinned after all: the runtime's copy path takes it
      device_src = nullptr;
    }
    if (device_src) {
      const int64_t chunks = bytes / 16;
      const int blocks = (int)((chunks + 255) / 256 < 64 ? (chunks + 255) / 256 : 64);
      copy_from_host_kernel<<<blocks, 256, 0, s>>>((int4*)dst, (const int4*)device_src, chunks);
      return lrs_check_launch("copy_h2d");
    }
  }
  hipError_t err = hipMemcpyAsync(dst, src, (size_t)bytes, hipMemcpyHostToDevice, s);
  if (err != hipSuccess) return lrs_fail("hipMemcpyAsync: %s", hipGetErrorString(err));
  return 0;
}

// Probe of the rate at which a kernel can stream memory: reads `chunks` 16-byte pieces once (four
// in flight per lane) and leaves one word per workgroup in `sink` so that nothing is optimised away.
__global__ __launch_bounds__(256) void stream_read_kernel(const int4* __restrict__ src, int64_t chunks, int* __restrict__ sink) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  int acc = 0;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (; i + 3 * stride < chunks; i += 4 * stride) {
    const int4 a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
    acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
  }
  for (; i < chunks; i += stride) {
    const int4 a = src[i];
    acc ^= a.x ^ a.y ^ a.z ^ a.w;
  }
  acc ^= __shfl_xor(acc, 32, 64);
  if (threadIdx.x == 0) sink[blockIdx.x] = acc;
}

LRS_API int lrs_stream_read(const void* src, int64_t bytes, int* sink, int blocks, void* stream) {
  LRS_REQUIRE(bytes >= 16 && (uintptr_t)src % 16 == 0 && blocks > 0 && sink, "stream_read: needs 16-byte aligned memory, a sink and blocks");
  stream_read_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>((const int4*)src, bytes / 16, sink);
  return lrs_check_launch("stream_read");
}
