// Shared declarations of the gfx950 kernel library: scalar types, error reporting
// and wave-level reductions.  Every extern "C" entry point returns 0 on success or
// a non-zero code after storing a message that lrs_last_error() returns.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define LRS_API extern "C" __attribute__((visibility("default")))

// dtype codes used by every entry point
enum { LRS_F32 = 0, LRS_BF16 = 1 };

typedef __bf16 bf16;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int WAVE = 64;

int lrs_fail(const char* fmt, ...);
int lrs_check_launch(const char* what);

#define LRS_REQUIRE(cond, ...)                \
  do {                                        \
    if (!(cond)) return lrs_fail(__VA_ARGS__); \
  } while (0)

template <typename T>
__device__ __forceinline__ float to_float(T v) { return (float)v; }
template <typename T>
__device__ __forceinline__ T from_float(float v) { return (T)v; }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, WAVE));
  return v;
}

// Sum over a whole workgroup of up to 1024 threads; `scratch` holds 16 floats of LDS.
// Every thread gets the result.  Contains two barriers.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int waves = (blockDim.x + WAVE - 1) / WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int i = 0; i < waves; ++i) total += scratch[i];
  return total;
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
  v = wave_max(v);
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int waves = (blockDim.x + WAVE - 1) / WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = -INFINITY;
  for (int i = 0; i < waves; ++i) total = fmaxf(total, scratch[i]);
  return total;
}
