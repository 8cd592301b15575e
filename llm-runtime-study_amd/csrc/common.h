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

// Memory straight into LDS (global_load_lds_dwordx4): lane l of the wave fetches the 16 bytes at
// base + lane_offset (base the same for the whole wave) and they land at LDS byte address lds_address +
// 16 l; nothing passes through registers and the wave goes on at once.  The compiler does not know these
// fetches: whoever reads the LDS they fill waits for them with fetched_then_barrier (they finish in the
// order they were asked for, and count in vmcnt).  LDS that only they write must still be named as an
// address here, which is what tells the compiler that its contents change.
__device__ __forceinline__ void fetch_to_lds(const void* base, unsigned lane_offset, unsigned lds_address) {
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)base);
  const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)((uintptr_t)base >> 32));
  const unsigned long long uniform_base = ((unsigned long long)hi << 32) | lo;
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :: "s"(__builtin_amdgcn_readfirstlane(lds_address)), "v"(lane_offset), "s"(uniform_base) : "memory");
}
// Waits until at most `PENDING` of this wave's fetches are still on their way, then for the workgroup.
template <int PENDING>
__device__ __forceinline__ void fetched_then_barrier() {
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" :: "n"(PENDING) : "memory");
}
