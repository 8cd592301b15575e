// Three measurements of the compute unit itself, for `microbench lds`, `microbench mfma` and `microbench lines`:
// what they show decided the LDS layouts and the instruction order of the prefill attention kernel and how the
// few-rows products load their weights.  Nothing on the product path calls them.
#include "common.h"

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Every lane reads 16 bytes, the way a matrix-core fragment is read: the lane's row is lane % 16 and its
// piece lane / 16, rows `stride` bytes apart.  Eight such reads an iteration, at different places.
__global__ __launch_bounds__(256, 2) void probe_lds_kernel(unsigned* sink, int iters, int stride) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[32768];
  for (int i = threadIdx.x; i < 8192; i += 256) ((unsigned*)lds)[i] = i;
  __syncthreads();
  const int lane = threadIdx.x % WAVE;
  unsigned acc = 0;
  for (int it = 0; it < iters; ++it) {
    asm volatile("" ::: "memory");                               // the reads are made again every time round
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const unsigned char* p = lds + (u & 1) * 16 * stride + (u >> 1) * 1024 + (lane & 15) * stride + (lane >> 4) * 16;
      const u32x4 v = *(const u32x4*)p;
      acc ^= v[0] ^ v[1] ^ v[2] ^ v[3];
    }
  }
  if (acc == 0x12345678u) sink[threadIdx.x] = acc;
}

// 32 matrix instructions an iteration (16 accumulators in turn) with `VALU` multiply-adds after each and
// `EXPS` exponentials after every second one.
template <int VALU, int EXPS>
__global__ __launch_bounds__(256, 2) void probe_mfma_kernel(float* sink, int iters) {
  const int lane = threadIdx.x;
  bf16x8 a, b;
  for (int i = 0; i < 8; ++i) {
    a[i] = (bf16)(float)(lane + i);
    b[i] = (bf16)(float)(lane * 3 + i);
  }
  floatx4 acc[16];
  for (int i = 0; i < 16; ++i) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};
  float v[8];
  for (int i = 0; i < 8; ++i) v[i] = lane * 0.001f + i;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int n = 0; n < 32; ++n) {
      acc[n % 16] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[n % 16], 0, 0, 0);
#pragma unroll
      for (int j = 0; j < VALU; ++j) v[(n + j) & 7] = fmaf(v[(n + j) & 7], 1.0001f, 0.5f);
      if (EXPS && n % 2 == 0) v[n & 7] = __builtin_amdgcn_exp2f(v[n & 7] * 1e-9f);
    }
  }
  float total = 0.f;
  for (int i = 0; i < 16; ++i) total += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
  for (int i = 0; i < 8; ++i) total += v[i];
  if (total == 12345.678f) sink[lane] = total;
}

// A workgroup streams `bytes_each` bytes of its own, 4 KB (16 rows of 256 bytes) a wave and turn, four 16-byte
// loads a lane, the next turn asked for before this one is used.  Which 16 bytes a lane takes:
//   0  row lane % 16, piece lane / 16 (+ 4 a load): the order of a matrix-core fragment, 16 rows to 16 neighbouring lanes
//   1  byte lane * 16 (+ 1 KB a load): whole lines, 256 bytes to 16 neighbouring lanes
//   2  row lane / 4, piece lane % 4 (+ 4 a load): 64 bytes of a row to 4 neighbouring lanes, 4 rows to 16
template <int PATTERN>
__global__ __launch_bounds__(1024) void probe_lines_kernel(const unsigned char* __restrict__ base, size_t bytes_each, unsigned* sink) {
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, waves = blockDim.x / WAVE;
  const unsigned char* mine = base + (size_t)blockIdx.x * bytes_each;
  const int turns = (int)(bytes_each / 4096);
  auto at = [&](int c) {
    return PATTERN == 0 ? (lane % 16) * 256 + (lane / 16) * 16 + c * 64 : PATTERN == 1 ? lane * 16 + c * 1024 : (lane / 4) * 256 + (lane % 4) * 16 + c * 64;
  };
  u32x4 now[4], next[4];
  unsigned acc = 0;
  if (wave < turns)
#pragma unroll
    for (int c = 0; c < 4; ++c) now[c] = *(const u32x4*)(mine + (size_t)wave * 4096 + at(c));
  for (int turn = wave; turn < turns; turn += waves) {
    const bool more = turn + waves < turns;
    if (more)
#pragma unroll
      for (int c = 0; c < 4; ++c) next[c] = *(const u32x4*)(mine + (size_t)(turn + waves) * 4096 + at(c));
#pragma unroll
    for (int c = 0; c < 4; ++c) acc ^= now[c][0] ^ now[c][1] ^ now[c][2] ^ now[c][3];
    if (more)
#pragma unroll
      for (int c = 0; c < 4; ++c) now[c] = next[c];
  }
  if (acc == 0x12345678u) sink[threadIdx.x % 256] = acc;
}

LRS_API int lrs_probe_lines(const void* data, size_t bytes, void* sink, int blocks, int threads, size_t bytes_each, int pattern, void* stream) {
  LRS_REQUIRE(data && sink && blocks > 0, "probe_lines: data, sink and blocks are required");
  LRS_REQUIRE(threads >= 64 && threads <= 1024 && threads % 64 == 0, "probe_lines: %d threads a workgroup, must be 64..1024 in whole waves", threads);
  LRS_REQUIRE(bytes_each >= 4096 && bytes_each % 4096 == 0 && (size_t)blocks * bytes_each <= bytes && (uintptr_t)data % 16 == 0,
              "probe_lines: %d workgroups of %zu bytes (a multiple of 4,096) need more than the %zu bytes given", blocks, bytes_each, bytes);
  hipStream_t s = (hipStream_t)stream;
  switch (pattern) {
    case 0: probe_lines_kernel<0><<<blocks, threads, 0, s>>>((const unsigned char*)data, bytes_each, (unsigned*)sink); break;
    case 1: probe_lines_kernel<1><<<blocks, threads, 0, s>>>((const unsigned char*)data, bytes_each, (unsigned*)sink); break;
    case 2: probe_lines_kernel<2><<<blocks, threads, 0, s>>>((const unsigned char*)data, bytes_each, (unsigned*)sink); break;
    default: return lrs_fail("probe_lines: pattern must be 0, 1 or 2, got %d", pattern);
  }
  return lrs_check_launch("probe_lines");
}

// sink: at least 1 KB of device memory (never written unless the sums happen to hit a magic value)
LRS_API int lrs_probe_lds(void* sink, int blocks, int iters, int stride, void* stream) {
  LRS_REQUIRE(sink && blocks > 0 && iters > 0, "probe_lds: sink, blocks and iters are required");
  LRS_REQUIRE(stride >= 16 && stride % 16 == 0 && 32 * stride + 3 * 1024 + 64 <= 32768, "probe_lds: stride %d must be a multiple of 16 of at most 912", stride);
  probe_lds_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>((unsigned*)sink, iters, stride);
  return lrs_check_launch("probe_lds");
}

LRS_API int lrs_probe_mfma(void* sink, int blocks, int iters, int valu, int exps, void* stream) {
  LRS_REQUIRE(sink && blocks > 0 && iters > 0, "probe_mfma: sink, blocks and iters are required");
  hipStream_t s = (hipStream_t)stream;
#define PROBE(V, E) probe_mfma_kernel<V, E><<<blocks, 256, 0, s>>>((float*)sink, iters)
  if (exps) {
    switch (valu) {
      case 2: PROBE(2, 1); break;
      case 3: PROBE(3, 1); break;
      default: return lrs_fail("probe_mfma: with exponentials, 2 or 3 multiply-adds per product, got %d", valu);
    }
  } else {
    switch (valu) {
      case 0: PROBE(0, 0); break;
      case 1: PROBE(1, 0); break;
      case 2: PROBE(2, 0); break;
      case 3: PROBE(3, 0); break;
      case 4: PROBE(4, 0); break;
      case 6: PROBE(6, 0); break;
      default: return lrs_fail("probe_mfma: 0, 1, 2, 3, 4 or 6 multiply-adds per product, got %d", valu);
    }
  }
#undef PROBE
  return lrs_check_launch("probe_mfma");
}
