// Two measurements of the compute unit itself, for `microbench lds` and `microbench mfma`: what they
// show decided the LDS layouts and the instruction order of the prefill attention kernel.  Nothing on
// the product path calls them.
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
