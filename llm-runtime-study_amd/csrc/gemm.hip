// Matrix products y = x W^T (+ bias) with W stored [out, in] as in the checkpoint.
//   x [M, K] row-major, W [N, K] row-major, both of dtype T (float or bf16).
// Output modes: store as T, store as float32, or add into a float32 matrix (the residual
// stream).  Accumulation is float32 in every kernel; the float32 kernels use plain FMAs and
// no matrix cores, so a float32 run is float32 throughout.  The order of the sum over K
// for one output element never depends on M, so a row's result does not depend on what
// else is in the batch.
#include "common.h"

enum { OUT_STORE = 0, OUT_STORE_F32 = 1, OUT_ADD_F32 = 2 };

template <typename T>
__device__ __forceinline__ void emit(void* out, int mode, int64_t index, float value) {
  if (mode == OUT_STORE) ((T*)out)[index] = from_float<T>(value);
  else if (mode == OUT_STORE_F32) ((float*)out)[index] = value;
  else ((float*)out)[index] += value;
}

// ------------------------------------------------- generic tiled FMA kernel
// 64x64 output tile, 16-deep K slices through LDS, 4x4 outputs per thread.  Any M, N, K.
template <typename T>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(void* __restrict__ out, int mode,
                                                         const T* __restrict__ a,
                                                         const T* __restrict__ w,
                                                         const T* __restrict__ bias, int m, int n,
                                                         int k, int lda, int ldc) {
  constexpr int BM = 64, BN = 64, BK = 16;
  __shared__ float as[BK][BM + 4];
  __shared__ float ws[BK][BN + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int tm = (tid / 16) * 4, tn = (tid % 16) * 4;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < k; k0 += BK) {
    for (int e = tid; e < BM * BK; e += 256) {
      const int r = e / BK, c = e % BK;
      const int gm = m0 + r, gn = n0 + r, gk = k0 + c;
      as[c][r] = (gm < m && gk < k) ? to_float(a[(int64_t)gm * lda + gk]) : 0.f;
      ws[c][r] = (gn < n && gk < k) ? to_float(w[(int64_t)gn * k + gk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = as[kk][tm + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = ws[kk][tn + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
  for (int i = 0; i < 4; ++i) {
    const int gm = m0 + tm + i;
    if (gm >= m) continue;
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + tn + j;
      if (gn >= n) continue;
      float v = acc[i][j];
      if (bias) v += to_float(bias[gn]);
      emit<T>(out, mode, (int64_t)gm * ldc + gn, v);
    }
  }
}

// ------------------------------------------------------- bf16 MFMA kernel
// 128x128 output tile per workgroup of 4 waves (2x2), each wave 64x64 as 2x2 MFMA
// 32x32x16 tiles.  K is walked in slices of 32 through LDS.  Needs K % 8 == 0 so that
// every 8-element chunk is a 16-byte aligned load; rows past M or N and chunks past K
// are zero-filled.
__global__ __launch_bounds__(256) void gemm_bf16_mfma_kernel(void* __restrict__ out, int mode,
                                                             const bf16* __restrict__ a,
                                                             const bf16* __restrict__ w,
                                                             const bf16* __restrict__ bias, int m,
                                                             int n, int k, int lda, int ldc) {
  constexpr int BM = 128, BN = 128, BK = 32, LD = BK + 8;  // padded LDS rows
  __shared__ __attribute__((aligned(16))) bf16 as[BM * LD];
  __shared__ __attribute__((aligned(16))) bf16 ws[BN * LD];
  const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int wm = (wave / 2) * 64, wn = (wave % 2) * 64;
  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int k0 = 0; k0 < k; k0 += BK) {
    // 128 rows x 4 chunks of 8 per operand, 2 chunks per thread per operand
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int e = tid + it * 256;
      const int r = e / 4, c = (e % 4) * 8;
      const int gk = k0 + c;
      bf16x8 av = zero, wv = zero;
      if (m0 + r < m && gk < k) av = *(const bf16x8*)(a + (int64_t)(m0 + r) * lda + gk);
      if (n0 + r < n && gk < k) wv = *(const bf16x8*)(w + (int64_t)(n0 + r) * k + gk);
      *(bf16x8*)(as + r * LD + c) = av;
      *(bf16x8*)(ws + r * LD + c) = wv;
    }
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < BK; ks += 16) {
      bf16x8 af[2], wf[2];
      const int kc = ks + (lane / 32) * 8;
#pragma unroll
      for (int i = 0; i < 2; ++i) af[i] = *(const bf16x8*)(as + (wm + i * 32 + lane % 32) * LD + kc);
#pragma unroll
      for (int j = 0; j < 2; ++j) wf[j] = *(const bf16x8*)(ws + (wn + j * 32 + lane % 32) * LD + kc);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], wf[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
  }
  // accumulator layout of the 32x32 tile: column = lane % 32, row = 8*(r/4) + 4*(lane/32) + r%4
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int gn = n0 + wn + j * 32 + lane % 32;
      if (gn >= n) continue;
      const float b = bias ? (float)bias[gn] : 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int gm = m0 + wm + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + r % 4;
        if (gm < m) emit<bf16>(out, mode, (int64_t)gm * ldc + gn, acc[i][j][r] + b);
      }
    }
}

// out [M, N] (row stride ldc) = a [M, K] (row stride lda) times w[N, K]^T.
LRS_API int lrs_gemm(void* out, int mode, const void* a, const void* w, const void* bias, int dtype,
                     int m, int n, int k, int lda, int ldc, void* stream) {
  LRS_REQUIRE(m > 0 && n > 0 && k > 0, "gemm: sizes m=%d n=%d k=%d must be positive", m, n, k);
  LRS_REQUIRE(lda >= k && ldc >= n, "gemm: strides lda=%d ldc=%d too small for k=%d n=%d", lda, ldc, k, n);
  LRS_REQUIRE(mode >= OUT_STORE && mode <= OUT_ADD_F32, "gemm: unknown output mode %d", mode);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == LRS_F32) {
    dim3 grid((n + 63) / 64, (m + 63) / 64);
    gemm_tiled_kernel<float><<<grid, 256, 0, s>>>(out, mode, (const float*)a, (const float*)w,
                                                  (const float*)bias, m, n, k, lda, ldc);
  } else if (dtype == LRS_BF16) {
    const bool aligned = k % 8 == 0 && lda % 8 == 0 && ((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0);
    if (aligned) {
      dim3 grid((n + 127) / 128, (m + 127) / 128);
      gemm_bf16_mfma_kernel<<<grid, 256, 0, s>>>(out, mode, (const bf16*)a, (const bf16*)w,
                                                 (const bf16*)bias, m, n, k, lda, ldc);
    } else {
      dim3 grid((n + 63) / 64, (m + 63) / 64);
      gemm_tiled_kernel<bf16><<<grid, 256, 0, s>>>(out, mode, (const bf16*)a, (const bf16*)w,
                                                   (const bf16*)bias, m, n, k, lda, ldc);
    }
  } else {
    return lrs_fail("gemm: unknown dtype %d", dtype);
  }
  return lrs_check_launch("gemm");
}
