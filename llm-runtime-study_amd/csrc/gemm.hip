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

// ------------------------------------------------- bf16 kernel for few rows
// Decode-sized products (M <= 64): the weight matrix is streamed exactly once and the time
// is the time to read it.  One workgroup owns 16 weight rows; its waves split K between them
// and add their partial sums through LDS in a fixed order.  Weights are the MFMA A operand
// (16 rows x 32 k, each lane one 16-byte load of a row), the activations the B operand
// (32 k x 16 tokens, read from L2); MT is the number of 16-token blocks.  UNROLL steps of 32 k
// are loaded before any is used, so each wave keeps UNROLL KB of weights in flight.
template <int MT, int WAVES, int UNROLL>
__global__ __launch_bounds__(WAVES * 64) void gemm_bf16_skinny_kernel(
    void* __restrict__ out, int mode, const bf16* __restrict__ x, const bf16* __restrict__ w,
    const bf16* __restrict__ bias, int m, int n, int k, int lda, int ldc) {
  __shared__ floatx4 partial[WAVES][MT][WAVE];
  const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int row = n0 + r < n ? n0 + r : n - 1;
  const bf16* wp = w + (int64_t)row * k + g * 8;
  const bf16* xp[MT];
  bool live[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int token = t * 16 + r;
    live[t] = token < m;
    xp[t] = x + (int64_t)(live[t] ? token : 0) * lda + g * 8;
  }
  floatx4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  const int steps = (k + 31) / 32;
  const int per_wave = (steps + WAVES - 1) / WAVES;
  int s = wave * per_wave;
  const int s_end = s + per_wave < steps ? s + per_wave : steps;
  const int full_end = k / 32 < s_end ? k / 32 : s_end;   // steps whose 32 k are all inside K
  for (; s + UNROLL <= full_end; s += UNROLL) {
    bf16x8 a[UNROLL], b[UNROLL][MT];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) a[u] = *(const bf16x8*)(wp + (s + u) * 32);
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t) b[u][t] = live[t] ? *(const bf16x8*)(xp[t] + (s + u) * 32) : zero;
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], b[u][t], acc[t], 0, 0, 0);
  }
  for (; s < s_end; ++s) {
    const bool inside = s * 32 + g * 8 < k;
    const bf16x8 a = inside ? *(const bf16x8*)(wp + s * 32) : zero;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const bf16x8 b = (inside && live[t]) ? *(const bf16x8*)(xp[t] + s * 32) : zero;
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[t], 0, 0, 0);
    }
  }
#pragma unroll
  for (int t = 0; t < MT; ++t) partial[wave][t][lane] = acc[t];
  __syncthreads();
  // accumulator layout: token = t*16 + lane % 16, weight row = n0 + 4 * (lane / 16) + i
  for (int e = tid; e < MT * WAVE * 4; e += WAVES * WAVE) {
    const int t = e / (WAVE * 4), l = (e / 4) % WAVE, i = e % 4;
    const int token = t * 16 + (l & 15), gn = n0 + 4 * (l >> 4) + i;
    if (token >= m || gn >= n) continue;
    float v = 0.f;
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv) v += partial[wv][t][l][i];
    if (bias) v += (float)bias[gn];
    emit<bf16>(out, mode, (int64_t)token * ldc + gn, v);
  }
}

template <int MT>
static void launch_skinny(void* out, int mode, const bf16* a, const bf16* w, const bf16* bias, int m, int n,
                          int k, int lda, int ldc, hipStream_t s) {
  const int tiles = (n + 15) / 16;
  constexpr int UNROLL = MT == 1 ? 8 : (MT == 2 ? 4 : 2);
  if (tiles <= 2048)
    gemm_bf16_skinny_kernel<MT, 8, UNROLL><<<tiles, 8 * 64, 0, s>>>(out, mode, a, w, bias, m, n, k, lda, ldc);
  else
    gemm_bf16_skinny_kernel<MT, 4, UNROLL><<<tiles, 4 * 64, 0, s>>>(out, mode, a, w, bias, m, n, k, lda, ldc);
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
    if (aligned && m <= 64) {
      const bf16 *ap = (const bf16*)a, *wp = (const bf16*)w, *bp = (const bf16*)bias;
      if (m <= 16) launch_skinny<1>(out, mode, ap, wp, bp, m, n, k, lda, ldc, s);
      else if (m <= 32) launch_skinny<2>(out, mode, ap, wp, bp, m, n, k, lda, ldc, s);
      else if (m <= 48) launch_skinny<3>(out, mode, ap, wp, bp, m, n, k, lda, ldc, s);
      else launch_skinny<4>(out, mode, ap, wp, bp, m, n, k, lda, ldc, s);
    } else if (aligned) {
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
