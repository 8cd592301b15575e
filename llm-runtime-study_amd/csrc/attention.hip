// Causal attention over the paged cache for a ragged batch: every query token attends to
// the cached keys of its own request at positions lo..p, p being the token's absolute
// position and lo = max(0, p - window + 1) when a window is given.  Keys and values of this
// step's tokens are already in the cache when these kernels run.
//
// Pages are [page, kv_head, slot, dim]; block_table[r, i] is the page holding positions
// i*page_size .. (i+1)*page_size-1 of request r.  Scores, softmax and the weighted sum are
// float32.  Key tiles start at multiples of the tile size counted from position 0, so the
// rounding of a query's result depends on its position only, never on how the sequence
// was cut into steps.
#include "common.h"

// ---------------------------------------------------------- generic kernel
// One workgroup per (query token, query head); any head_dim up to 4 * threads.
template <typename T, int THREADS>
__global__ __launch_bounds__(THREADS) void attention_generic_kernel(
    T* __restrict__ out, int out_stride, const T* __restrict__ q, int q_stride,
    const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    const int* __restrict__ block_table, int table_stride, const int* __restrict__ token_request,
    const int* __restrict__ positions, int nq, int nkv, int d, int page_size, float scale,
    int window) {
  extern __shared__ float smem[];
  float* qs = smem;                           // [d]
  float* probs = qs + d;                      // [THREADS]
  int64_t* bases = (int64_t*)(probs + THREADS);  // [THREADS] element offset of each key row
  __shared__ float scratch[16];

  const int token = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
  const int request = token_request[token];
  const int pos = positions[token];
  const int kv_head = head / (nq / nkv);
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int* table = block_table + (int64_t)request * table_stride;

  for (int i = tid; i < d; i += THREADS) qs[i] = to_float(q[(int64_t)token * q_stride + (int64_t)head * d + i]);
  __syncthreads();

  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  float running_max = -INFINITY, running_sum = 0.f;
  for (int tile = (lo / THREADS) * THREADS; tile <= pos; tile += THREADS) {
    const int key = tile + tid;
    const bool valid = key >= lo && key <= pos;
    float score = -INFINITY;
    int64_t base = 0;
    if (valid) {
      const int64_t page = table[key / page_size];
      base = ((page * nkv + kv_head) * page_size + key % page_size) * d;
      const T* kr = k_pages + base;
      float dot = 0.f;
      for (int i = 0; i < d; ++i) dot = fmaf(qs[i], to_float(kr[i]), dot);
      score = dot * scale;
    }
    const float tile_max = block_max(score, scratch);
    const float new_max = fmaxf(running_max, tile_max);
    const float p = valid ? expf(score - new_max) : 0.f;
    const float tile_sum = block_sum(p, scratch);
    const float alpha = expf(running_max - new_max);  // exp(-inf) = 0 on the first tile
    running_sum = running_sum * alpha + tile_sum;
    running_max = new_max;
    probs[tid] = p;
    bases[tid] = base;
    __syncthreads();
    const int count = (pos - tile + 1 < THREADS) ? pos - tile + 1 : THREADS;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int dim = tid + c * THREADS;
      if (dim < d) {
        float a = acc[c] * alpha;
        for (int j = 0; j < count; ++j) {
          const float pj = probs[j];
          if (pj != 0.f) a = fmaf(pj, to_float(v_pages[bases[j] + dim]), a);
        }
        acc[c] = a;
      }
    }
    __syncthreads();
  }
  const float inv = 1.0f / running_sum;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int dim = tid + c * THREADS;
    if (dim < d) out[(int64_t)token * out_stride + (int64_t)head * d + dim] = from_float<T>(acc[c] * inv);
  }
}

// out [tokens, nq*d] (row stride out_stride); q rows are [nq*d] with row stride q_stride.
LRS_API int lrs_attention(void* out, int out_stride, const void* q, int q_stride, const void* k_pages,
                          const void* v_pages, const int* block_table, int table_stride,
                          const int* token_request, const int* positions, int dtype, int tokens,
                          int nq, int nkv, int d, int page_size, float scale, int window,
                          void* stream) {
  LRS_REQUIRE(tokens > 0 && nq > 0 && nkv > 0 && d > 0 && page_size > 0, "attention: bad sizes tokens=%d nq=%d nkv=%d d=%d page=%d", tokens, nq, nkv, d, page_size);
  LRS_REQUIRE(nq % nkv == 0, "attention: %d query heads do not divide into %d kv heads", nq, nkv);
  LRS_REQUIRE(d <= 512, "attention: head_dim %d above the supported 512", d);
  LRS_REQUIRE(window >= 0, "attention: window must be >= 0 (0 = none)");
  constexpr int THREADS = 128;
  dim3 grid(tokens, nq);
  const size_t lds = sizeof(float) * (d + THREADS) + sizeof(int64_t) * THREADS + 16;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == LRS_F32)
    attention_generic_kernel<float, THREADS><<<grid, THREADS, lds, s>>>(
        (float*)out, out_stride, (const float*)q, q_stride, (const float*)k_pages, (const float*)v_pages,
        block_table, table_stride, token_request, positions, nq, nkv, d, page_size, scale, window);
  else if (dtype == LRS_BF16)
    attention_generic_kernel<bf16, THREADS><<<grid, THREADS, lds, s>>>(
        (bf16*)out, out_stride, (const bf16*)q, q_stride, (const bf16*)k_pages, (const bf16*)v_pages,
        block_table, table_stride, token_request, positions, nq, nkv, d, page_size, scale, window);
  else
    return lrs_fail("attention: unknown dtype %d", dtype);
  return lrs_check_launch("attention");
}
