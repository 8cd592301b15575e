// Token choice on the device, one workgroup per logits row.
//   greedy: the lowest index among the largest logits.
//   temperature: a draw from softmax(logits / temperature) through the exponential race
//   argmax_i (logit_i / temperature - log E_i), E_i ~ Exp(1) from a counter-based generator
//   keyed by (seed, draw counter, token index): the draw of a request depends on its own
//   seed and on how many tokens it has drawn, never on the other rows of the batch.
//   Entries equal to -inf (filtered out beforehand) are never chosen.
#include "common.h"
#include "no_alloc.h"

#include <mutex>

__device__ __forceinline__ uint32_t mix32(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7feb352dU;
  x ^= x >> 15;
  x *= 0x846ca68bU;
  x ^= x >> 16;
  return x;
}

__device__ __forceinline__ float exponential_variate(uint32_t seed_lo, uint32_t seed_hi,
                                                     uint32_t counter, uint32_t index) {
  uint32_t x = mix32(index ^ 0x9e3779b9U);
  x = mix32(x + seed_lo);
  x = mix32(x ^ seed_hi);
  x = mix32(x + counter * 0x85ebca6bU);
  // v uniform in (0, 1); E = -log(1 - v) keeps full relative precision for small v
  float v = ((float)x + 0.5f) * 2.3283064365386963e-10f;
  v = fminf(v, 0.99999994f);
  return -log1pf(-v);
}

__global__ __launch_bounds__(1024) void choose_token_kernel(
    int* __restrict__ out, const float* __restrict__ logits, int64_t row_stride, int vocab,
    const float* __restrict__ temperature, const uint64_t* __restrict__ seeds,
    const uint32_t* __restrict__ counters) {
  __shared__ float best_value[16];
  __shared__ int best_index[16];
  const int row = blockIdx.x, tid = threadIdx.x;
  const float* src = logits + (int64_t)row * row_stride;
  const float temp = temperature ? temperature[row] : 0.f;
  const uint64_t seed = seeds ? seeds[row] : 0;
  const uint32_t counter = counters ? counters[row] : 0;
  float value = -INFINITY;
  int index = 0x7fffffff;
  for (int i = tid; i < vocab; i += blockDim.x) {
    float v = src[i];
    if (temp > 0.f && v > -INFINITY)
      v = v / temp - logf(exponential_variate((uint32_t)seed, (uint32_t)(seed >> 32), counter, (uint32_t)i));
    if (v > value || (v == value && i < index)) {
      value = v;
      index = i;
    }
  }
#pragma unroll
  for (int off = WAVE / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(value, off, WAVE);
    const int oi = __shfl_xor(index, off, WAVE);
    if (ov > value || (ov == value && oi < index)) {
      value = ov;
      index = oi;
    }
  }
  const int wave = tid / WAVE, lane = tid % WAVE;
  if (lane == 0) {
    best_value[wave] = value;
    best_index[wave] = index;
  }
  __syncthreads();
  if (tid == 0) {
    const int waves = (blockDim.x + WAVE - 1) / WAVE;
    for (int i = 1; i < waves; ++i)
      if (best_value[i] > value || (best_value[i] == value && best_index[i] < index)) {
        value = best_value[i];
        index = best_index[i];
      }
    out[row] = index;
  }
}

// The same choice in two passes for large vocabularies: `parts` workgroups per row each reduce a
// slice to its best (value, index); one workgroup per row then takes the best of those.  The order
// of preference (larger value, then lower index) makes the result equal to the one-pass kernel's.
__global__ __launch_bounds__(256) void choose_token_part_kernel(
    float* __restrict__ part_value, int* __restrict__ part_index, const float* __restrict__ logits,
    int64_t row_stride, int vocab, int parts, const float* __restrict__ temperature,
    const uint64_t* __restrict__ seeds, const uint32_t* __restrict__ counters) {
  __shared__ float best_value[4];
  __shared__ int best_index[4];
  const int row = blockIdx.y, part = blockIdx.x, tid = threadIdx.x;
  const float* src = logits + (int64_t)row * row_stride;
  const float temp = temperature ? temperature[row] : 0.f;
  const uint64_t seed = seeds ? seeds[row] : 0;
  const uint32_t counter = counters ? counters[row] : 0;
  const int per = (vocab + parts - 1) / parts;
  const int begin = part * per, end = begin + per < vocab ? begin + per : vocab;
  float value = -INFINITY;
  int index = 0x7fffffff;
  for (int i = begin + tid; i < end; i += 256) {
    float v = src[i];
    if (temp > 0.f && v > -INFINITY)
      v = v / temp - logf(exponential_variate((uint32_t)seed, (uint32_t)(seed >> 32), counter, (uint32_t)i));
    if (v > value || (v == value && i < index)) {
      value = v;
      index = i;
    }
  }
#pragma unroll
  for (int off = WAVE / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(value, off, WAVE);
    const int oi = __shfl_xor(index, off, WAVE);
    if (ov > value || (ov == value && oi < index)) {
      value = ov;
      index = oi;
    }
  }
  if (tid % WAVE == 0) {
    best_value[tid / WAVE] = value;
    best_index[tid / WAVE] = index;
  }
  __syncthreads();
  if (tid == 0) {
    for (int i = 1; i < 4; ++i)
      if (best_value[i] > value || (best_value[i] == value && best_index[i] < index)) {
        value = best_value[i];
        index = best_index[i];
      }
    part_value[(int64_t)row * parts + part] = value;
    part_index[(int64_t)row * parts + part] = index;
  }
}

__global__ void choose_token_final_kernel(int* __restrict__ out, const float* __restrict__ part_value,
                                          const int* __restrict__ part_index, int parts) {
  const int row = blockIdx.x, lane = threadIdx.x;
  float value = -INFINITY;
  int index = 0x7fffffff;
  for (int i = lane; i < parts; i += WAVE) {
    const float v = part_value[(int64_t)row * parts + i];
    const int at = part_index[(int64_t)row * parts + i];
    if (v > value || (v == value && at < index)) {
      value = v;
      index = at;
    }
  }
#pragma unroll
  for (int off = WAVE / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(value, off, WAVE);
    const int oi = __shfl_xor(index, off, WAVE);
    if (ov > value || (ov == value && oi < index)) {
      value = ov;
      index = oi;
    }
  }
  if (lane == 0) out[row] = index;
}

// out[r] = chosen token of row r.  temperature == nullptr or temperature[r] == 0: greedy.
// part_value / part_index [rows, parts] are scratch for the two-pass form (parts > 1).
LRS_API int lrs_choose_tokens_split(int* out, const float* logits, int64_t row_stride, int rows, int vocab,
                                    const float* temperature, const uint64_t* seeds, const uint32_t* counters,
                                    float* part_value, int* part_index, int parts, void* stream) {
  LRS_REQUIRE(rows > 0 && vocab > 0 && parts > 0, "choose_tokens: rows=%d vocab=%d parts=%d must be positive", rows, vocab, parts);
  LRS_REQUIRE(row_stride >= vocab, "choose_tokens: row stride below vocab");
  LRS_REQUIRE(part_value && part_index, "choose_tokens: the two-pass form needs its scratch buffers");
  choose_token_part_kernel<<<dim3(parts, rows), 256, 0, (hipStream_t)stream>>>(part_value, part_index, logits, row_stride, vocab,
                                                                               parts, temperature, seeds, counters);
  if (lrs_check_launch("choose_tokens_part")) return 1;
  choose_token_final_kernel<<<rows, WAVE, 0, (hipStream_t)stream>>>(out, part_value, part_index, parts);
  return lrs_check_launch("choose_tokens_final");
}

// ---- The two-pass choice for callers that cannot allocate (declared in no_alloc.h).
// Its scratch, the best (value, index) of every slice of every row, lies in a file-scope device array
// instead of a buffer that the caller brings.  Every GPU of the process holds a copy of the array, at
// an address of its own, until the process ends; host code never uses the array's name as an address
// but asks the runtime once per device (choose_scratch_of) and passes the answer to the kernels.
// Nothing in the array has to start at zero: the first pass writes every element the second reads.
// Calls that overlap on one GPU (two streams, two threads) share the array and race.
static __device__ __align__(256) unsigned char choose_scratch[LRS_CHOOSE_STATIC_MAX_PARTS * 8];

constexpr int CHOOSE_MAX_DEVICES = 64;
static void* g_choose_scratch[CHOOSE_MAX_DEVICES] = {};
static std::mutex g_choose_scratch_lock;

// The address of the current device's copy of choose_scratch, asked from the runtime the first time.
static int choose_scratch_of(void** address) {
  int device = -1;
  hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess) return lrs_fail("choose_tokens_static: hipGetDevice: %s", hipGetErrorString(err));
  if (device < 0 || device >= CHOOSE_MAX_DEVICES) return lrs_fail("choose_tokens_static: device %d is beyond the %d this library keeps scratch for", device, CHOOSE_MAX_DEVICES);
  std::lock_guard<std::mutex> hold(g_choose_scratch_lock);
  if (!g_choose_scratch[device]) {
    void* found = nullptr;
    err = hipGetSymbolAddress(&found, HIP_SYMBOL(choose_scratch));
    if (err != hipSuccess || !found) return lrs_fail("choose_tokens_static: hipGetSymbolAddress: %s", hipGetErrorString(err));
    g_choose_scratch[device] = found;
  }
  *address = g_choose_scratch[device];
  return 0;
}

LRS_API int lrs_choose_tokens_static_init() {
  void* unused = nullptr;
  return choose_scratch_of(&unused);
}

LRS_API int lrs_choose_tokens_static_max_parts() { return LRS_CHOOSE_STATIC_MAX_PARTS; }

LRS_API int lrs_choose_tokens_static(int* out, const float* logits, int64_t row_stride, int rows, int vocab,
                                     const float* temperature, const uint64_t* seeds, const uint32_t* counters,
                                     int parts, void* stream) {
  LRS_REQUIRE(rows > 0 && vocab > 0 && parts > 0, "choose_tokens_static: rows=%d vocab=%d parts=%d must be positive", rows, vocab, parts);
  LRS_REQUIRE(row_stride >= vocab, "choose_tokens_static: row stride below vocab");
  LRS_REQUIRE(out && logits, "choose_tokens_static: out and logits are required");
  LRS_REQUIRE((int64_t)rows * parts <= LRS_CHOOSE_STATIC_MAX_PARTS,
              "choose_tokens_static: rows x parts = %d x %d is more than the %d slices the static scratch holds", rows, parts, LRS_CHOOSE_STATIC_MAX_PARTS);
  void* scratch = nullptr;
  if (int rc = choose_scratch_of(&scratch)) return rc;
  float* part_value = (float*)scratch;
  int* part_index = (int*)((unsigned char*)scratch + (size_t)LRS_CHOOSE_STATIC_MAX_PARTS * 4);
  choose_token_part_kernel<<<dim3(parts, rows), 256, 0, (hipStream_t)stream>>>(part_value, part_index, logits, row_stride, vocab,
                                                                               parts, temperature, seeds, counters);
  if (lrs_check_launch("choose_tokens_static_part")) return 1;
  choose_token_final_kernel<<<rows, WAVE, 0, (hipStream_t)stream>>>(out, part_value, part_index, parts);
  return lrs_check_launch("choose_tokens_static_final");
}

// out[r] = chosen token of row r.  temperature == nullptr or temperature[r] == 0: greedy.
LRS_API int lrs_choose_tokens(int* out, const float* logits, int64_t row_stride, int rows, int vocab,
                              const float* temperature, const uint64_t* seeds,
                              const uint32_t* counters, void* stream) {
  LRS_REQUIRE(rows > 0 && vocab > 0, "choose_tokens: rows=%d vocab=%d must be positive", rows, vocab);
  LRS_REQUIRE(row_stride >= vocab, "choose_tokens: row stride below vocab");
  const int threads = vocab >= 4096 ? 1024 : 256;
  choose_token_kernel<<<rows, threads, 0, (hipStream_t)stream>>>(out, logits, row_stride, vocab,
                                                                 temperature, seeds, counters);
  return lrs_check_launch("choose_tokens");
}

// Keeps the logits that survive top-k and top-p of softmax(logits / temperature), sets the
// others to -inf, in place.  One workgroup per row.  Rule (the reference's): after scaling
// by 1/temperature keep the k largest; then, in descending order, drop a token once the
// probability mass strictly before it reaches top_p, so the token that crosses stays.
// Both thresholds are found by bisection over the ordered bit patterns of float32 (at most
// 32 passes over the row each), which needs no sort.
__device__ __forceinline__ uint32_t ordered_key(float v) {
  const uint32_t bits = __float_as_uint(v);
  return (bits & 0x80000000U) ? ~bits : (bits | 0x80000000U);
}

__global__ __launch_bounds__(1024) void filter_logits_kernel(float* __restrict__ logits,
                                                             int64_t row_stride, int vocab,
                                                             const float* __restrict__ temperature,
                                                             const int* __restrict__ top_k,
                                                             const float* __restrict__ top_p) {
  __shared__ float scratch[16];
  const int row = blockIdx.x, tid = threadIdx.x;
  float* z = logits + (int64_t)row * row_stride;
  const float temp = temperature[row];
  if (!(temp > 0.f)) return;
  const int k = top_k ? top_k[row] : 0;
  const float p = top_p ? top_p[row] : 1.f;
  const bool use_k = k > 0 && k < vocab, use_p = p < 1.f;
  if (!use_k && !use_p) return;

  float vmax = -INFINITY, vmin = INFINITY;
  for (int i = tid; i < vocab; i += blockDim.x) {
    const float v = z[i] / temp;
    vmax = fmaxf(vmax, v);
    if (v > -INFINITY) vmin = fminf(vmin, v);
  }
  vmax = block_max(vmax, scratch);
  vmin = -block_max(-vmin, scratch);
  const uint32_t key_min = ordered_key(vmin), key_max = ordered_key(vmax);

  // largest key t with count(key >= t) >= k: the k-th largest value
  uint32_t threshold = key_min;
  if (use_k) {
    uint32_t lo = key_min, hi = key_max;
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo + 1) / 2;
      float count = 0.f;
      for (int i = tid; i < vocab; i += blockDim.x) count += (ordered_key(z[i] / temp) >= mid) ? 1.f : 0.f;
      count = block_sum(count, scratch);
      if (count >= (float)k) lo = mid; else hi = mid - 1;
    }
    threshold = lo;
  }
  if (use_p) {
    float total = 0.f;
    for (int i = tid; i < vocab; i += blockDim.x) {
      const float v = z[i] / temp;
      if (ordered_key(v) >= threshold) total += expf(v - vmax);
    }
    total = block_sum(total, scratch);
    // smallest key t with mass(keys > t) < p * total; mass above the maximum is 0, so it exists
    uint32_t lo = threshold, hi = key_max;
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo) / 2;
      float above = 0.f;
      for (int i = tid; i < vocab; i += blockDim.x) {
        const float v = z[i] / temp;
        if (ordered_key(v) > mid) above += expf(v - vmax);
      }
      above = block_sum(above, scratch);
      if (above < p * total) hi = mid; else lo = mid + 1;
    }
    threshold = lo;
  }
  for (int i = tid; i < vocab; i += blockDim.x)
    if (ordered_key(z[i] / temp) < threshold) z[i] = -INFINITY;
}

LRS_API int lrs_filter_logits(float* logits, int64_t row_stride, int rows, int vocab,
                              const float* temperature, const int* top_k, const float* top_p,
                              void* stream) {
  LRS_REQUIRE(rows > 0 && vocab > 0, "filter_logits: rows=%d vocab=%d must be positive", rows, vocab);
  LRS_REQUIRE(temperature != nullptr, "filter_logits: temperature is required");
  filter_logits_kernel<<<rows, 1024, 0, (hipStream_t)stream>>>(logits, row_stride, vocab, temperature, top_k, top_p);
  return lrs_check_launch("filter_logits");
}
