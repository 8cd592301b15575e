// Token choice on the device, one workgroup per logits row.
//   greedy: the lowest index among the largest logits.
//   temperature: a draw from softmax(logits / temperature) through the exponential race
//   argmax_i (logit_i / temperature - log E_i), E_i ~ Exp(1) from a counter-based generator
//   keyed by (seed, draw counter, token index): the draw of a request depends on its own
//   seed and on how many tokens it has drawn, never on the other rows of the batch.
//   Entries equal to -inf (filtered out beforehand) are never chosen.
//   A row that holds a value that is not finite is refused, as the reference refuses it
//   (mini_llm/sampling.py:104-113): its token comes out as -1, which the host turns into an error.
//   Rows that filter_logits() has been over (`filtered`, and a positive temperature) may hold -inf;
//   NaN and +inf are refused there too, and filter_logits() leaves a NaN in a row that was not finite
//   when it came.
#include "common.h"
#include "no_alloc.h"

#include <mutex>
#include <type_traits>

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
    const uint32_t* __restrict__ counters, int filtered) {
  __shared__ float best_value[16];
  __shared__ int best_index[16];
  const int row = blockIdx.x, tid = threadIdx.x;
  const float* src = logits + (int64_t)row * row_stride;
  const float temp = temperature ? temperature[row] : 0.f;
  const uint64_t seed = seeds ? seeds[row] : 0;
  const uint32_t counter = counters ? counters[row] : 0;
  const bool may_hold_minus_inf = filtered && temp > 0.f;
  float value = -INFINITY;
  int index = 0x7fffffff;
  int bad = 0;
  for (int i = tid; i < vocab; i += blockDim.x) {
    float v = src[i];
    if (!(fabsf(v) < INFINITY) && !(may_hold_minus_inf && v == -INFINITY)) bad = 1;
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
  bad = __syncthreads_or(bad);
  if (tid == 0) {
    const int waves = (blockDim.x + WAVE - 1) / WAVE;
    for (int i = 1; i < waves; ++i)
      if (best_value[i] > value || (best_value[i] == value && best_index[i] < index)) {
        value = best_value[i];
        index = best_index[i];
      }
    out[row] = bad || index == 0x7fffffff ? -1 : index;      // nothing finite to choose from is refused too
  }
}

// The same choice in two passes for large vocabularies: `parts` workgroups per row each reduce a
// slice to its best (value, index); one workgroup per row then takes the best of those.  The order
// of preference (larger value, then lower index) makes the result equal to the one-pass kernel's.
__global__ __launch_bounds__(256) void choose_token_part_kernel(
    float* __restrict__ part_value, int* __restrict__ part_index, const float* __restrict__ logits,
    int64_t row_stride, int vocab, int parts, const float* __restrict__ temperature,
    const uint64_t* __restrict__ seeds, const uint32_t* __restrict__ counters, int filtered) {
  __shared__ float best_value[4];
  __shared__ int best_index[4];
  const int row = blockIdx.y, part = blockIdx.x, tid = threadIdx.x;
  const float* src = logits + (int64_t)row * row_stride;
  const float temp = temperature ? temperature[row] : 0.f;
  const uint64_t seed = seeds ? seeds[row] : 0;
  const uint32_t counter = counters ? counters[row] : 0;
  const bool may_hold_minus_inf = filtered && temp > 0.f;
  const int per = (vocab + parts - 1) / parts;
  const int begin = part * per, end = begin + per < vocab ? begin + per : vocab;
  float value = -INFINITY;
  int index = 0x7fffffff;
  int bad = 0;
  for (int i = begin + tid; i < end; i += 256) {
    float v = src[i];
    if (!(fabsf(v) < INFINITY) && !(may_hold_minus_inf && v == -INFINITY)) bad = 1;
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
  bad = __syncthreads_or(bad);
  if (tid == 0) {
    for (int i = 1; i < 4; ++i)
      if (best_value[i] > value || (best_value[i] == value && best_index[i] < index)) {
        value = best_value[i];
        index = best_index[i];
      }
    part_value[(int64_t)row * parts + part] = bad ? NAN : value;      // a NaN tells the second pass to refuse the row
    part_index[(int64_t)row * parts + part] = index;
  }
}

__global__ void choose_token_final_kernel(int* __restrict__ out, const float* __restrict__ part_value,
                                          const int* __restrict__ part_index, int parts) {
  const int row = blockIdx.x, lane = threadIdx.x;
  float value = -INFINITY;
  int index = 0x7fffffff;
  bool bad = false;
  for (int i = lane; i < parts; i += WAVE) {
    const float v = part_value[(int64_t)row * parts + i];
    const int at = part_index[(int64_t)row * parts + i];
    if (v != v) bad = true;
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
  bad = __any(bad);
  if (lane == 0) out[row] = bad || index == 0x7fffffff ? -1 : index;
}

// out[r] = chosen token of row r, or -1 for a row that is not finite.  temperature == nullptr or temperature[r] == 0:
// greedy.  filtered: filter_logits() has been over the rows (those of positive temperature may hold -inf).
// part_value / part_index [rows, parts] are scratch for the two-pass form (parts > 1).
LRS_API int lrs_choose_tokens_split(int* out, const float* logits, int64_t row_stride, int rows, int vocab,
                                    const float* temperature, const uint64_t* seeds, const uint32_t* counters,
                                    float* part_value, int* part_index, int parts, int filtered, void* stream) {
  LRS_REQUIRE(rows > 0 && vocab > 0 && parts > 0, "choose_tokens: rows=%d vocab=%d parts=%d must be positive", rows, vocab, parts);
  LRS_REQUIRE(row_stride >= vocab, "choose_tokens: row stride below vocab");
  LRS_REQUIRE(part_value && part_index, "choose_tokens: the two-pass form needs its scratch buffers");
  choose_token_part_kernel<<<dim3(parts, rows), 256, 0, (hipStream_t)stream>>>(part_value, part_index, logits, row_stride, vocab,
                                                                               parts, temperature, seeds, counters, filtered);
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
                                     int parts, int filtered, void* stream) {
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
                                                                               parts, temperature, seeds, counters, filtered);
  if (lrs_check_launch("choose_tokens_static_part")) return 1;
  choose_token_final_kernel<<<rows, WAVE, 0, (hipStream_t)stream>>>(out, part_value, part_index, parts);
  return lrs_check_launch("choose_tokens_static_final");
}

// out[r] = chosen token of row r.  temperature == nullptr or temperature[r] == 0: greedy.
LRS_API int lrs_choose_tokens(int* out, const float* logits, int64_t row_stride, int rows, int vocab,
                              const float* temperature, const uint64_t* seeds,
                              const uint32_t* counters, int filtered, void* stream) {
  LRS_REQUIRE(rows > 0 && vocab > 0, "choose_tokens: rows=%d vocab=%d must be positive", rows, vocab);
  LRS_REQUIRE(row_stride >= vocab, "choose_tokens: row stride below vocab");
  const int threads = vocab >= 4096 ? 1024 : 256;
  choose_token_kernel<<<rows, threads, 0, (hipStream_t)stream>>>(out, logits, row_stride, vocab,
                                                                 temperature, seeds, counters, filtered);
  return lrs_check_launch("choose_tokens");
}

// Keeps the logits that survive top-k and top-p of softmax(logits / temperature), sets the
// others to -inf, in place.  One workgroup per row.  Rule (the reference's): after scaling
// by 1/temperature keep the k largest; then, in descending order, drop a token once the
// probability mass strictly before it reaches top_p, so the token that crosses stays.
// Values equal to a threshold are all kept: where the reference's topk and sort keep one of several equal
// values and drop another, whichever their order of the equal ones says, both stay here (a kept set that does
// not depend on an order of arrival).
// Both thresholds are values of the row itself and are found without a sort, by selection over the
// ordered bit patterns of float32, 11 + 11 + 10 bits at a time: a pass over the row counts (top-k) or
// weighs (top-p) the values by the next digit of their pattern in LDS, the digit whose bin holds the
// k-th largest value (the value at which the mass from the top reaches p of the whole) is fixed, and the
// next pass looks inside that bin.  Three passes each instead of a bisection's thirty-two.  Masses are
// added up as integers (exp(v - max) * 2^35), so the sums, and with them the tokens kept, do not depend on
// the order in which the threads arrive.
__device__ __forceinline__ uint32_t ordered_key(float v) {
  const uint32_t bits = __float_as_uint(v);
  return (bits & 0x80000000U) ? ~bits : (bits | 0x80000000U);
}

constexpr int FILTER_BINS = 2048;

// The largest bin b whose own content and everything above it come to `need` or more, and what lies above it.
// All threads call; the first wave works.  bins[] is complete (a barrier has passed) and may be cleared after.
template <typename V>
__device__ __forceinline__ void filter_find_bin(const V* bins, int nbins, double need, int* found_bin, double* found_above) {
  const int lane = threadIdx.x % WAVE;
  if (threadIdx.x < WAVE) {
    const int per = nbins / WAVE;
    double mine = 0.0;
    for (int i = 0; i < per; ++i) mine += (double)bins[lane * per + i];
    double with_mine = mine;                                   // this lane's bins and those of the lanes above
    for (int step = 1; step < WAVE; step <<= 1) {
      const double other = __shfl_down(with_mine, step, WAVE);
      if (lane + step < WAVE) with_mine += other;
    }
    const unsigned long long reach = __ballot(with_mine >= need);
    const int owner = reach ? 63 - __builtin_clzll(reach) : 0;   // the highest lane that reaches it (lane 0 if none: cannot happen)
    if (lane == owner) {
      double above = with_mine - mine;
      int bin = lane * per;
      for (int i = per - 1; i >= 0; --i) {
        const double here = (double)bins[lane * per + i];
        if (above + here >= need) { bin = lane * per + i; break; }
        above += here;
      }
      *found_bin = bin;
      *found_above = above;
    }
  }
  __syncthreads();
}

__global__ __launch_bounds__(1024) void filter_logits_kernel(float* __restrict__ logits,
                                                             int64_t row_stride, int vocab,
                                                             const float* __restrict__ temperature,
                                                             const int* __restrict__ top_k,
                                                             const float* __restrict__ top_p) {
  __shared__ float scratch[16];
  __shared__ unsigned long long bins[FILTER_BINS];             // counts or masses
  __shared__ int found_bin;
  __shared__ double found_above;
  const int row = blockIdx.x, tid = threadIdx.x;
  float* z = logits + (int64_t)row * row_stride;
  const float temp = temperature[row];
  if (!(temp > 0.f)) return;
  const int k = top_k ? top_k[row] : 0;
  const float p = top_p ? top_p[row] : 1.f;
  const bool use_k = k > 0 && k < vocab, use_p = p < 1.f;

  // A pass over the row: body(index, logit) for each of this thread's values.  Four loads of 16 bytes are asked
  // for before any is used (a thread's loads one after the other, each waited for, were what a pass took its
  // time for); rows that do not begin on 16 bytes go one value at a time.  The patterns compared are those of the
  // scaled values logit / temperature, as the reference compares them: two logits whose quotients round to one
  // float32 are a tie there and are kept or dropped together.  The masses are exp((logit - largest logit) / temperature).
  const bool in_fours = ((uintptr_t)z % 16) == 0;
  auto walk = [&](auto&& body) {
    const int fours = in_fours ? vocab / 4 : 0;
    for (int first = tid; first < fours; first += 4 * (int)blockDim.x) {
      floatx4 part[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int at = first + j * (int)blockDim.x;
        part[j] = ((const floatx4*)z)[at < fours ? at : first];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int at = first + j * (int)blockDim.x;
        if (at < fours) {
#pragma unroll
          for (int e = 0; e < 4; ++e) body(at * 4 + e, part[j][e]);
        }
      }
    }
    for (int i = fours * 4 + tid; i < vocab; i += blockDim.x) body(i, z[i]);
  };

  // Every row of positive temperature is looked over once, filtered or not: a row that is not finite as it comes
  // (the reference refuses it, mini_llm/sampling.py:104-113) gets a NaN that the token choice after this kernel
  // refuses, since it can no longer tell a -inf that came from one that a filter left.
  float zmax = -INFINITY;
  int bad = 0;
  walk([&](int, float v) {
    zmax = fmaxf(zmax, v);
    if (!(fabsf(v) < INFINITY)) bad = 1;
  });
  bad = __syncthreads_or(bad);
  if (bad) {
    if (tid == 0) z[0] = NAN;
    return;
  }
  if (!use_k && !use_p) return;
  zmax = block_max(zmax, scratch);
  const float per_temp2 = 1.4426950408889634f / temp;          // exp(x / temp) = exp2(x * this)

  // One selection: MASS false: the largest pattern t with count(pattern >= t) >= need; MASS true: the largest
  // pattern t, among those >= floor, with mass(pattern >= t) >= share of the mass of all those >= floor.
  auto select = [&](auto mass, double need, uint32_t floor, float share) -> uint32_t {
    constexpr bool MASS = decltype(mass)::value;
    uint32_t prefix = 0;
#pragma unroll
    for (int level = 0; level < 3; ++level) {
      const int shift = level == 0 ? 21 : level == 1 ? 10 : 0, nbins = level == 2 ? 1024 : 2048;
      for (int i = tid; i < nbins; i += blockDim.x) bins[i] = 0;
      __syncthreads();
      uint32_t run_bin = 0xFFFFFFFFu;                          // values that follow each other into one bin are added up first
      unsigned long long run = 0;
      walk([&](int, float v) {
        const uint32_t key = ordered_key(v / temp);
        if (MASS && key < floor) return;
        if (level == 1 && (key >> 21) != prefix) return;
        if (level == 2 && (key >> 10) != prefix) return;
        const uint32_t bin = (key >> shift) & (uint32_t)(nbins - 1);
        const unsigned long long weight = MASS ? (unsigned long long)(__builtin_amdgcn_exp2f((v - zmax) * per_temp2) * 34359738368.f) : 1ull;
        if (bin == run_bin) {
          run += weight;
        } else {
          if (run_bin != 0xFFFFFFFFu) atomicAdd(&bins[run_bin], run);
          run_bin = bin;
          run = weight;
        }
      });
      if (run_bin != 0xFFFFFFFFu) atomicAdd(&bins[run_bin], run);
      __syncthreads();
      if (MASS && level == 0) {                                // the whole mass: every bin of the first pass
        double whole = 0.0;
        if (tid < WAVE) {
          for (int i = tid; i < nbins; i += WAVE) whole += (double)bins[i];
          for (int step = WAVE / 2; step > 0; step >>= 1) whole += __shfl_xor(whole, step, WAVE);
          if (tid == 0) found_above = whole;
        }
        __syncthreads();
        need = (double)share * found_above;
        __syncthreads();
      }
      filter_find_bin(bins, nbins, need, &found_bin, &found_above);
      need -= found_above;
      prefix = (prefix << (level == 2 ? 10 : 11)) | (uint32_t)found_bin;
      __syncthreads();                                         // everyone has read the result before the bins are cleared
    }
    return prefix;
  };

  uint32_t threshold = 0;
  if (use_k) threshold = select(std::false_type{}, (double)k, 0u, 0.f);
  if (use_p) threshold = select(std::true_type{}, 0.0, threshold, p);
  walk([&](int i, float v) {
    if (ordered_key(v / temp) < threshold) z[i] = -INFINITY;
  });
}

LRS_API int lrs_filter_logits(float* logits, int64_t row_stride, int rows, int vocab,
                              const float* temperature, const int* top_k, const float* top_p,
                              void* stream) {
  LRS_REQUIRE(rows > 0 && vocab > 0, "filter_logits: rows=%d vocab=%d must be positive", rows, vocab);
  LRS_REQUIRE(temperature != nullptr, "filter_logits: temperature is required");
  filter_logits_kernel<<<rows, 1024, 0, (hipStream_t)stream>>>(logits, row_stride, vocab, temperature, top_k, top_p);
  return lrs_check_launch("filter_logits");
}
