// Memory-bound parts of the step: embedding gather, RMSNorm, rotary tables, the fused
// per-head q/k norm + rotation + cache write, and the gated activation.
// The residual stream is float32 in every precision mode; `T` below is the dtype of
// weights and activations (float or bf16).  All statistics are computed in float32.
#include "common.h"

// ------------------------------------------------------------------ embedding
template <typename T>
__global__ void embed_kernel(float* __restrict__ out, const T* __restrict__ table,
                             const int* __restrict__ ids, int hidden, float multiplier) {
  const int64_t row = ids[blockIdx.x];
  const T* src = table + row * hidden;
  float* dst = out + (int64_t)blockIdx.x * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_float(src[i]) * multiplier;
}

LRS_API int lrs_embed(float* out, const void* table, int dtype, const int* ids, int tokens,
                      int hidden, float multiplier, void* stream) {
  LRS_REQUIRE(tokens > 0 && hidden > 0, "embed: tokens=%d hidden=%d must be positive", tokens, hidden);
  dim3 grid(tokens), block(256);
  if (dtype == LRS_F32)
    embed_kernel<float><<<grid, block, 0, (hipStream_t)stream>>>(out, (const float*)table, ids, hidden, multiplier);
  else if (dtype == LRS_BF16)
    embed_kernel<bf16><<<grid, block, 0, (hipStream_t)stream>>>(out, (const bf16*)table, ids, hidden, multiplier);
  else
    return lrs_fail("embed: unknown dtype %d", dtype);
  return lrs_check_launch("embed");
}

// -------------------------------------------------------------------- RMSNorm
// y = w * x * rsqrt(mean(x^2) + eps); x is a float32 row (optionally picked through `rows`),
// the result is rounded once to the output dtype.  With `add` (bf16 [rows, hidden], no row
// picking) the row is first updated in place, x += add, and the norm is taken of the sum: the
// residual add after a library matrix product and the norm that follows it in one pass.
template <typename TW, typename TO>
__global__ void rmsnorm_kernel(TO* __restrict__ out, float* __restrict__ x, const bf16* __restrict__ add,
                               const TW* __restrict__ weight, const int* __restrict__ rows,
                               int hidden, float eps) {
  __shared__ float scratch[16];
  const int64_t src_row = rows ? rows[blockIdx.x] : blockIdx.x;
  float* src = x + src_row * hidden;
  TO* dst = out + (int64_t)blockIdx.x * hidden;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float v = src[i];
    if (add) {
      v += (float)add[src_row * hidden + i];
      src[i] = v;                                   // read again below by the same thread only
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)hidden + eps);
  for (int i = threadIdx.x; i < hidden; i += blockDim.x)
    dst[i] = from_float<TO>(to_float(weight[i]) * (src[i] * inv));
}

// The same with the row held in registers: every thread owns up to VEC chunks of 4 values, read
// once with 16-byte loads; for hidden % 4 == 0 and hidden <= 4 * VEC * threads.
template <typename TW, typename TO, int VEC>
__global__ void rmsnorm_vec_kernel(TO* __restrict__ out, float* __restrict__ x, const bf16* __restrict__ add,
                                   const TW* __restrict__ weight, const int* __restrict__ rows,
                                   int hidden, float eps, const float* __restrict__ sums = nullptr, int splits = 0) {
  __shared__ float scratch[16];
  const int64_t src_row = rows ? rows[blockIdx.x] : blockIdx.x;
  floatx4* src = (floatx4*)(x + src_row * hidden);
  const int chunks = hidden / 4;
  floatx4 v[VEC], w[VEC];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    const int c = threadIdx.x + j * blockDim.x;
    if (c < chunks) {
      v[j] = src[c];
      if (add) {
        const bf16x4 y = *(const bf16x4*)(add + src_row * hidden + c * 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) v[j][i] += (float)y[i];
        src[c] = v[j];
      }
      if (sums) {
        // what the K splits of the product before left, [splits, rows, hidden], added up in split order
        floatx4 y = floatx4{0.f, 0.f, 0.f, 0.f};
        for (int sp = 0; sp < splits; ++sp)
          y += *(const floatx4*)(sums + ((int64_t)sp * gridDim.x + src_row) * hidden + c * 4);
        v[j] += y;
        src[c] = v[j];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) w[j][i] = to_float(weight[c * 4 + i]);
      ss += v[j][0] * v[j][0] + v[j][1] * v[j][1] + v[j][2] * v[j][2] + v[j][3] * v[j][3];
    }
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)hidden + eps);
  TO* dst = out + (int64_t)blockIdx.x * hidden;
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    const int c = threadIdx.x + j * blockDim.x;
    if (c < chunks) {
#pragma unroll
      for (int i = 0; i < 4; ++i) dst[c * 4 + i] = from_float<TO>(w[j][i] * (v[j][i] * inv));
    }
  }
}

static int launch_rmsnorm(void* out, int out_dtype, float* x, const bf16* add, const void* weight, int w_dtype,
                          const int* rows, int n_rows, int hidden, float eps, void* stream) {
  LRS_REQUIRE(n_rows > 0 && hidden > 0, "rmsnorm: rows=%d hidden=%d must be positive", n_rows, hidden);
  LRS_REQUIRE(eps > 0.f, "rmsnorm: eps must be positive");
  LRS_REQUIRE(add == nullptr || rows == nullptr, "rmsnorm: the fused residual add takes all rows in order");
  dim3 grid(n_rows), block(hidden >= 2048 ? 512 : 256);
  hipStream_t s = (hipStream_t)stream;
  if (hidden % 4 == 0 && hidden <= 4 * 4 * 512 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)add % 8) == 0) {
    const int threads = hidden <= 1024 ? 64 : (hidden <= 4096 ? 256 : 512);
#define LAUNCH_VEC(TW, TO) \
  rmsnorm_vec_kernel<TW, TO, 4><<<grid, threads, 0, s>>>((TO*)out, x, add, (const TW*)weight, rows, hidden, eps)
    if (w_dtype == LRS_F32 && out_dtype == LRS_F32) LAUNCH_VEC(float, float);
    else if (w_dtype == LRS_BF16 && out_dtype == LRS_BF16) LAUNCH_VEC(bf16, bf16);
    else if (w_dtype == LRS_F32 && out_dtype == LRS_BF16) LAUNCH_VEC(float, bf16);
    else if (w_dtype == LRS_BF16 && out_dtype == LRS_F32) LAUNCH_VEC(bf16, float);
    else return lrs_fail("rmsnorm: unknown dtypes %d/%d", w_dtype, out_dtype);
#undef LAUNCH_VEC
    return lrs_check_launch("rmsnorm");
  }
#define LAUNCH(TW, TO) \
  rmsnorm_kernel<TW, TO><<<grid, block, 0, s>>>((TO*)out, x, add, (const TW*)weight, rows, hidden, eps)
  if (w_dtype == LRS_F32 && out_dtype == LRS_F32) LAUNCH(float, float);
  else if (w_dtype == LRS_BF16 && out_dtype == LRS_BF16) LAUNCH(bf16, bf16);
  else if (w_dtype == LRS_F32 && out_dtype == LRS_BF16) LAUNCH(float, bf16);
  else if (w_dtype == LRS_BF16 && out_dtype == LRS_F32) LAUNCH(bf16, float);
  else return lrs_fail("rmsnorm: unknown dtypes %d/%d", w_dtype, out_dtype);
#undef LAUNCH
  return lrs_check_launch("rmsnorm");
}

LRS_API int lrs_rmsnorm(void* out, int out_dtype, const float* x, const void* weight, int w_dtype,
                        const int* rows, int n_rows, int hidden, float eps, void* stream) {
  return launch_rmsnorm(out, out_dtype, (float*)x, nullptr, weight, w_dtype, rows, n_rows, hidden, eps, stream);
}

// The first half of "add the K splits' sums to the residual stream, then RMSNorm", spread over rows x 1,024
// columns (a workgroup of four waves each) instead of one workgroup a row: x += sum of the splits; next_x =
// bf16(x * weight); the workgroup's sum of x^2 goes to next_sumsq [gridDim.x, rows].  The product that reads
// next_x multiplies its rows by rsqrt(sum of the parts / hidden + eps): the factor is constant along a row.
constexpr int NORM_BEGIN_COLUMNS = 1024;
template <typename TW>
__global__ __launch_bounds__(NORM_BEGIN_COLUMNS / 4) void split_add_norm_begin_kernel(
    float* __restrict__ x, const float* __restrict__ sums, int splits, const TW* __restrict__ weight,
    bf16* __restrict__ next_x, float* __restrict__ next_sumsq, int hidden) {
  __shared__ float scratch[16];
  const int row = blockIdx.y, rows = gridDim.y, c = (blockIdx.x * (NORM_BEGIN_COLUMNS / 4) + threadIdx.x) * 4;
  float ss = 0.f;
  if (c < hidden) {
    const int64_t at = (int64_t)row * hidden + c;
    floatx4 v = *(const floatx4*)(x + at);
    floatx4 y = floatx4{0.f, 0.f, 0.f, 0.f};
    for (int sp0 = 0; sp0 < splits; sp0 += 8) {       // eight splits asked for at a time (usually all there are)
      floatx4 part[8];
#pragma unroll
      for (int i = 0; i < 8; ++i)
        part[i] = sp0 + i < splits ? *(const floatx4*)(sums + ((int64_t)(sp0 + i) * rows) * hidden + at) : floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < 8; ++i) y += part[i];
    }
    v += y;
    *(floatx4*)(x + at) = v;
    bf16x4 nx;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      nx[i] = (bf16)(v[i] * to_float(weight[c + i]));
      ss += v[i] * v[i];
    }
    *(bf16x4*)(next_x + at) = nx;
  }
  ss = block_sum(ss, scratch);
  if (threadIdx.x == 0) next_sumsq[(int64_t)blockIdx.x * rows + row] = ss;
}

LRS_API int lrs_norm_begin_parts(int hidden) { return (hidden + NORM_BEGIN_COLUMNS - 1) / NORM_BEGIN_COLUMNS; }

LRS_API int lrs_split_add_norm_begin(float* x, const float* sums, int splits, const void* weight, int w_dtype, void* next_x,
                                     float* next_sumsq, int n_rows, int hidden, void* stream) {
  LRS_REQUIRE(n_rows > 0 && n_rows <= 65535 && hidden > 0 && splits > 0 && sums && next_x && next_sumsq,
              "split_add_norm_begin: rows=%d hidden=%d splits=%d must be positive", n_rows, hidden, splits);
  LRS_REQUIRE(hidden % 4 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)sums % 16) == 0 && ((uintptr_t)next_x % 8) == 0,
              "split_add_norm_begin: needs hidden %% 4 == 0 and aligned rows (hidden=%d)", hidden);
  const dim3 grid(lrs_norm_begin_parts(hidden), n_rows);
  constexpr int threads = NORM_BEGIN_COLUMNS / 4;
  hipStream_t s = (hipStream_t)stream;
  if (w_dtype == LRS_F32) split_add_norm_begin_kernel<float><<<grid, threads, 0, s>>>(x, sums, splits, (const float*)weight, (bf16*)next_x, next_sumsq, hidden);
  else if (w_dtype == LRS_BF16) split_add_norm_begin_kernel<bf16><<<grid, threads, 0, s>>>(x, sums, splits, (const bf16*)weight, (bf16*)next_x, next_sumsq, hidden);
  else return lrs_fail("split_add_norm_begin: unknown weight dtype %d", w_dtype);
  return lrs_check_launch("split_add_norm_begin");
}

// x [n_rows, hidden] float32 += the sum over `splits` of sums[split, n_rows, hidden], then out = RMSNorm(x): what
// follows a product of many rows whose K was divided between workgroups, in one pass over the rows.
LRS_API int lrs_split_add_rmsnorm(void* out, int out_dtype, float* x, const float* sums, int splits, const void* weight,
                                  int w_dtype, int n_rows, int hidden, float eps, void* stream) {
  LRS_REQUIRE(n_rows > 0 && hidden > 0 && splits > 0 && sums && out && x && weight, "split_add_rmsnorm: rows=%d hidden=%d splits=%d must be positive", n_rows, hidden, splits);
  LRS_REQUIRE(eps > 0.f, "split_add_rmsnorm: eps must be positive");
  LRS_REQUIRE(hidden % 4 == 0 && hidden <= 4 * 4 * 512 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)sums % 16) == 0,
              "split_add_rmsnorm: needs hidden %% 4 == 0, at most 8192 columns and 16-byte aligned rows (hidden=%d)", hidden);
  const int threads = hidden <= 1024 ? 64 : (hidden <= 4096 ? 256 : 512);
  hipStream_t s = (hipStream_t)stream;
#define LAUNCH_VEC(TW, TO) \
  rmsnorm_vec_kernel<TW, TO, 4><<<n_rows, threads, 0, s>>>((TO*)out, x, nullptr, (const TW*)weight, nullptr, hidden, eps, sums, splits)
  if (w_dtype == LRS_F32 && out_dtype == LRS_F32) LAUNCH_VEC(float, float);
  else if (w_dtype == LRS_BF16 && out_dtype == LRS_BF16) LAUNCH_VEC(bf16, bf16);
  else if (w_dtype == LRS_F32 && out_dtype == LRS_BF16) LAUNCH_VEC(float, bf16);
  else if (w_dtype == LRS_BF16 && out_dtype == LRS_F32) LAUNCH_VEC(bf16, float);
  else return lrs_fail("split_add_rmsnorm: unknown dtypes %d/%d", w_dtype, out_dtype);
#undef LAUNCH_VEC
  return lrs_check_launch("split_add_rmsnorm");
}

// x [n_rows, hidden] float32 += y (bf16), then out = RMSNorm(x): see rmsnorm_kernel.
LRS_API int lrs_add_rmsnorm(void* out, int out_dtype, float* x, const void* y, const void* weight, int w_dtype,
                            int n_rows, int hidden, float eps, void* stream) {
  LRS_REQUIRE(y != nullptr, "add_rmsnorm: nothing to add");
  return launch_rmsnorm(out, out_dtype, x, (const bf16*)y, weight, w_dtype, nullptr, n_rows, hidden, eps, stream);
}

// ------------------------------------------------------------- rotary tables
// cos/sin [tokens, half] of angle = float(position) * inv_freq[i], all in float32.
__global__ void rope_table_kernel(float* __restrict__ cosv, float* __restrict__ sinv,
                                  const int* __restrict__ positions,
                                  const float* __restrict__ inv_freq, int half) {
  const float p = (float)positions[blockIdx.x];
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const float angle = p * inv_freq[i];
    cosv[(int64_t)blockIdx.x * half + i] = cosf(angle);
    sinv[(int64_t)blockIdx.x * half + i] = sinf(angle);
  }
}

LRS_API int lrs_rope_table(float* cosv, float* sinv, const int* positions, const float* inv_freq,
                           int tokens, int half, void* stream) {
  LRS_REQUIRE(tokens > 0 && half > 0, "rope_table: tokens=%d half=%d must be positive", tokens, half);
  rope_table_kernel<<<dim3(tokens), dim3(64), 0, (hipStream_t)stream>>>(cosv, sinv, positions, inv_freq, half);
  return lrs_check_launch("rope_table");
}

// ------------------------------------- per-head norm + rotation + cache write
// One wave per (token, head) of the fused projection row [q heads | k heads | v heads].
// q heads: optional RMSNorm over head_dim, optional half-split rotation of the first
// 2*rot_half dims, written back in place.  k heads: the same, written into the paged key
// cache [page, kv_head, slot, dim]; v heads: copied into the paged value cache, which is
// transposed inside a page: [page, kv_head, dim, slot].
// `slots[t]` is page * page_size + offset of token t (negative: do not store).
template <typename T, typename TW>
__global__ void qk_prep_kernel(T* __restrict__ qkv, int row_stride, int nq, int nkv, int d,
                               const TW* __restrict__ q_weight, const TW* __restrict__ k_weight,
                               float eps, const float* __restrict__ cosv,
                               const float* __restrict__ sinv, int rot_half,
                               T* __restrict__ k_pages, T* __restrict__ v_pages,
                               const int* __restrict__ slots, int page_size, int first_head) {
  // v_pages == null: the values are stored by values_to_pages_kernel instead; first_head: the heads before it are left alone
  const int token = blockIdx.x, head = blockIdx.y + first_head, lane = threadIdx.x;
  T* src = qkv + (int64_t)token * row_stride + (int64_t)head * d;
  const bool is_q = head < nq, is_k = !is_q && head < nq + nkv;
  T* dst = src;
  if (!is_q) {
    const int slot = slots[token];
    if (slot < 0) return;
    const int kv_head = is_k ? head - nq : head - nq - nkv;
    const int64_t page = slot / page_size, off = slot % page_size;
    if (!is_k) {
      if (!v_pages) return;
      T* vdst = v_pages + (page * nkv + kv_head) * d * page_size + off;
      for (int i = lane; i < d; i += WAVE) vdst[(int64_t)i * page_size] = src[i];
      return;
    }
    dst = k_pages + ((page * nkv + kv_head) * page_size + off) * d;
  }
  const TW* weight = is_q ? q_weight : k_weight;
  float inv = 1.f;
  if (weight) {
    float ss = 0.f;
    for (int i = lane; i < d; i += WAVE) {
      const float v = to_float(src[i]);
      ss += v * v;
    }
    ss = wave_sum(ss);
    inv = 1.0f / sqrtf(ss / (float)d + eps);
  }
  // pairs (i, i + rot_half) rotate together; dims >= 2*rot_half pass through
  for (int i = lane; i < rot_half; i += WAVE) {
    float a = to_float(src[i]) * inv, b = to_float(src[i + rot_half]) * inv;
    if (weight) {
      a *= to_float(weight[i]);
      b *= to_float(weight[i + rot_half]);
    }
    const float c = cosv[(int64_t)token * rot_half + i], s = sinv[(int64_t)token * rot_half + i];
    dst[i] = from_float<T>(a * c - b * s);
    dst[i + rot_half] = from_float<T>(b * c + a * s);
  }
  for (int i = 2 * rot_half + lane; i < d; i += WAVE) {
    float a = to_float(src[i]) * inv;
    if (weight) a *= to_float(weight[i]);
    dst[i] = from_float<T>(a);
  }
}

// N values of type TW as floats, read in pieces of at most 16 bytes (p aligned to a piece).
template <typename TW, int N>
__device__ __forceinline__ void load_floats(const TW* __restrict__ p, float* out) {
  constexpr int PER = (int)(16 / sizeof(TW)) < N ? (int)(16 / sizeof(TW)) : N;
  typedef TW piece __attribute__((ext_vector_type(PER)));
#pragma unroll
  for (int c = 0; c < N / PER; ++c) {
    const piece v = *(const piece*)(p + c * PER);
#pragma unroll
    for (int i = 0; i < PER; ++i) out[c * PER + i] = to_float(v[i]);
  }
}

// The v heads of 16 consecutive tokens of the step and one kv head into the value pages
// [page, kv_head, dim, slot]: tokens that follow each other in one page land side by side, so a
// thread gathers the values of 16 / sizeof(T) such tokens for one dim (neighbouring lanes read
// neighbouring dims of one token) and writes them with one 16-byte store; it falls back to single
// stores where a run is broken by a page edge, another request or a slot that is not to be stored.
// For steps of many tokens: storing token by token scatters 2-byte writes a page row apart.
template <typename T>
__device__ __forceinline__ void values_to_pages(const T* __restrict__ qkv, int row_stride, int v_offset, int tokens, int nkv,
                                                int d, T* __restrict__ v_pages, const int* __restrict__ slots, int page_size,
                                                int token0, int kvh, int* slot_of) {
  constexpr int RUN = 16 / sizeof(T);
  typedef T vec __attribute__((ext_vector_type(RUN)));
  const int tid = threadIdx.x;
  if (tid < 16) slot_of[tid] = token0 + tid < tokens ? slots[token0 + tid] : -1;
  __syncthreads();
  for (int e = tid; e < d * (16 / RUN); e += 256) {
    const int dim = e % d, first = (e / d) * RUN;
    const int slot0 = slot_of[first];
    bool run = slot0 >= 0 && slot0 % RUN == 0 && slot0 % page_size + RUN <= page_size;
#pragma unroll
    for (int i = 1; i < RUN; ++i) run = run && slot_of[first + i] == slot0 + i;
    const T* src = qkv + (int64_t)(token0 + first) * row_stride + v_offset + (int64_t)kvh * d + dim;
    if (run) {
      vec v;
#pragma unroll
      for (int i = 0; i < RUN; ++i) v[i] = src[(int64_t)i * row_stride];
      const int64_t page = slot0 / page_size, off = slot0 % page_size;
      *(vec*)(v_pages + ((page * nkv + kvh) * d + dim) * page_size + off) = v;
    } else {
#pragma unroll
      for (int i = 0; i < RUN; ++i) {
        const int slot = slot_of[first + i];
        if (slot < 0) continue;
        const int64_t page = slot / page_size, off = slot % page_size;
        v_pages[((page * nkv + kvh) * d + dim) * page_size + off] = src[(int64_t)i * row_stride];
      }
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void values_to_pages_kernel(const T* __restrict__ qkv, int row_stride, int v_offset,
                                                              int tokens, int nkv, int d, T* __restrict__ v_pages,
                                                              const int* __restrict__ slots, int page_size) {
  __shared__ int slot_of[16];
  values_to_pages<T>(qkv, row_stride, v_offset, tokens, nkv, d, v_pages, slots, page_size, blockIdx.x * 16, blockIdx.y, slot_of);
}

// qk_prep for the common shape, with 16-byte accesses: head_dim a power of two times 32 / sizeof(T),
// rotation over the whole head (or none).  A thread owns VE = 16 / sizeof(T) consecutive dims of the
// first half of a head and their VE rotation partners in the second half; d / (2 VE) neighbouring
// threads share a head, and a workgroup takes 256 / that many consecutive (token, head) pairs of the
// `heads` first heads of every token.  Workgroups from `prep_blocks` on (if any) store the v heads
// instead, 16 tokens of one kv head each, as values_to_pages() does.
template <typename T, typename TW, int TOGETHER>
__global__ __launch_bounds__(256) void qk_prep_vec_kernel(T* __restrict__ qkv, int row_stride, int tokens, int heads, int nq,
                                                          int nkv, int d, const TW* __restrict__ q_weight,
                                                          const TW* __restrict__ k_weight, float eps,
                                                          const float* __restrict__ cosv, const float* __restrict__ sinv,
                                                          int rot_half, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                                          const int* __restrict__ slots, int page_size, int prep_blocks,
                                                          const float* __restrict__ sums, int splits,
                                                          int sum_columns, int first_head) {
  // first_head: the heads before it (the q heads, or none) are left as they are.
  // sums != null: the heads come as the float32 sums that the K splits of the q/k/v product left,
  // [splits, tokens, sum_columns], added up here in split order; qkv only receives the prepared q heads.
  constexpr int VE = 16 / sizeof(T);
  typedef T vec __attribute__((ext_vector_type(VE)));
  __shared__ int slot_of[16];
  if ((int)blockIdx.x >= prep_blocks) {      // the whole workgroup
    const int vb = blockIdx.x - prep_blocks;
    values_to_pages<T>(qkv, row_stride, (nq + nkv) * d, tokens, nkv, d, v_pages, slots, page_size, (vb / nkv) * 16, vb % nkv, slot_of);
    return;
  }
  const int per_head = d / (2 * VE), half = d / 2;
  // A group of per_head threads takes TOGETHER consecutive heads of one token (a whole number of such runs
  // fill a token's heads): the token's rotation tables and the norm weights, which every head needs again, are
  // read once a group, and all the heads' values are asked for before the first is worked on.
  constexpr int together = TOGETHER;
  const int groups_per_token = (heads - first_head) / together;
  const int64_t pair = (int64_t)blockIdx.x * (256 / per_head) + threadIdx.x / per_head;
  const int j = threadIdx.x % per_head;
  if (pair >= (int64_t)tokens * groups_per_token) return;   // whole groups of per_head lanes leave together
  const int token = pair / groups_per_token, head0 = first_head + (int)(pair % groups_per_token) * together;
  float c[VE], sn[VE], wq[2][VE], wk[2][VE];
  if (rot_half) {
    load_floats<float, VE>(cosv + (int64_t)token * rot_half + VE * j, c);
    load_floats<float, VE>(sinv + (int64_t)token * rot_half + VE * j, sn);
  }
  if (q_weight) {
    load_floats<TW, VE>(q_weight + VE * j, wq[0]);
    load_floats<TW, VE>(q_weight + half + VE * j, wq[1]);
    load_floats<TW, VE>(k_weight + VE * j, wk[0]);
    load_floats<TW, VE>(k_weight + half + VE * j, wk[1]);
  }
  const int slot = heads > nq ? slots[token] : -1;
  vec lo[TOGETHER], hi[TOGETHER];
  if (!sums) {
#pragma unroll
    for (int t = 0; t < TOGETHER; ++t) {
      const T* from = qkv + (int64_t)token * row_stride + (int64_t)(head0 + t) * d;
      lo[t] = *(const vec*)(from + VE * j);
      hi[t] = *(const vec*)(from + half + VE * j);
    }
  }
#pragma unroll
  for (int t = 0; t < TOGETHER; ++t) {
    const int head = head0 + t;
    T* src = qkv + (int64_t)token * row_stride + (int64_t)head * d;
    const bool is_q = head < nq, is_k = !is_q && head < nq + nkv;
    float a[VE], b[VE], inv = 1.f;
    if (sums) {
#pragma unroll
      for (int e = 0; e < VE; ++e) a[e] = b[e] = 0.f;
      const float* from = sums + (int64_t)token * sum_columns + (int64_t)head * d;
      const int64_t apart = (int64_t)tokens * sum_columns;
      for (int sp0 = 0; sp0 < splits; sp0 += 4) {       // four splits asked for at a time: one trip to memory, not four
        float pa[4][VE], pb[4][VE];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (sp0 + i < splits) {
            load_floats<float, VE>(from + (sp0 + i) * apart + VE * j, pa[i]);
            load_floats<float, VE>(from + (sp0 + i) * apart + half + VE * j, pb[i]);
          }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (sp0 + i < splits) {
#pragma unroll
            for (int e = 0; e < VE; ++e) {
              a[e] += pa[i][e];
              b[e] += pb[i][e];
            }
          }
        }
      }
    } else {
#pragma unroll
      for (int e = 0; e < VE; ++e) {
        a[e] = to_float(lo[t][e]);
        b[e] = to_float(hi[t][e]);
      }
    }
    int64_t page = 0, off = 0;
    int kv_head = 0;
    if (!is_q) {
      if (slot < 0) continue;
      kv_head = is_k ? head - nq : head - nq - nkv;
      page = slot / page_size;
      off = slot % page_size;
      if (!is_k) {
        T* vdst = v_pages + (page * nkv + kv_head) * d * page_size + off;
#pragma unroll
        for (int e = 0; e < VE; ++e) {
          vdst[(int64_t)(VE * j + e) * page_size] = from_float<T>(a[e]);
          vdst[(int64_t)(half + VE * j + e) * page_size] = from_float<T>(b[e]);
        }
        continue;
      }
    }
    if (q_weight) {
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < VE; ++e) ss += a[e] * a[e] + b[e] * b[e];
      for (int step = per_head / 2; step > 0; step >>= 1) ss += __shfl_xor(ss, step, WAVE);
      inv = 1.0f / sqrtf(ss / (float)d + eps);
#pragma unroll
      for (int e = 0; e < VE; ++e) {
        a[e] = a[e] * inv * (is_q ? wq[0][e] : wk[0][e]);
        b[e] = b[e] * inv * (is_q ? wq[1][e] : wk[1][e]);
      }
    }
    vec out_lo, out_hi;
    if (rot_half) {
#pragma unroll
      for (int e = 0; e < VE; ++e) {
        out_lo[e] = from_float<T>(a[e] * c[e] - b[e] * sn[e]);
        out_hi[e] = from_float<T>(b[e] * c[e] + a[e] * sn[e]);
      }
    } else {
#pragma unroll
      for (int e = 0; e < VE; ++e) {
        out_lo[e] = from_float<T>(a[e]);
        out_hi[e] = from_float<T>(b[e]);
      }
    }
    T* dst = is_q ? src : k_pages + ((page * nkv + kv_head) * page_size + off) * d;
    *(vec*)(dst + VE * j) = out_lo;
    *(vec*)(dst + half + VE * j) = out_hi;
  }
}

LRS_API int lrs_compute_units();

static int qk_prep_launch(void* qkv, int dtype, int tokens, int row_stride, int nq, int nkv, int d,
                          const void* q_weight, const void* k_weight, int w_dtype, float eps,
                          const float* cosv, const float* sinv, int rot_half, void* k_pages,
                          void* v_pages, const int* slots, int page_size, void* stream,
                          const float* sums, int splits, int sum_columns, int skip_q = 0) {
  LRS_REQUIRE(!skip_q || (nkv > 0 && !sums), "qk_prep: leaving the q heads alone needs k and v heads to prepare, and no sums");
  LRS_REQUIRE(tokens > 0 && nq > 0 && nkv >= 0 && d > 0, "qk_prep: bad sizes tokens=%d nq=%d nkv=%d d=%d", tokens, nq, nkv, d);
  LRS_REQUIRE(rot_half >= 0 && 2 * rot_half <= d, "qk_prep: rotary width %d exceeds head_dim %d", 2 * rot_half, d);
  LRS_REQUIRE(rot_half == 0 || (cosv && sinv), "qk_prep: rotation asked for without tables");
  LRS_REQUIRE((q_weight == nullptr) == (k_weight == nullptr), "qk_prep: q and k norm weights must come together");
  LRS_REQUIRE(nkv == 0 || (k_pages && v_pages && slots && page_size > 0), "qk_prep: cache write needs pages, slots and a page size");
  LRS_REQUIRE(row_stride >= (nq + 2 * nkv) * d, "qk_prep: row stride %d too small", row_stride);
  dim3 grid(tokens, nq + 2 * nkv), block(WAVE);
  hipStream_t s = (hipStream_t)stream;
  // many tokens: the values are written in whole runs of slots, by workgroups of their own
  const size_t elem = dtype == LRS_F32 ? 4 : 2;
  const int ve = (int)(16 / elem);
  const bool values_apart = !sums && nkv > 0 && tokens >= 128 && page_size % ve == 0 && ((uintptr_t)v_pages % 16) == 0;
  const int per_head = d / (2 * ve);
  const bool vectors = d % (2 * ve) == 0 && per_head <= 64 && (per_head & (per_head - 1)) == 0 && (rot_half == 0 || 2 * rot_half == d) &&
                       row_stride % ve == 0 && ((uintptr_t)qkv % 16) == 0 && ((uintptr_t)k_pages % 16) == 0 &&
                       ((uintptr_t)q_weight % 16) == 0 && ((uintptr_t)k_weight % 16) == 0 && ((uintptr_t)cosv % 16) == 0 &&
                       ((uintptr_t)sinv % 16) == 0;
  if (vectors) {
    const int heads = nq + (values_apart ? nkv : 2 * nkv);    // heads the (token, head) pairs run over
    // heads of one token that a group of threads takes in turn: the largest of 5, 4, 2 that divides them, for
    // steps of many tokens (a decode step has too few groups to fill the chip as it is)
    const int first_head = skip_q ? nq : 0, taken = heads - first_head;
    // ... as long as that leaves two workgroups for every compute unit
    const int per_block = 256 / per_head;
    int together = 1;
    if (tokens >= 128 && !sums)
      for (int many : {5, 4, 2})
        if (taken % many == 0 && (int64_t)tokens * (taken / many) / per_block >= 2 * lrs_compute_units()) {
          together = many;
          break;
        }
    const int64_t pairs = (int64_t)tokens * (taken / together);
    const int64_t prep_blocks = (pairs + per_block - 1) / per_block;
    const int64_t value_blocks = values_apart ? (int64_t)((tokens + 15) / 16) * nkv : 0;
    LRS_REQUIRE(prep_blocks + value_blocks < (1ll << 31), "qk_prep: %d tokens are too many for one launch", tokens);
    dim3 vgrid((unsigned)(prep_blocks + value_blocks));
#define LAUNCH_VEC_OF(T, TW, TOGETHER)                                                                                   \
  qk_prep_vec_kernel<T, TW, TOGETHER><<<vgrid, 256, 0, s>>>((T*)qkv, row_stride, tokens, heads, nq, nkv, d, (const TW*)q_weight, \
                                                            (const TW*)k_weight, eps, cosv, sinv, rot_half, (T*)k_pages,   \
                                                            (T*)v_pages, slots, page_size, (int)prep_blocks, sums, splits, sum_columns, first_head)
#define LAUNCH_VEC(T, TW)                        \
  do {                                           \
    if (together == 5) LAUNCH_VEC_OF(T, TW, 5);  \
    else if (together == 4) LAUNCH_VEC_OF(T, TW, 4); \
    else if (together == 2) LAUNCH_VEC_OF(T, TW, 2); \
    else LAUNCH_VEC_OF(T, TW, 1);                \
  } while (0)
    if (dtype == LRS_F32 && w_dtype == LRS_F32) LAUNCH_VEC(float, float);
    else if (dtype == LRS_BF16 && w_dtype == LRS_BF16) LAUNCH_VEC(bf16, bf16);
    else if (dtype == LRS_BF16 && w_dtype == LRS_F32) LAUNCH_VEC(bf16, float);
    else if (dtype == LRS_F32 && w_dtype == LRS_BF16) LAUNCH_VEC(float, bf16);
    else return lrs_fail("qk_prep: unknown dtypes %d/%d", dtype, w_dtype);
#undef LAUNCH_VEC
#undef LAUNCH_VEC_OF
    return lrs_check_launch("qk_prep");
  }
  LRS_REQUIRE(!sums, "qk_prep: the sums of K splits need the shape the vector kernel takes (head_dim %d, rotation over %d)", d, 2 * rot_half);
  if (values_apart) {
    dim3 vgrid((tokens + 15) / 16, nkv);
    if (dtype == LRS_F32)
      values_to_pages_kernel<float><<<vgrid, 256, 0, s>>>((const float*)qkv, row_stride, (nq + nkv) * d, tokens, nkv, d, (float*)v_pages, slots, page_size);
    else if (dtype == LRS_BF16)
      values_to_pages_kernel<bf16><<<vgrid, 256, 0, s>>>((const bf16*)qkv, row_stride, (nq + nkv) * d, tokens, nkv, d, (bf16*)v_pages, slots, page_size);
    else
      return lrs_fail("qk_prep: unknown dtype %d", dtype);
    if (lrs_check_launch("values_to_pages")) return 1;
    v_pages = nullptr;
    grid.y = nq + nkv;
  }
  if (skip_q) grid.y -= nq;
#define LAUNCH(T, TW)                                                                          \
  qk_prep_kernel<T, TW><<<grid, block, 0, s>>>((T*)qkv, row_stride, nq, nkv, d, (const TW*)q_weight, \
                                               (const TW*)k_weight, eps, cosv, sinv, rot_half,  \
                                               (T*)k_pages, (T*)v_pages, slots, page_size, skip_q ? nq : 0)
  if (dtype == LRS_F32 && w_dtype == LRS_F32) LAUNCH(float, float);
  else if (dtype == LRS_BF16 && w_dtype == LRS_BF16) LAUNCH(bf16, bf16);
  else if (dtype == LRS_BF16 && w_dtype == LRS_F32) LAUNCH(bf16, float);
  else if (dtype == LRS_F32 && w_dtype == LRS_BF16) LAUNCH(float, bf16);
  else return lrs_fail("qk_prep: unknown dtypes %d/%d", dtype, w_dtype);
#undef LAUNCH
  return lrs_check_launch("qk_prep");
}

LRS_API int lrs_qk_prep(void* qkv, int dtype, int tokens, int row_stride, int nq, int nkv, int d,
                        const void* q_weight, const void* k_weight, int w_dtype, float eps,
                        const float* cosv, const float* sinv, int rot_half, void* k_pages,
                        void* v_pages, const int* slots, int page_size, int skip_q, void* stream) {
  return qk_prep_launch(qkv, dtype, tokens, row_stride, nq, nkv, d, q_weight, k_weight, w_dtype, eps, cosv, sinv, rot_half, k_pages,
                        v_pages, slots, page_size, stream, nullptr, 0, 0, skip_q);
}

// The same from the float32 sums that the K splits of the q/k/v product left, sums [splits, tokens, (nq + 2 nkv) d]:
// they are added up on the way, so no kernel of its own has to.  qkv receives the prepared q heads.
LRS_API int lrs_qk_prep_from_sums(void* qkv, int dtype, int tokens, int row_stride, int nq, int nkv, int d,
                                  const void* q_weight, const void* k_weight, int w_dtype, float eps,
                                  const float* cosv, const float* sinv, int rot_half, void* k_pages,
                                  void* v_pages, const int* slots, int page_size, const float* sums, int splits, void* stream) {
  LRS_REQUIRE(sums != nullptr && splits > 0 && ((uintptr_t)sums % 16) == 0, "qk_prep_from_sums: needs the sums and their number");
  return qk_prep_launch(qkv, dtype, tokens, row_stride, nq, nkv, d, q_weight, k_weight, w_dtype, eps, cosv, sinv, rot_half, k_pages,
                        v_pages, slots, page_size, stream, sums, splits, (nq + 2 * nkv) * d);
}

// ----------------------------------------------------------- gated activation
// out[t, i] = silu(gate) * up, silu evaluated in float32.  Plain layout: gate = gu[t, i],
// up = gu[t, inter + i].  Interleaved layout (groups of 8 gate columns followed by the 8 up
// columns of the same features): gate = gu[t, 16*(i/8) + i%8], up = the column 8 further on.
template <typename T>
__global__ void silu_mul_kernel(T* __restrict__ out, const T* __restrict__ gu, int inter, int64_t total,
                                int interleaved) {
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = idx / inter, i = idx % inter;
    const int64_t gate_at = interleaved ? t * 2 * inter + 16 * (i / 8) + i % 8 : t * 2 * inter + i;
    const float g = to_float(gu[gate_at]);
    const float u = to_float(gu[gate_at + (interleaved ? 8 : inter)]);
    out[idx] = from_float<T>(g / (1.0f + expf(-g)) * u);
  }
}

// Interleaved bf16 layout, 8 features per thread: 16 bytes of gate and 16 bytes of up in, 16 bytes out.
__global__ void silu_mul_interleaved_bf16_kernel(bf16* __restrict__ out, const bf16* __restrict__ gu, int64_t groups) {
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < groups;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const bf16x8 g = *(const bf16x8*)(gu + idx * 16), u = *(const bf16x8*)(gu + idx * 16 + 8);
    bf16x8 r;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float gv = (float)g[i];
      r[i] = (bf16)(gv / (1.0f + expf(-gv)) * (float)u[i]);
    }
    *(bf16x8*)(out + idx * 8) = r;
  }
}

LRS_API int lrs_silu_mul(void* out, const void* gu, int dtype, int tokens, int inter, int interleaved, void* stream) {
  LRS_REQUIRE(tokens > 0 && inter > 0, "silu_mul: tokens=%d inter=%d must be positive", tokens, inter);
  LRS_REQUIRE(!interleaved || inter % 8 == 0, "silu_mul: the interleaved layout needs inter %% 8 == 0, got %d", inter);
  const int64_t total = (int64_t)tokens * inter;
  const int blocks = (int)((total + 255) / 256 < 65536 ? (total + 255) / 256 : 65536);
  hipStream_t s = (hipStream_t)stream;
  if (interleaved && dtype == LRS_BF16 && ((uintptr_t)gu % 16) == 0 && ((uintptr_t)out % 16) == 0) {
    const int64_t groups = total / 8;
    const int vec_blocks = (int)((groups + 255) / 256 < 16384 ? (groups + 255) / 256 : 16384);
    silu_mul_interleaved_bf16_kernel<<<vec_blocks, 256, 0, s>>>((bf16*)out, (const bf16*)gu, groups);
    return lrs_check_launch("silu_mul");
  }
  if (dtype == LRS_F32)
    silu_mul_kernel<float><<<blocks, 256, 0, s>>>((float*)out, (const float*)gu, inter, total, interleaved);
  else if (dtype == LRS_BF16)
    silu_mul_kernel<bf16><<<blocks, 256, 0, s>>>((bf16*)out, (const bf16*)gu, inter, total, interleaved);
  else
    return lrs_fail("silu_mul: unknown dtype %d", dtype);
  return lrs_check_launch("silu_mul");
}

// -------------------------------------------------------------- residual add
// residual[i] += y[i]: the float32 residual stream takes the output of a product that was
// computed into the activation dtype.
template <typename T>
__global__ void add_into_kernel(float* __restrict__ residual, const T* __restrict__ y, int64_t total) {
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x)
    residual[idx] += to_float(y[idx]);
}

__global__ void add_into_bf16x8_kernel(float* __restrict__ residual, const bf16* __restrict__ y, int64_t groups) {
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < groups;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const bf16x8 v = *(const bf16x8*)(y + idx * 8);
    floatx4 a = *(floatx4*)(residual + idx * 8), b = *(floatx4*)(residual + idx * 8 + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a[i] += (float)v[i];
      b[i] += (float)v[4 + i];
    }
    *(floatx4*)(residual + idx * 8) = a;
    *(floatx4*)(residual + idx * 8 + 4) = b;
  }
}

LRS_API int lrs_add_into(float* residual, const void* y, int dtype, int64_t total, void* stream) {
  LRS_REQUIRE(total > 0, "add_into: nothing to add");
  const int blocks = (int)((total + 255) / 256 < 65536 ? (total + 255) / 256 : 65536);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == LRS_BF16 && total % 8 == 0 && ((uintptr_t)y % 16) == 0 && ((uintptr_t)residual % 16) == 0) {
    const int64_t groups = total / 8;
    const int vec_blocks = (int)((groups + 255) / 256 < 16384 ? (groups + 255) / 256 : 16384);
    add_into_bf16x8_kernel<<<vec_blocks, 256, 0, s>>>(residual, (const bf16*)y, groups);
    return lrs_check_launch("add_into");
  }
  if (dtype == LRS_F32) add_into_kernel<float><<<blocks, 256, 0, s>>>(residual, (const float*)y, total);
  else if (dtype == LRS_BF16) add_into_kernel<bf16><<<blocks, 256, 0, s>>>(residual, (const bf16*)y, total);
  else return lrs_fail("add_into: unknown dtype %d", dtype);
  return lrs_check_launch("add_into");
}

// ------------------------------------------------------------------ utilities
__global__ void fill_i32_kernel(int* dst, int value, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = value;
}
// ------------------------------------------------------------ scale_rows
// out[r, :] = x[r, :] * rsqrt(sum_p sumsq[p, r] / hidden + eps): finishes an RMSNorm whose input a
// matrix product left as bf16(h * weight) together with partial sums of h^2 (see gemm.hip), for a
// consumer that wants the normalised rows as a tensor.
__global__ __launch_bounds__(256) void scale_rows_kernel(bf16* __restrict__ out, const bf16* __restrict__ x,
                                                         const float* __restrict__ sumsq, int parts, int rows,
                                                         int hidden, float eps) {
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  float q = 0.f;
  for (int p = threadIdx.x; p < parts; p += blockDim.x) q += sumsq[(int64_t)p * rows + row];
  const float scale = 1.0f / sqrtf(block_sum(q, scratch) / (float)hidden + eps);
  for (int c = threadIdx.x; c < hidden; c += blockDim.x)
    out[(int64_t)row * hidden + c] = (bf16)((float)x[(int64_t)row * hidden + c] * scale);
}

LRS_API int lrs_scale_rows(void* out, const void* x, const float* sumsq, int parts, int rows, int hidden, float eps,
                           void* stream) {
  LRS_REQUIRE(rows > 0 && hidden > 0 && parts > 0 && eps > 0.f, "scale_rows: rows=%d hidden=%d parts=%d eps=%g must be positive", rows, hidden, parts, (double)eps);
  scale_rows_kernel<<<rows, 256, 0, (hipStream_t)stream>>>((bf16*)out, (const bf16*)x, sumsq, parts, rows, hidden, eps);
  return lrs_check_launch("scale_rows");
}

// ---------------------------------------------------- next decode step's metadata
// Several decode steps can run from one launch: between two of them the step's metadata is moved
// on by the device itself.  Each of the first *real_rows rows (the others pad the batch) takes the
// token just chosen for it, moves one position on, lengthens its request by one and counts the draw
// (`draws`, optional: the per-row counters of seeded sampling) ...
__global__ void advance_decode_kernel(int* __restrict__ token_ids, int* __restrict__ positions,
                                      const int* __restrict__ token_request, int* __restrict__ seq_lens,
                                      const int* __restrict__ chosen, int* __restrict__ draws,
                                      const int* __restrict__ real_rows, int rows) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= rows || t >= *real_rows) return;
  token_ids[t] = chosen[t] >= 0 ? chosen[t] : 0;     // -1: a row whose logits were not finite (the host raises when it reads it)
  positions[t] += 1;
  seq_lens[token_request[t]] += 1;
  if (draws) draws[t] += 1;
}

// ... and, per cache group, finds the slot of its new position in its request's block table.
__global__ void advance_slots_kernel(int* __restrict__ slots, const int* __restrict__ positions,
                                     const int* __restrict__ token_request, const int* __restrict__ block_table,
                                     int table_stride, int page_size, const int* __restrict__ real_rows, int rows) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= rows || t >= *real_rows) return;
  const int pos = positions[t];
  const int page = block_table[(int64_t)token_request[t] * table_stride + pos / page_size];
  slots[t] = page >= 0 ? page * page_size + pos % page_size : -1;
}

LRS_API int lrs_advance_decode(int* token_ids, int* positions, const int* token_request, int* seq_lens, const int* chosen,
                               int* draws, const int* real_rows, int rows, void* stream) {
  LRS_REQUIRE(rows > 0 && token_ids && positions && token_request && seq_lens && chosen && real_rows, "advance_decode: missing arrays or no rows");
  advance_decode_kernel<<<(rows + 255) / 256, 256, 0, (hipStream_t)stream>>>(token_ids, positions, token_request, seq_lens, chosen, draws, real_rows, rows);
  return lrs_check_launch("advance_decode");
}

LRS_API int lrs_advance_slots(int* slots, const int* positions, const int* token_request, const int* block_table,
                              int table_stride, int page_size, const int* real_rows, int rows, void* stream) {
  LRS_REQUIRE(rows > 0 && page_size > 0 && slots && positions && token_request && block_table && real_rows, "advance_slots: missing arrays or no rows");
  advance_slots_kernel<<<(rows + 255) / 256, 256, 0, (hipStream_t)stream>>>(slots, positions, token_request, block_table, table_stride, page_size, real_rows, rows);
  return lrs_check_launch("advance_slots");
}

// dst[pairs[2 i]] = pairs[2 i + 1] for i < count: the block table entries that changed on the host since the
// last step, written into the device's tables.  The host has checked every offset against the tables' size.
__global__ void scatter_i32_kernel(int* __restrict__ dst, const int* __restrict__ pairs, int count) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) dst[pairs[2 * i]] = pairs[2 * i + 1];
}

LRS_API int lrs_scatter_i32(int* dst, const int* pairs, int count, void* stream) {
  LRS_REQUIRE(count > 0 && dst && pairs, "scatter_i32: needs a destination, pairs and a positive count");
  scatter_i32_kernel<<<(count + 255) / 256, 256, 0, (hipStream_t)stream>>>(dst, pairs, count);
  return lrs_check_launch("scatter_i32");
}

LRS_API int lrs_fill_i32(int* dst, int value, int64_t n, void* stream) {
  LRS_REQUIRE(n > 0, "fill: n must be positive");
  const int blocks = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
  fill_i32_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>(dst, value, n);
  return lrs_check_launch("fill_i32");
}

// Copies picked float32 rows: out[i] = x[rows[i]].
__global__ void gather_rows_kernel(float* __restrict__ out, const float* __restrict__ x,
                                   const int* __restrict__ rows, int hidden) {
  const float* src = x + (int64_t)rows[blockIdx.x] * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) out[(int64_t)blockIdx.x * hidden + i] = src[i];
}
LRS_API int lrs_gather_rows(float* out, const float* x, const int* rows, int n_rows, int hidden, void* stream) {
  LRS_REQUIRE(n_rows > 0 && hidden > 0, "gather_rows: bad sizes");
  gather_rows_kernel<<<n_rows, 256, 0, (hipStream_t)stream>>>(out, x, rows, hidden);
  return lrs_check_launch("gather_rows");
}
