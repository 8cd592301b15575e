// Causal attention over the paged cache for a ragged batch: every query token attends to
// the cached keys of its own request at positions lo..p, p being the token's absolute
// position and lo = max(0, p - window + 1) when a window is given.  Keys and values of this
// step's tokens are already in the cache when these kernels run.
//
// Key pages are [page, kv_head, slot, dim], value pages [page, kv_head, dim, slot] (transposed
// inside a page); block_table[r, i] is the page holding positions i*page_size ..
// (i+1)*page_size-1 of request r.  Scores, softmax and the weighted sum are
// float32.  Key tiles start at multiples of the tile size counted from position 0, so the
// rounding of a query's result depends on its position only, never on how the sequence
// was cut into steps.
#include <type_traits>

#include "common.h"

// 2^x by the hardware instruction alone (arguments here are <= 0 or -inf; results below the
// smallest normal number may flush to zero, which a softmax weight can afford).
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// How far (in powers of two) a new maximum must exceed the reference point of a running softmax
// before the reference point moves and the accumulators are rescaled.
constexpr float RESCALE_STEP = 8.0f;

// ---------------------------------------------------------- generic kernel
// One workgroup per (query token, query head); any head_dim up to 4 * threads.
template <typename T, int THREADS>
__global__ __launch_bounds__(THREADS) void attention_generic_kernel(
    T* __restrict__ out, int out_stride, const T* __restrict__ q, int q_stride,
    const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    const int* __restrict__ block_table, int table_stride, const int* __restrict__ token_request,
    const int* __restrict__ positions, int nq, int nkv, int d, int page_size, float scale,
    int window) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  float* qs = smem;                           // [d]
  float* probs = qs + d + d % 2;              // [THREADS]
  int64_t* bases = (int64_t*)(probs + THREADS);  // [THREADS] element offset of each key's (page, kv head) block
  int* offsets = (int*)(bases + THREADS);        // [THREADS] slot of each key inside its page
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
    const int off = key % page_size;
    if (valid) {
      const int64_t page = table[key / page_size];
      base = (page * nkv + kv_head) * page_size * d;
      const T* kr = k_pages + base + (int64_t)off * d;
      float dot = 0.f;
      if (sizeof(T) == 4 && d % 4 == 0 && ((uintptr_t)k_pages % 16) == 0) {
        // float32 rows, 16 bytes a load; the products are added up in the same order as one by one
        for (int i = 0; i < d; i += 4) {
          const floatx4 kv = *(const floatx4*)((const float*)kr + i);
          dot = fmaf(qs[i], kv[0], dot);
          dot = fmaf(qs[i + 1], kv[1], dot);
          dot = fmaf(qs[i + 2], kv[2], dot);
          dot = fmaf(qs[i + 3], kv[3], dot);
        }
      } else {
        for (int i = 0; i < d; ++i) dot = fmaf(qs[i], to_float(kr[i]), dot);
      }
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
    offsets[tid] = off;
    __syncthreads();
    const int count = (pos - tile + 1 < THREADS) ? pos - tile + 1 : THREADS;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int dim = tid + c * THREADS;
      if (dim < d) {
        float a = acc[c] * alpha;
        if (sizeof(T) == 4 && page_size % 4 == 0 && THREADS % 4 == 0 && ((uintptr_t)v_pages % 16) == 0) {
          // four keys that lie side by side in a (transposed) page in one load of 16 bytes; added in key order as below
          int j = 0;
          for (; j + 4 <= count; j += 4) {
            if (tile + j < lo) {                                 // keys before the window have no page to read from
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                const float pj = probs[j + e];
                if (pj != 0.f) a = fmaf(pj, to_float(v_pages[bases[j + e] + (int64_t)dim * page_size + offsets[j + e]]), a);
              }
              continue;
            }
            const floatx4 vv = *(const floatx4*)((const float*)v_pages + bases[j] + (int64_t)dim * page_size + offsets[j]);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float pj = probs[j + e];
              if (pj != 0.f) a = fmaf(pj, vv[e], a);
            }
          }
          for (; j < count; ++j) {
            const float pj = probs[j];
            if (pj != 0.f) a = fmaf(pj, to_float(v_pages[bases[j] + (int64_t)dim * page_size + offsets[j]]), a);
          }
        } else {
          for (int j = 0; j < count; ++j) {
            const float pj = probs[j];
            if (pj != 0.f) a = fmaf(pj, to_float(v_pages[bases[j] + (int64_t)dim * page_size + offsets[j]]), a);
          }
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

// ------------------------------------------------- bf16 decode kernel
// What the decode kernel does to raw q, k and v rows when it also does the work of qk_prep: the
// per-head RMSNorm of q and k (weights null: none), the rotation of pairs (i, i + D/2) by the
// step's cos/sin tables (null: none) and the write of the new key and value into the pages.
struct DecodePrep {
  const void* q_weight;   // [D]
  const void* k_weight;   // [D]
  int weight_is_f32;
  float eps;
  const float* cosv;      // [tokens, D/2]
  const float* sinv;
  int kv_columns;         // kv heads held in the qkv rows after the q heads: k, then v; 0: keys and
                          // values are another layer's, already in the pages
};

// One head row, raw -> normalised and rotated, in the operand layout of the 16x16x32 products: the
// lane holds dims c*32 + g*8 .. +8 of every 32-dim chunk c, the four lanes g = 0..3 with equal
// lane % 16 hold one head between them.  All 64 lanes must call it together.
// head_from_values: the same from values already in registers (a row asked for earlier, so that its trip to memory
// ran beside other work).
template <int D>
__device__ __forceinline__ void head_from_values(bf16x8 (&r)[D / 32], float (&x)[D / 32][8], int g,
                                                 const void* __restrict__ weight, int weight_is_f32, float eps,
                                                 const float* __restrict__ cosrow, const float* __restrict__ sinrow) {
  constexpr int DS = D / 32;
  // weights and tables come in 16-byte loads (the host checks their alignment)
  if (weight) {
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < DS; ++c)
#pragma unroll
      for (int j = 0; j < 8; ++j) ss = fmaf(x[c][j], x[c][j], ss);
    ss += __shfl_xor(ss, 16, WAVE);
    ss += __shfl_xor(ss, 32, WAVE);
    const float inv = 1.0f / sqrtf(ss / (float)D + eps);
#pragma unroll
    for (int c = 0; c < DS; ++c) {
      float w[8];
      if (weight_is_f32) {
        const floatx4 w0 = *(const floatx4*)((const float*)weight + c * 32 + g * 8), w1 = *(const floatx4*)((const float*)weight + c * 32 + g * 8 + 4);
#pragma unroll
        for (int j = 0; j < 4; ++j) { w[j] = w0[j]; w[4 + j] = w1[j]; }
      } else {
        const bf16x8 wb = *(const bf16x8*)((const bf16*)weight + c * 32 + g * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j) w[j] = (float)wb[j];
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) x[c][j] = x[c][j] * inv * w[j];
    }
  }
  if (cosrow) {
#pragma unroll
    for (int c = 0; c < DS / 2; ++c) {
      const floatx4 c0 = *(const floatx4*)(cosrow + c * 32 + g * 8), c1 = *(const floatx4*)(cosrow + c * 32 + g * 8 + 4);
      const floatx4 s0 = *(const floatx4*)(sinrow + c * 32 + g * 8), s1 = *(const floatx4*)(sinrow + c * 32 + g * 8 + 4);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float cs = j < 4 ? c0[j & 3] : c1[j & 3], sn = j < 4 ? s0[j & 3] : s1[j & 3];
        const float a = x[c][j], b = x[c + DS / 2][j];
        x[c][j] = a * cs - b * sn;
        x[c + DS / 2][j] = b * cs + a * sn;
      }
    }
  }
#pragma unroll
  for (int c = 0; c < DS; ++c)
#pragma unroll
    for (int j = 0; j < 8; ++j) r[c][j] = (bf16)x[c][j];
}

template <int D>
__device__ __forceinline__ void prepare_head(bf16x8 (&r)[D / 32], const bf16* __restrict__ head, int g,
                                             const void* __restrict__ weight, int weight_is_f32, float eps,
                                             const float* __restrict__ cosrow, const float* __restrict__ sinrow) {
  float x[D / 32][8];
#pragma unroll
  for (int c = 0; c < D / 32; ++c) {
    const bf16x8 raw = *(const bf16x8*)(head + c * 32 + g * 8);
#pragma unroll
    for (int j = 0; j < 8; ++j) x[c][j] = (float)raw[j];
  }
  head_from_values<D>(r, x, g, weight, weight_is_f32, eps, cosrow, sinrow);
}

// One query token per request (a decode step).  A workgroup of four waves owns one
// (token, kv head, split): the query heads that share the kv head (at most 16) sit in the
// columns of the matrix-core tiles, so every key and value is loaded once for the whole
// group.  Keys are walked in tiles of 32; the tiles of a token are divided between `splits`
// workgroups (so that few long requests still fill the chip) and, inside a workgroup,
// dealt to the waves in turn.  Per tile:
//     S[key, head]   = K[key, :] . Q[head, :]          A = K rows (16 keys x 32 dims per MFMA)
//     P              = exp2(S * scale*log2(e) - max)   online softmax per head column
//     O^T[dim, head] += V^T[dim, key] . P[key, head]   A = V^T rows, read from the transposed page
// S comes out of the first product with a head per lane column and four keys per lane, which
// is exactly the operand layout the second product wants for P, so P never leaves registers.
// Waves are merged through LDS, splits by attention_merge_kernel.
// PREP: q holds the raw rows of the q/k/v product; the kernel prepares q itself, and the wave that
// meets the token's own position prepares the new key, takes it and the new value in place of what
// the pages hold there, and writes both into the pages (see DecodePrep).
template <int D, bool PREP, int WAVES, bool AHEAD>
__global__ __launch_bounds__(WAVES * 64) void attention_decode_bf16_kernel(
    bf16* __restrict__ out, int out_stride, float* __restrict__ part_o, float* __restrict__ part_ml,
    const bf16* __restrict__ q, int q_stride, bf16* __restrict__ k_pages,
    bf16* __restrict__ v_pages, const int* __restrict__ block_table, int table_stride,
    const int* __restrict__ token_request, const int* __restrict__ positions, int nq, int nkv,
    int page_size, float scale, int window, int splits, DecodePrep prep) {
  constexpr int DS = D / 32, DB = D / 16, THREADS = WAVES * 64;
  __shared__ float sm_m[WAVES][16], sm_l[WAVES][16];
  __shared__ float sm_o[WAVES][D][16];
  const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
  const int col = lane & 15, g = lane >> 4;
  const int split = blockIdx.x, kvh = blockIdx.y, token = blockIdx.z;
  const int group = nq / nkv;
  const int pos = positions[token];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int* table = block_table + (int64_t)token_request[token] * table_stride;
  const int first_tile = lo / 32, last_tile = pos / 32;
  const int per_split = (last_tile - first_tile + splits) / splits;
  const int tile_begin = first_tile + split * per_split;
  const int tile_end = tile_begin + per_split <= last_tile + 1 ? tile_begin + per_split : last_tile + 1;
  // PREP: the wave that may have to prepare the token's new key asks for the raw key and value rows now, before
  // anything here waits for memory: the rows are then there when their turn comes, two trips to memory later
  // (they are the token's own, whichever workgroup turns out to walk its position)
  const bf16* q_row = q + (int64_t)token * q_stride;
  bf16x8 raw_k[DS];
  bf16 raw_v[(D + WAVE - 1) / WAVE];
  if constexpr (PREP) {
    if (prep.kv_columns > 0 && wave == WAVES - 1) {
#pragma unroll
      for (int c = 0; c < DS; ++c) raw_k[c] = *(const bf16x8*)(q_row + (int64_t)(nq + kvh) * D + c * 32 + g * 8);
      const bf16* v_row = q_row + (int64_t)(nq + prep.kv_columns + kvh) * D;
#pragma unroll
      for (int n = 0; n < (D + WAVE - 1) / WAVE; ++n)
        if (lane + n * WAVE < D) raw_v[n] = v_row[lane + n * WAVE];
    }
  }

  // the block table entries of this workgroup's tiles, in LDS: the address of a key must not
  // wait for a trip to memory of its own
  extern __shared__ int page_ids[];
  const int first_block = tile_begin * 32 / page_size;
  const int last_key = tile_end * 32 - 1 < pos ? tile_end * 32 - 1 : pos;
  if (tile_begin < tile_end)
    for (int i = tid; i <= last_key / page_size - first_block; i += THREADS) page_ids[i] = table[first_block + i];

  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  // Every key and value fragment of a tile is requested before any is used, so a tile costs one
  // trip to memory instead of two.  Which of the tile's 32 keys a row of the two key blocks stands
  // for is chosen so that a lane ends up with the weights of eight consecutive keys, g*8 .. g*8+7:
  // block h, row 4*r + i is key 8*r + 4*h + i.  The values of those eight keys lie side by side in
  // the (transposed) page, one 16-byte load a dim.
  const int key_of_row = (col >> 2) * 8 + (col & 3);           // + 4*h
  auto fetch = [&](int tile, bf16x8 (&kf)[2][DS], bf16x8 (&vf)[DB]) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int key = tile * 32 + key_of_row + 4 * h;
      if (key <= pos && key >= lo) {
        const int64_t page = page_ids[key / page_size - first_block];
        const bf16* kp = k_pages + ((page * nkv + kvh) * page_size + key % page_size) * D + g * 8;
#pragma unroll
        for (int c = 0; c < DS; ++c) kf[h][c] = *(const bf16x8*)(kp + c * 32);
      } else {
#pragma unroll
        for (int c = 0; c < DS; ++c) kf[h][c] = zero8;
      }
    }
    const int key8 = tile * 32 + g * 8;                        // this lane's eight keys; pages hold multiples of 16
    if (key8 <= pos && key8 + 7 >= lo) {
      const int64_t page = page_ids[key8 / page_size - first_block];
      const bf16* vp = v_pages + (page * nkv + kvh) * (int64_t)D * page_size + (int64_t)col * page_size + key8 % page_size;
#pragma unroll
      for (int b = 0; b < DB; ++b) vf[b] = *(const bf16x8*)(vp + (int64_t)b * 16 * page_size);
    } else {
#pragma unroll
      for (int b = 0; b < DB; ++b) vf[b] = zero8;
    }
  };
  // AHEAD: the wave's first tile is asked for as soon as the page ids are there, before the query (and
  // the new key) are prepared, so that the first trip to memory runs beside that work.
  bf16x8 kf_a[AHEAD ? 2 : 1][AHEAD ? DS : 1], vf_a[AHEAD ? DB : 1];
  if constexpr (AHEAD) {
    __syncthreads();
    if (tile_begin + wave < tile_end) fetch(tile_begin + wave, (bf16x8(&)[2][DS])kf_a, (bf16x8(&)[DB])vf_a);
  }
  bf16x8 qf[DS];
  if (PREP) {
    const float* cosrow = prep.cosv ? prep.cosv + (int64_t)token * (D / 2) : nullptr;
    const float* sinrow = prep.sinv ? prep.sinv + (int64_t)token * (D / 2) : nullptr;
    prepare_head<D>(qf, q_row + (int64_t)(kvh * group + (col < group ? col : 0)) * D, g, prep.q_weight, prep.weight_is_f32,
                    prep.eps, cosrow, sinrow);
#pragma unroll
    for (int c = 0; c < DS; ++c) qf[c] = col < group ? qf[c] : zero8;
  } else {
#pragma unroll
    for (int c = 0; c < DS; ++c)
      qf[c] = col < group ? *(const bf16x8*)(q_row + (int64_t)(kvh * group + col) * D + c * 32 + g * 8) : zero8;
  }
  // The workgroup that walks the token's own position prepares the new key once (its last wave,
  // which is dealt the fewest tiles), leaves it and the new value in LDS for the wave that meets
  // the position, and writes both into the pages.
  __shared__ __attribute__((aligned(16))) bf16 own_k[D];
  __shared__ bf16 own_v[D];
  const bool holds_own = PREP && prep.kv_columns > 0 && tile_begin <= last_tile && last_tile < tile_end;
  if (holds_own && wave == WAVES - 1) {
    bf16x8 kn[DS];
    float kx[DS][8];
#pragma unroll
    for (int c = 0; c < DS; ++c)
#pragma unroll
      for (int j = 0; j < 8; ++j) kx[c][j] = (float)raw_k[c][j];
    head_from_values<D>(kn, kx, g, prep.k_weight, prep.weight_is_f32, prep.eps,
                        prep.cosv ? prep.cosv + (int64_t)token * (D / 2) : nullptr,
                        prep.sinv ? prep.sinv + (int64_t)token * (D / 2) : nullptr);
    // (among this workgroup's entries, since it walks the position; they are in LDS once a barrier has been passed)
    const int64_t page = AHEAD ? page_ids[pos / page_size - first_block] : table[pos / page_size];
    const int off = pos % page_size;
    if (col == 0) {
      bf16* kdst = k_pages + ((page * nkv + kvh) * page_size + off) * D + g * 8;
#pragma unroll
      for (int c = 0; c < DS; ++c) {
        *(bf16x8*)&own_k[c * 32 + g * 8] = kn[c];
        if (page >= 0) *(bf16x8*)(kdst + c * 32) = kn[c];
      }
    }
#pragma unroll
    for (int n = 0; n < (D + WAVE - 1) / WAVE; ++n) {
      const int i = lane + n * WAVE;
      if (i < D) {
        const bf16 vn = raw_v[n];
        own_v[i] = vn;
        if (page >= 0) v_pages[(page * nkv + kvh) * (int64_t)D * page_size + (int64_t)i * page_size + off] = vn;
      }
    }
  }
  __syncthreads();

  floatx4 o[DB];
#pragma unroll
  for (int b = 0; b < DB; ++b) o[b] = floatx4{0.f, 0.f, 0.f, 0.f};
  float run_max = -INFINITY, run_sum = 0.f;
  const float scale2 = scale * 1.4426950408889634f;

  auto work = [&](int tile, bf16x8 (&kf)[2][DS], bf16x8 (&vf)[DB]) {
    if (holds_own && tile == last_tile) {
      // the token's own key and value take the place of what the pages hold at its position
      const int own = pos % 32;
      const int own_h = (own % 8) / 4, own_col = (own / 8) * 4 + own % 4, own_g = own / 8, own_j = own % 8;
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int c = 0; c < DS; ++c)
          if (h == own_h && col == own_col) kf[h][c] = *(const bf16x8*)&own_k[c * 32 + g * 8];
#pragma unroll
      for (int b = 0; b < DB; ++b) {
        const bf16 vn = own_v[b * 16 + col];
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (g == own_g && j == own_j) vf[b][j] = vn;
      }
    }
    floatx4 s[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      s[h] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < DS; ++c) s[h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[h][c], qf[c], s[h], 0, 0, 0);
    }
    float tile_max = -INFINITY;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = tile * 32 + g * 8 + h * 4 + i;
        const bool valid = key <= pos && key >= lo;
        s[h][i] = valid ? s[h][i] * scale2 : -INFINITY;
        tile_max = fmaxf(tile_max, s[h][i]);
      }
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, WAVE));
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, WAVE));
    const float new_max = tile_max > run_max + RESCALE_STEP ? tile_max : run_max;   // see RESCALE_STEP
    const float alpha = fast_exp2(run_max - new_max);
    run_max = new_max;
    bf16x8 pf;
    float tile_sum = 0.f;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = fast_exp2(s[h][i] - new_max);
        tile_sum += p;
        pf[h * 4 + i] = (bf16)p;
      }
    run_sum = run_sum * alpha + tile_sum;
    const bool rescale = __any(alpha != 1.f);
#pragma unroll
    for (int b = 0; b < DB; ++b) {
      if (rescale) o[b] *= alpha;
      o[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[b], pf, o[b], 0, 0, 0);
    }
  };
  if constexpr (AHEAD) {
    // two register sets in turn: the next tile of this wave is on its way while this one is worked on
    bf16x8 (&kf_first)[2][DS] = (bf16x8(&)[2][DS])kf_a;
    bf16x8 (&vf_first)[DB] = (bf16x8(&)[DB])vf_a;
    bf16x8 kf_b[2][DS], vf_b[DB];
    for (int tile = tile_begin + wave; tile < tile_end; tile += 2 * WAVES) {
      if (tile + WAVES < tile_end) fetch(tile + WAVES, kf_b, vf_b);
      work(tile, kf_first, vf_first);
      if (tile + WAVES >= tile_end) break;
      if (tile + 2 * WAVES < tile_end) fetch(tile + 2 * WAVES, kf_first, vf_first);
      work(tile + WAVES, kf_b, vf_b);
    }
  } else {
    for (int tile = tile_begin + wave; tile < tile_end; tile += WAVES) {
      bf16x8 kf[2][DS], vf[DB];
      fetch(tile, kf, vf);
      work(tile, kf, vf);
    }
  }
  run_sum += __shfl_xor(run_sum, 16, WAVE);
  run_sum += __shfl_xor(run_sum, 32, WAVE);
  if (g == 0) {
    sm_m[wave][col] = run_max;
    sm_l[wave][col] = run_sum;
  }
#pragma unroll
  for (int b = 0; b < DB; ++b)
#pragma unroll
    for (int i = 0; i < 4; ++i) sm_o[wave][b * 16 + g * 4 + i][col] = o[b][i];
  __syncthreads();
  for (int e = tid; e < D * 16; e += THREADS) {
    const int dim = e / 16, h = e % 16;
    if (h >= group) continue;
    float top = sm_m[0][h];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) top = fmaxf(top, sm_m[w][h]);
    float acc = 0.f, total = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      const float weight = top == -INFINITY ? 0.f : fast_exp2(sm_m[w][h] - top);
      acc += sm_o[w][dim][h] * weight;
      total += sm_l[w][h] * weight;
    }
    const int head = kvh * group + h;
    if (splits == 1) {
      out[(int64_t)token * out_stride + (int64_t)head * D + dim] = (bf16)(acc / total);
    } else {
      const int64_t slot = ((int64_t)token * nq + head) * splits + split;
      part_o[slot * D + dim] = acc;
      if (dim == 0) {
        part_ml[slot * 2] = top;
        part_ml[slot * 2 + 1] = total;
      }
    }
  }
}

// Merges the partial results of the splits of one (token, head): out = sum_s o_s 2^(m_s - m) / sum_s l_s 2^(m_s - m).
// A kernel of its own on purpose: letting the last workgroup to finish merge inside the decode
// kernel needs a device-wide fence in every workgroup, and on this chip (eight L2s) those fences
// write back and invalidate whole caches; measured, they cost many times what this kernel does.
__global__ void attention_merge_kernel(bf16* __restrict__ out, int out_stride, const float* __restrict__ part_o,
                                       const float* __restrict__ part_ml, int nq, int d, int splits) {
  const int token = blockIdx.x, head = blockIdx.y;
  const int64_t base = ((int64_t)token * nq + head) * splits;
  // Everything is asked for before anything is used: the partial sums of a split do not wait for its maximum
  // (a split that saw no key holds zeros and gets the weight zero), so the kernel is one trip to memory long.
  constexpr int AT_ONCE = 8;
  for (int dim = threadIdx.x; dim < d; dim += blockDim.x) {
    float top = -INFINITY, total = 0.f, acc = 0.f;
    for (int s0 = 0; s0 < splits; s0 += AT_ONCE) {
      float m[AT_ONCE], l[AT_ONCE], o[AT_ONCE];
#pragma unroll
      for (int i = 0; i < AT_ONCE; ++i) {
        const int s = s0 + i < splits ? s0 + i : splits - 1;
        m[i] = part_ml[(base + s) * 2];
        l[i] = part_ml[(base + s) * 2 + 1];
        o[i] = part_o[(base + s) * d + dim];
      }
      float chunk_top = top;
#pragma unroll
      for (int i = 0; i < AT_ONCE; ++i)
        if (s0 + i < splits) chunk_top = fmaxf(chunk_top, m[i]);
      const float keep = top == -INFINITY ? 0.f : fast_exp2(top - chunk_top);   // what was added up so far, against the new maximum
      total *= keep;
      acc *= keep;
      top = chunk_top;
#pragma unroll
      for (int i = 0; i < AT_ONCE; ++i) {
        const float weight = (s0 + i < splits && m[i] > -INFINITY) ? fast_exp2(m[i] - top) : 0.f;
        total += l[i] * weight;
        acc += o[i] * weight;
      }
    }
    out[(int64_t)token * out_stride + (int64_t)head * d + dim] = (bf16)(acc / total);
  }
}

// The same merge for steps of many tokens (prompt portions whose keys were divided): a thread owns four dims of one
// (token, head) and asks for everything it needs at once, 16 bytes a load; workgroups of four waves over all of them,
// where a workgroup a (token, head) would be tens of thousands of workgroups of two waves with a few loads each.  The
// sums are added in split order, as attention_merge_kernel adds them: the same bits.
template <int SPLITS>
__global__ __launch_bounds__(256) void attention_merge_wide_kernel(bf16* __restrict__ out, int out_stride, const float* __restrict__ part_o,
                                                                   const float* __restrict__ part_ml, int64_t quads, int nq, int d) {
  const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= quads) return;
  const int per_head = d / 4;
  const int64_t pair = e / per_head;                 // token * nq + head
  const int dim = (int)(e % per_head) * 4;
  const int64_t base = pair * SPLITS;
  float m[SPLITS], l[SPLITS];
  floatx4 o[SPLITS];
#pragma unroll
  for (int s = 0; s < SPLITS; ++s) {
    const float2 ml = *(const float2*)(part_ml + (base + s) * 2);
    m[s] = ml.x;
    l[s] = ml.y;
    o[s] = *(const floatx4*)(part_o + (base + s) * d + dim);
  }
  float top = -INFINITY;
#pragma unroll
  for (int s = 0; s < SPLITS; ++s) top = fmaxf(top, m[s]);
  float total = 0.f;
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < SPLITS; ++s) {
    const float weight = m[s] > -INFINITY ? fast_exp2(m[s] - top) : 0.f;
    total += l[s] * weight;
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] += o[s][i] * weight;
  }
  const int64_t token = pair / nq, head = pair % nq;
  bf16x4 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) r[i] = (bf16)(acc[i] / total);
  *(bf16x4*)(out + token * out_stride + head * d + dim) = r;
}

static void launch_attention_merge(bf16* out, int out_stride, const float* part_o, const float* part_ml, int tokens, int nq, int d,
                                   int splits, hipStream_t s) {
  const bool wide = tokens >= 64 && d % 4 == 0 && out_stride % 4 == 0 && (uintptr_t)out % 8 == 0 && (uintptr_t)part_o % 16 == 0 &&
                    (uintptr_t)part_ml % 8 == 0 && (splits == 2 || splits == 3 || splits == 4 || splits == 8);
  if (wide) {
    const int64_t quads = (int64_t)tokens * nq * (d / 4);
    const int blocks = (int)((quads + 255) / 256);
    if (splits == 2) attention_merge_wide_kernel<2><<<blocks, 256, 0, s>>>(out, out_stride, part_o, part_ml, quads, nq, d);
    else if (splits == 3) attention_merge_wide_kernel<3><<<blocks, 256, 0, s>>>(out, out_stride, part_o, part_ml, quads, nq, d);
    else if (splits == 4) attention_merge_wide_kernel<4><<<blocks, 256, 0, s>>>(out, out_stride, part_o, part_ml, quads, nq, d);
    else attention_merge_wide_kernel<8><<<blocks, 256, 0, s>>>(out, out_stride, part_o, part_ml, quads, nq, d);
  } else {
    attention_merge_kernel<<<dim3(tokens, nq), d < 64 ? 64 : d, 0, s>>>(out, out_stride, part_o, part_ml, nq, d, splits);
  }
}

// Decode step in bf16: one query token per request.  part_o [tokens, nq, splits, d] and part_ml
// [tokens, nq, splits, 2] float32 are needed when splits > 1.  Returns an error for shapes the
// matrix-core kernel does not take (the caller then uses lrs_attention).
// prepare != 0: q points at the raw rows [q heads | kv_columns k heads | kv_columns v heads] of the
// q/k/v product and the kernel does the work of lrs_qk_prep as well (rotation over the whole head
// or none; kv_columns is nkv, or 0 for a layer that reads another layer's pages).
LRS_API int lrs_attention_decode(void* out, int out_stride, float* part_o, float* part_ml, const void* q,
                                 int q_stride, void* k_pages, void* v_pages,
                                 const int* block_table, int table_stride, const int* token_request,
                                 const int* positions, int tokens, int max_context, int nq, int nkv, int d,
                                 int page_size, float scale, int window, int splits, int form, int prepare,
                                 const void* q_weight, const void* k_weight, int w_dtype, float eps,
                                 const float* cosv, const float* sinv, int kv_columns, void* stream) {
  LRS_REQUIRE(tokens > 0 && nq > 0 && nkv > 0 && nq % nkv == 0, "attention_decode: bad sizes tokens=%d nq=%d nkv=%d", tokens, nq, nkv);
  LRS_REQUIRE(nq / nkv <= 16, "attention_decode: %d query heads per kv head, at most 16 fit a tile", nq / nkv);
  LRS_REQUIRE(page_size % 16 == 0, "attention_decode: page size %d is not a multiple of 16", page_size);
  LRS_REQUIRE(splits >= 1 && (splits == 1 || (part_o && part_ml)), "attention_decode: splits=%d needs partial buffers", splits);
  LRS_REQUIRE(window >= 0, "attention_decode: window must be >= 0 (0 = none)");
  LRS_REQUIRE(form >= 0 && form <= 2, "attention_decode: form must be 0, 1 or 2, got %d", form);
  LRS_REQUIRE(q_stride % 8 == 0 && ((uintptr_t)q % 16) == 0, "attention_decode: q rows must be 16-byte aligned");
  dim3 grid(splits, nkv, tokens);
  hipStream_t s = (hipStream_t)stream;
  // LDS copy of the block table entries one workgroup walks
  LRS_REQUIRE(max_context >= 1, "attention_decode: max_context must be the longest context length of the step");
  const int span = window > 0 && window + 64 < max_context ? window + 64 : max_context;
  const size_t table_lds = sizeof(int) * (size_t)((span / 32 + splits) / splits * 32 / page_size + 4);
  LRS_REQUIRE(table_lds <= 24 * 1024, "attention_decode: a context of %d tokens in %d splits needs more block table entries than fit LDS", max_context, splits);
  if (prepare) {
    LRS_REQUIRE((q_weight == nullptr) == (k_weight == nullptr), "attention_decode: q and k norm weights must come together");
    LRS_REQUIRE(q_weight == nullptr || eps > 0.f, "attention_decode: eps must be positive");
    LRS_REQUIRE((cosv == nullptr) == (sinv == nullptr), "attention_decode: cos and sin tables must come together");
    LRS_REQUIRE(cosv == nullptr || d % 64 == 0, "attention_decode: the kernel rotates heads of 64, 128 or 192 dims only, got %d", d);
    LRS_REQUIRE(kv_columns == 0 || kv_columns == nkv, "attention_decode: kv_columns must be 0 or the number of kv heads (%d), got %d", nkv, kv_columns);
    LRS_REQUIRE(q_stride >= (nq + 2 * kv_columns) * d, "attention_decode: q row stride %d too small for q, k and v heads", q_stride);
    LRS_REQUIRE((uintptr_t)q_weight % 16 == 0 && (uintptr_t)k_weight % 16 == 0 && (uintptr_t)cosv % 16 == 0 && (uintptr_t)sinv % 16 == 0,
                "attention_decode: norm weights and rotation tables must be 16-byte aligned");
  }
  const DecodePrep prep{q_weight, k_weight, w_dtype == LRS_F32, eps, cosv, sinv, kv_columns};
  // `form`: 0 = four waves, a tile at a time; 1 = four waves, 2 = eight waves, each wave with its next
  // tile on the way while it works (heads of 192 dims have no registers for that and stay with 0)
#define ARGS                                                                                                 \
  (bf16*)out, out_stride, part_o, part_ml, (const bf16*)q, q_stride, (bf16*)k_pages, (bf16*)v_pages, block_table, \
      table_stride, token_request, positions, nq, nkv, page_size, scale, window, splits, prep
#define LAUNCH_PREP(D, PREP)                                                                                 \
  do {                                                                                                       \
    if (form == 2 && D <= 128) attention_decode_bf16_kernel<D, PREP, 8, (D <= 128)><<<grid, 512, table_lds, s>>>(ARGS); \
    else if (form == 1 && D <= 128) attention_decode_bf16_kernel<D, PREP, 4, (D <= 128)><<<grid, 256, table_lds, s>>>(ARGS); \
    else attention_decode_bf16_kernel<D, PREP, 4, false><<<grid, 256, table_lds, s>>>(ARGS);                  \
  } while (0)
#define LAUNCH(D)                        \
  do {                                   \
    if (prepare) LAUNCH_PREP(D, true);   \
    else LAUNCH_PREP(D, false);          \
  } while (0)
  switch (d) {
    case 32: LAUNCH(32); break;
    case 64: LAUNCH(64); break;
    case 96: LAUNCH(96); break;
    case 128: LAUNCH(128); break;
    case 192: LAUNCH(192); break;
    default: return lrs_fail("attention_decode: head_dim %d has no matrix-core kernel (32, 64, 96, 128, 192)", d);
  }
#undef LAUNCH
#undef LAUNCH_PREP
#undef ARGS
  if (lrs_check_launch("attention_decode")) return 1;
  if (splits > 1) {
    launch_attention_merge((bf16*)out, out_stride, part_o, part_ml, tokens, nq, d, splits, s);
    return lrs_check_launch("attention_merge");
  }
  return 0;
}

// ------------------------------------------------- bf16 kernel for any step
// Ragged batch of prompt portions and single tokens.  The step's tokens are cut on the host into
// groups of at most 16*QB consecutive tokens of one request; a workgroup owns one (group, kv head)
// and each of its (up to four) waves one query head of the kv group.  Keys are walked in tiles of
// 32: the workgroup brings a tile's keys and (transposed) values into LDS once, all waves take
// their matrix-core operands from there, and the next tile is on its way from memory while the
// current one is worked on (two LDS buffers, one barrier a tile).  A wave holds QB blocks of 16
// queries, so every fragment it reads serves QB products.  The arithmetic is that of the decode
// kernel with 16 queries in the tile columns instead of the heads: S[key, query] = K Q^T, online
// softmax per query column with the causal (and window) mask of that query's position,
// O^T[dim, query] += V^T P.  Every query is finished by one wave, so nothing is merged.
// Two workgroups share a compute unit (at most 256 registers a lane, which also keeps the
// accumulators out of the AGPRs, where rescaling them would cost moves at every tile), so one
// wave's exponentials run beside another's matrix products.  The grid is one-dimensional: groups
// come longest first, and in every second chunk of `chunk` workgroups (one per compute unit) the
// order is turned round, so that the two workgroups that meet on a compute unit are a long and a
// short one; the kv head changes fastest, which keeps one kv head's keys in one XCD's L2.
// splits > 1 (few queries over long contexts): the key tiles of every group are divided between
// `splits` workgroups, which leave unnormalised sums, maxima and weights in part_o / part_ml
// [tokens, heads, splits, ...] for attention_merge_kernel, as the decode kernel does.
template <int D, int QB>
__global__ __launch_bounds__(256, D <= 128 ? 2 : 1) void attention_prefill_bf16_kernel(
    bf16* __restrict__ out, int out_stride, const bf16* __restrict__ q, int q_stride,
    const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
    const int* __restrict__ block_table, int table_stride, const int* __restrict__ token_request,
    const int* __restrict__ positions, const int* __restrict__ qblock_token0,
    const int* __restrict__ qblock_count, int n_blocks, int chunk, int nq, int nkv, int page_size, float scale,
    int window, int splits, float* __restrict__ part_o, float* __restrict__ part_ml) {
  constexpr int DS = D / 32, DB = D / 16;
  // Padded LDS rows.  Every fragment is read 16 bytes a lane, 16 rows at a time (the lane's row is col, its
  // piece g), which the LDS serves at its full 256 bytes a cycle when rows lie 32 bytes more than a multiple
  // of 64 apart, and at half of that, or worse, otherwise (measured for every stride; 8-byte reads reach
  // half at best).  Key rows are D elements long; a row of the transposed value tile holds a dimension's 32
  // keys in the order the second product wants them, so that a lane's eight are one 16-byte piece: position
  // g * 8 + h * 4 + i for key h * 16 + g * 4 + i, which is where the first product leaves that key's weight.
  constexpr int KLD = D + 16, VLD = 32 + 16;
  __shared__ __attribute__((aligned(16))) bf16 ks[2][32 * KLD];
  __shared__ __attribute__((aligned(16))) bf16 vs[2][D * VLD];
  const int tid = threadIdx.x, threads = blockDim.x;
  const int lane = tid % WAVE, wave = tid / WAVE, waves = threads / WAVE;
  const int col = lane & 15, g = lane >> 4;
  const int group = nq / nkv;
  const int work = blockIdx.x % (n_blocks * nkv), split = blockIdx.x / (n_blocks * nkv);
  const int which_chunk = work / chunk, in_chunk = work % chunk;
  const int chunk_block0 = which_chunk * (chunk / nkv);
  const int chunk_blocks = n_blocks - chunk_block0 < chunk / nkv ? n_blocks - chunk_block0 : chunk / nkv;
  const int kvh = in_chunk % nkv;
  const int qblock = chunk_block0 + ((which_chunk & 1) ? chunk_blocks - 1 - in_chunk / nkv : in_chunk / nkv);
  const int token0 = qblock_token0[qblock], count = qblock_count[qblock];
  const int pos_first = positions[token0], pos_last = positions[token0 + count - 1];
  const int lo_first = (window > 0 && pos_first - window + 1 > 0) ? pos_first - window + 1 : 0;
  const int lo_last = (window > 0 && pos_last - window + 1 > 0) ? pos_last - window + 1 : 0;
  const int* table = block_table + (int64_t)token_request[token0] * table_stride;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const float scale2 = scale * 1.4426950408889634f;
  const float rescale_step = RESCALE_STEP / scale2;              // in units of the unscaled scores
  int first_tile = lo_first / 32, last_tile = pos_last / 32;
  if (splits > 1) {                                              // this workgroup's share of the tiles (may be none)
    const int per_split = (last_tile - first_tile + splits) / splits;
    first_tile += split * per_split;
    if (first_tile + per_split - 1 < last_tile) last_tile = first_tile + per_split - 1;
  }
  // the part of the request's block table that the tiles need, in LDS: the address of a key must
  // not wait for a trip to memory of its own
  extern __shared__ int page_ids[];
  const int last_key = last_tile * 32 + 31 < pos_last ? last_tile * 32 + 31 : pos_last;
  {
    const int first = first_tile * 32 / page_size;
    if (first_tile <= last_tile)
      for (int i = tid; i <= last_key / page_size - first; i += threads) page_ids[i] = table[first + i];
  }
  __syncthreads();

  // Pieces of a tile this thread brings in: keys [32, D] and transposed values [D, 32].  A run of 16 keys
  // lies in one page, and a wave serves one run (waves 0 and 1 the tile's first, 2 and 3 its second), so
  // everything about the run's place in memory is the same for the whole wave and is worked out in
  // scalar registers: one block table entry, one base address; a lane adds a distance that never changes.
  constexpr int KPIECES = D / 8, RUN_CHUNKS = 16 * KPIECES, TPR = 128, KPT = (RUN_CHUNKS + TPR - 1) / TPR;
  constexpr int VRUN_CHUNKS = 2 * D, VPT = (VRUN_CHUNKS + TPR - 1) / TPR;
  bf16x8 kreg_a[KPT], vreg_a[VPT];
  const int wrun = __builtin_amdgcn_readfirstlane(tid / TPR), t1 = tid % TPR;
  const int pages16 = page_size / 16;                            // runs of 16 keys in a page
  const unsigned magic = pages16 > 1 ? 0xFFFFFFFFu / (unsigned)pages16 + 1u : 0u;   // run / pages16 = umulhi(run, magic)
  const int first_block = pages16 > 1 ? (int)__umulhi((unsigned)(first_tile * 2), magic) : first_tile * 2;
  unsigned koff[KPT], voff[VPT];
#pragma unroll
  for (int i = 0; i < KPT; ++i) koff[i] = (unsigned)(((t1 + i * TPR) / KPIECES) * D + ((t1 + i * TPR) % KPIECES) * 8);
#pragma unroll
  for (int i = 0; i < VPT; ++i) voff[i] = (unsigned)(((t1 + i * TPR) / 2) * page_size + ((t1 + i * TPR) % 2) * 8);
  auto fetch = [&](int tile, bf16x8 (&kreg)[KPT], bf16x8 (&vreg)[VPT]) {
    const int run = tile * 2 + wrun, key0 = run * 16;
    const bool present = key0 <= pos_last && key0 + 15 >= lo_first;
    if (present) {
      const int block = pages16 > 1 ? (int)__umulhi((unsigned)run, magic) : run;
      const int64_t page = __builtin_amdgcn_readfirstlane(page_ids[block - first_block]);
      const int off = (run - block * pages16) * 16;
      const bf16* kbase = k_pages + ((page * nkv + kvh) * page_size + off) * D;
      const bf16* vbase = v_pages + (page * nkv + kvh) * (int64_t)D * page_size + off;
#pragma unroll
      for (int i = 0; i < KPT; ++i) kreg[i] = t1 + i * TPR < RUN_CHUNKS ? *(const bf16x8*)(kbase + koff[i]) : zero8;
#pragma unroll
      for (int i = 0; i < VPT; ++i) vreg[i] = t1 + i * TPR < VRUN_CHUNKS ? *(const bf16x8*)(vbase + voff[i]) : zero8;
    } else {
#pragma unroll
      for (int i = 0; i < KPT; ++i) kreg[i] = zero8;
#pragma unroll
      for (int i = 0; i < VPT; ++i) vreg[i] = zero8;
    }
  };
  auto stash = [&](int buffer, const bf16x8 (&kreg)[KPT], const bf16x8 (&vreg)[VPT]) {
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      const int c = t1 + i * TPR;
      if (c < RUN_CHUNKS) *(bf16x8*)(ks[buffer] + (wrun * 16 + c / KPIECES) * KLD + (c % KPIECES) * 8) = kreg[i];
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int c = t1 + i * TPR;
      if (c < VRUN_CHUNKS) {
        // keys wrun * 16 + (c % 2) * 8 + 0..7 of dimension c / 2: h = wrun, g = (c % 2) * 2 and the next
        bf16* dst = vs[buffer] + (c / 2) * VLD + (c % 2) * 16 + wrun * 4;
        *(bf16x4*)dst = bf16x4{vreg[i][0], vreg[i][1], vreg[i][2], vreg[i][3]};
        *(bf16x4*)(dst + 8) = bf16x4{vreg[i][4], vreg[i][5], vreg[i][6], vreg[i][7]};
      }
    }
  };

  // kv groups of more than four heads take several passes over the keys
  for (int head0 = kvh * group; head0 < (kvh + 1) * group; head0 += waves) {
    const int head = head0 + wave;
    const bool active = head < (kvh + 1) * group;
    bf16x8 qf[QB][DS];
    floatx4 o[QB][DB];
    float run_max[QB], run_sum[QB];
    int pos[QB], lo[QB];
    bool live[QB];
#pragma unroll
    for (int b = 0; b < QB; ++b) {
      live[b] = active && b * 16 + col < count;
      const int token = token0 + (live[b] ? b * 16 + col : 0);
      pos[b] = live[b] ? positions[token] : -1;                // a dead column sees no key
      lo[b] = (window > 0 && pos[b] - window + 1 > 0) ? pos[b] - window + 1 : 0;
      run_max[b] = -INFINITY;
      run_sum[b] = 0.f;
#pragma unroll
      for (int c = 0; c < DS; ++c)
        qf[b][c] = live[b] ? *(const bf16x8*)(q + (int64_t)token * q_stride + (int64_t)head * D + c * 32 + g * 8) : zero8;
#pragma unroll
      for (int e = 0; e < DB; ++e) o[b][e] = floatx4{0.f, 0.f, 0.f, 0.f};
    }

    // The three parts of a tile's work.
    // scores: S[key, query] = K Q^T, unscaled (the scale enters with the exponent).
    auto scores = [&](int buffer, floatx4 (&sc)[QB][2]) {
      const bf16* kt = ks[buffer];
#pragma unroll
      for (int b = 0; b < QB; ++b) sc[b][0] = sc[b][1] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int c = 0; c < DS; ++c) {
          const bf16x8 kfrag = *(const bf16x8*)(kt + (h * 16 + col) * KLD + c * 32 + g * 8);
#pragma unroll
          for (int b = 0; b < QB; ++b) sc[b][h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kfrag, qf[b][c], sc[b][h], 0, 0, 0);
        }
    };
    // weights: one step of the running softmax, p = 2^(s * scale2 - reference * scale2) as bfloat16 operands.
    // The reference point of a query's exponentials need not be its maximum: any value that keeps the
    // weights inside float32 and bfloat16 gives the same result up to rounding.  So a tile that needs no
    // mask first tries the reference it has, without looking for the tile's maximum at all (`weights`,
    // which changes nothing if it fails); only if a weight sum comes out above 2^60 (or the query has no
    // reference yet) is the tile done the long way (`weights_with_maximum`), which moves the reference to
    // the tile's maximum when that exceeds it by more than 2^8 and rescales the accumulators.  That
    // happens a few times per sequence.
    auto weights_with_maximum = [&](int tile, floatx4 (&sc)[QB][2], auto masked, bf16x8 (&pf)[QB]) {
      constexpr bool MASKED = decltype(masked)::value;
      float alpha[QB];
      bool rescale = false;
#pragma unroll
      for (int b = 0; b < QB; ++b) {
        float tile_max = -INFINITY;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            if (MASKED) {
              const int key = tile * 32 + h * 16 + g * 4 + i;
              sc[b][h][i] = (key <= pos[b] && key >= lo[b]) ? sc[b][h][i] : -INFINITY;
            }
            tile_max = fmaxf(tile_max, sc[b][h][i]);
          }
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, WAVE));
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, WAVE));
        const float new_max = tile_max > run_max[b] + rescale_step ? tile_max : run_max[b];
        // a query whose window or position leaves it no key so far keeps its state
        const bool empty = MASKED && new_max == -INFINITY;
        alpha[b] = empty ? 1.f : fast_exp2((run_max[b] - new_max) * scale2);
        const float shift = empty ? 0.f : -new_max * scale2;
        run_max[b] = new_max;
        float tile_sum = 0.f;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float p = fast_exp2(fmaf(sc[b][h][i], scale2, shift));
            tile_sum += p;
            pf[b][h * 4 + i] = (bf16)p;
          }
        run_sum[b] = run_sum[b] * alpha[b] + tile_sum;
        rescale |= alpha[b] != 1.f;
      }
      // once the reference points have settled no column needs rescaling: skip the multiplies
      if (__any(rescale)) {
#pragma unroll
        for (int b = 0; b < QB; ++b)
#pragma unroll
          for (int e = 0; e < DB; ++e) o[b][e] *= alpha[b];
      }
    };
    auto weights = [&](floatx4 (&sc)[QB][2], bf16x8 (&pf)[QB]) -> bool {
      float sums[QB];
      bool again = false;
#pragma unroll
      for (int b = 0; b < QB; ++b) {
        const float shift = -run_max[b] * scale2;                // +inf before the query's first tile: the sum then says "again"
        float tile_sum = 0.f;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float p = fast_exp2(fmaf(sc[b][h][i], scale2, shift));
            tile_sum += p;
            pf[b][h * 4 + i] = (bf16)p;
          }
        sums[b] = tile_sum;
        again |= !(tile_sum <= 0x1p60f);                         // too large, infinite or not a number
      }
      if (__any(again)) return false;
#pragma unroll
      for (int b = 0; b < QB; ++b) run_sum[b] += sums[b];
      return true;
    };
    // values: O^T[dim, query] += V^T P
    auto values = [&](int buffer, const bf16x8 (&pf)[QB]) {
      const bf16* vt = vs[buffer];
#pragma unroll
      for (int e = 0; e < DB; ++e) {
        const bf16x8 vv = *(const bf16x8*)(vt + (e * 16 + col) * VLD + g * 8);
#pragma unroll
        for (int b = 0; b < QB; ++b) o[b][e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vv, pf[b], o[b][e], 0, 0, 0);
      }
    };

    // Tiles [whole_begin, whole_end) need no mask: every query of the group sees every key of theirs.
    int whole_begin = (lo_last + 31) / 32, whole_end = (pos_first + 1) / 32;
    if (whole_begin < first_tile) whole_begin = first_tile;
    if (whole_begin > last_tile + 1) whole_begin = last_tile + 1;
    if (whole_end > last_tile + 1) whole_end = last_tile + 1;
    if (whole_end < whole_begin) whole_end = whole_begin;

    // The walk over the tiles.  At the top of a turn `tile` is in LDS buffer (tile - first_tile) % 2; the
    // next tile is asked for before the work on this one and put into the other buffer after it.  Most
    // turns take the short way through the weights; the inner loop holds only those, so that nothing in it
    // touches the accumulators but the matrix products.  A tile that needs the mask, or whose weights
    // came out too large for the reference point it was tried with, leaves the inner loop, is finished
    // the long way and the inner loop begins again behind it.
    __syncthreads();                                           // the buffers of an earlier pass are done with
    if (first_tile <= last_tile) {
      fetch(first_tile, kreg_a, vreg_a);
      stash(0, kreg_a, vreg_a);
    }
    __syncthreads();
    floatx4 sc[QB][2];
    bf16x8 pf[QB];
    int tile = first_tile;
    for (;;) {
      bool unfinished = false;
      for (; tile <= last_tile; ++tile) {
        const int buffer = (tile - first_tile) & 1;
        if (tile < last_tile) fetch(tile + 1, kreg_a, vreg_a);
        scores(buffer, sc);
        if (tile < whole_begin || tile >= whole_end || !weights(sc, pf)) {
          unfinished = true;
          break;
        }
        values(buffer, pf);
        if (tile < last_tile) stash(buffer ^ 1, kreg_a, vreg_a);
        __syncthreads();
      }
      if (!unfinished) break;
      const int buffer = (tile - first_tile) & 1;
      if (tile < whole_begin || tile >= whole_end) weights_with_maximum(tile, sc, std::true_type{}, pf);
      else weights_with_maximum(tile, sc, std::false_type{}, pf);
      values(buffer, pf);
      if (tile < last_tile) stash(buffer ^ 1, kreg_a, vreg_a);
      __syncthreads();
      ++tile;
    }
#pragma unroll
    for (int b = 0; b < QB; ++b) {
      float total = run_sum[b];
      total += __shfl_xor(total, 16, WAVE);
      total += __shfl_xor(total, 32, WAVE);
      if (live[b] && splits > 1) {
        const int64_t slot = ((int64_t)(token0 + b * 16 + col) * nq + head) * splits + split;
#pragma unroll
        for (int e = 0; e < DB; ++e) *(floatx4*)(part_o + slot * D + e * 16 + g * 4) = o[b][e];
        if (g == 0) {
          part_ml[slot * 2] = run_max[b] * scale2;               // -inf stays -inf: no key seen
          part_ml[slot * 2 + 1] = total;
        }
      } else if (live[b]) {
        const float inv = 1.0f / total;
        bf16* dst = out + (int64_t)(token0 + b * 16 + col) * out_stride + (int64_t)head * D + g * 4;
#pragma unroll
        for (int e = 0; e < DB; ++e) {
          const bf16x4 packed = {(bf16)(o[b][e][0] * inv), (bf16)(o[b][e][1] * inv), (bf16)(o[b][e][2] * inv), (bf16)(o[b][e][3] * inv)};
          *(bf16x4*)(dst + e * 16) = packed;
        }
      }
    }
  }
}

// ------------------------------------- bf16 kernel for any step, head size 128
// The same walk as attention_prefill_bf16_kernel with the tiles brought in differently: memory
// writes them straight into LDS (global_load_lds_dwordx4: a wave's 64 lanes fetch 16 bytes each,
// from addresses of their own choice, and the 1,024 bytes land in lane order at the address in m0),
// so a tile passes through no registers, three tiles are in flight instead of one, nothing is written
// to LDS by the waves, and where a piece lies in LDS is decided by which lane fetches it.
//
// LDS serves 16-byte reads at its full 256 bytes a cycle when the lanes it takes together (eight
// consecutive rows of the fragment, pieces g and g + 1) fall on 64 different banks; measured, and
// that is what the layout is made for:
//   keys    eight blocks of 1,024 bytes (four rows of 256), block j at j * 1,056; row (h, col) of
//           the first product's fragments lies in block col % 8 as its row 2 h + col / 8, so eight
//           consecutive columns meet eight blocks, each 8 banks further on than the one before.
//   values  transposed, a half for each run of 16 keys: [half][dim][16 keys], the second half 16
//           bytes out of step; lanes g = 0, 2 read the first half's two pieces, g = 1, 3 the second's.
// A block is one fetch of one wave and comes from one page.  Which key a fragment row holds is free
// as long as the second product meets the weights where the first left them: lanes of group g hold
// the scores of keys 8 m + 4 h + i (m = 0, 2, 1, 3 for g = 0..3; h the fragment, i the register), and
// read the values of keys 8 m .. 8 m + 7 as one piece.
// The wave that fetched a tile waits for its own fetches (vmcnt) before the barrier that opens the
// tile to the others; the fetches of the tile after it stay in flight.  The fetches are written in
// assembly because the compiler would wait for all of them before any LDS read it cannot tell apart.
template <int QB, bool MANY_WAVES, bool IDLE_WAVES>
__global__ __launch_bounds__(MANY_WAVES ? 512 : 256, MANY_WAVES ? 1 : 2) void attention_prefill_d128_bf16_kernel(
    bf16* __restrict__ out, int out_stride, const bf16* __restrict__ q, int q_stride,
    const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
    const int* __restrict__ block_table, int table_stride, const int* __restrict__ token_request,
    const int* __restrict__ positions, const int* __restrict__ qblock_token0,
    const int* __restrict__ qblock_count, int n_blocks, int chunk, int nq, int nkv, int page_size, float scale,
    int window, int splits, float* __restrict__ part_o, float* __restrict__ part_ml, int prepare_q, DecodePrep prep) {
  constexpr int D = 128, DS = D / 32, DB = D / 16, STAGES = 3;
  constexpr int KBLOCK = 1024 + 32, KBYTES = 8 * KBLOCK, VHALF = 16 * D * 2 + 16, VBYTES = 2 * VHALF;
  constexpr int VSTAGE = (VBYTES + 63) / 64 * 64;
  __shared__ __attribute__((aligned(64))) unsigned char key_tiles[STAGES * KBYTES];
  __shared__ __attribute__((aligned(64))) unsigned char value_tiles[STAGES * VSTAGE];
  const int tid = threadIdx.x;
  const int lane = tid % WAVE, wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
  const int col = lane & 15, g = lane >> 4;
  const int key_chunk = ((g & 1) << 1) | (g >> 1);                 // m: the eight keys this lane group holds weights of
  const int group = nq / nkv;
  const int work = blockIdx.x % (n_blocks * nkv), split = blockIdx.x / (n_blocks * nkv);
  const int which_chunk = work / chunk, in_chunk = work % chunk;
  const int chunk_block0 = which_chunk * (chunk / nkv);
  const int chunk_blocks = n_blocks - chunk_block0 < chunk / nkv ? n_blocks - chunk_block0 : chunk / nkv;
  const int kvh = in_chunk % nkv;
  const int qblock = chunk_block0 + ((which_chunk & 1) ? chunk_blocks - 1 - in_chunk / nkv : in_chunk / nkv);
  const int token0 = qblock_token0[qblock], count = qblock_count[qblock];
  const int pos_first = positions[token0], pos_last = positions[token0 + count - 1];
  const int lo_first = (window > 0 && pos_first - window + 1 > 0) ? pos_first - window + 1 : 0;
  const int lo_last = (window > 0 && pos_last - window + 1 > 0) ? pos_last - window + 1 : 0;
  const int* table = block_table + (int64_t)token_request[token0] * table_stride;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const float scale2 = scale * 1.4426950408889634f;
  const float rescale_step = RESCALE_STEP / scale2;              // in units of the unscaled scores
  int first_tile = lo_first / 32, last_tile = pos_last / 32;
  if (splits > 1) {                                              // this workgroup's share of the tiles (may be none)
    const int per_split = (last_tile - first_tile + splits) / splits;
    first_tile += split * per_split;
    if (first_tile + per_split - 1 < last_tile) last_tile = first_tile + per_split - 1;
  }
  const int first_run = lo_first / 16, last_run = pos_last / 16;   // runs of 16 keys that hold a key some query sees

  // What this wave fetches of a tile: key blocks `wave` (first run) and `wave + 4` (second run), and the
  // dimensions 32 wave .. 32 wave + 31 of both value halves.  A lane's distance from the run's first key
  // (or first slot) never changes; the run's page is looked up once a wave.
  const int pages16 = page_size / 16;                            // runs of 16 keys in a page
  const unsigned magic = pages16 > 1 ? 0xFFFFFFFFu / (unsigned)pages16 + 1u : 0u;   // run / pages16 = umulhi(run, magic)
  // lane l of a key block brings row l / 16 (h = row / 2, k = row % 2), piece l % 16: key 8 k + 4 h + wave of its run
  const unsigned key_offset = (unsigned)(((((lane >> 4) & 1) * 8 + (lane >> 5) * 4 + wave) * D + (lane & 15) * 8) * 2);
  // lane l of a value block brings dimension 32 wave + l / 2, keys 8 (l % 2) .. + 7 of the run
  const unsigned value_offset = (unsigned)((((wave * 32 + (lane >> 1)) * page_size) + (lane & 1) * 8) * 2);
  const unsigned keys_address = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)key_tiles;
  const unsigned values_address = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)value_tiles;
  // Where a run of 16 keys lies in memory.  Everything about it is the same for the whole workgroup, so the
  // page comes from the block table by a scalar load and the rest is a handful of scalar instructions; a
  // tile's two pages are asked for a turn before its addresses are wanted.  A run no query sees is masked:
  // any page with numbers in it will do, so runs are clamped to those the queries do see.
  const unsigned page_bytes = (unsigned)(nkv * page_size * D * 2);   // from page to page, keys and values alike
  const char* const k_head = (const char*)(k_pages + (int64_t)kvh * page_size * D);
  const char* const v_head = (const char*)(v_pages + (int64_t)kvh * page_size * D);
  // INSIDE: the tile lies behind the first of the walk, so that only the far end needs the clamp
  auto run_in_reach = [&](auto inside, int tile, int half) {
    const int run = tile * 2 + half;
    if (decltype(inside)::value) return run > last_run ? last_run : run;
    return run < first_run ? first_run : run > last_run ? last_run : run;
  };
  auto pages_of = [&](auto inside, int tile, int (&pages)[2]) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int run = run_in_reach(inside, tile, half);
      pages[half] = table[pages16 > 1 ? (int)__umulhi((unsigned)run, magic) : run];
    }
  };
  auto locate = [&](auto inside, int tile, const int (&pages)[2], const char* (&kbase)[2], const char* (&vbase)[2]) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const uint64_t at = (uint64_t)(unsigned)pages[half] * page_bytes;
      if (pages16 > 1) {
        const int run = run_in_reach(inside, tile, half);
        const unsigned off = (unsigned)(run - (int)__umulhi((unsigned)run, magic) * pages16) * 16u;
        kbase[half] = k_head + at + off * (unsigned)(D * 2);
        vbase[half] = v_head + at + off * 2u;
      } else {
        kbase[half] = k_head + at;
        vbase[half] = v_head + at;
      }
    }
  };
  // (a kv group of five to eight heads brings as many waves, so that one walk over the keys serves them all;
  // the first four waves bring the tiles in)
  auto fetch_keys = [&](const char* const (&kbase)[2], int stage) {      // two fetches a wave
    if (wave >= 4) return;
#pragma unroll
    for (int half = 0; half < 2; ++half)
      fetch_to_lds(kbase[half], key_offset, keys_address + (unsigned)(stage * KBYTES + (wave + 4 * half) * KBLOCK));
  };
  auto fetch_values = [&](const char* const (&vbase)[2], int stage) {    // two fetches a wave
    if (wave >= 4) return;
#pragma unroll
    for (int half = 0; half < 2; ++half)
      fetch_to_lds(vbase[half], value_offset, values_address + (unsigned)(stage * VSTAGE + half * VHALF + wave * 1024));
  };
  // where this lane's fragments lie in a stage
  const int key_fragment = (col & 7) * KBLOCK + (col >> 3) * 256 + g * 16;              // + h * 512 + c * 64
  const int value_fragment = (g & 1) * VHALF + col * 32 + (g >> 1) * 16;                // + e * 512

  // kv groups of more than four heads take several passes over the keys
  const int waves = blockDim.x / WAVE;
  for (int head0 = kvh * group; head0 < (kvh + 1) * group; head0 += waves) {
    const int head = head0 + wave;
    const bool active = head < (kvh + 1) * group;
    bf16x8 qf[QB][DS];
    floatx4 o[QB][DB];
    float run_max[QB], run_sum[QB];
    int pos[QB], lo[QB];
    bool live[QB];
#pragma unroll
    for (int b = 0; b < QB; ++b) {
      live[b] = active && b * 16 + col < count;
      const int token = token0 + (live[b] ? b * 16 + col : 0);
      pos[b] = live[b] ? positions[token] : -1;                // a dead column sees no key
      lo[b] = (window > 0 && pos[b] - window + 1 > 0) ? pos[b] - window + 1 : 0;
      run_max[b] = -INFINITY;
      run_sum[b] = 0.f;
      if (prepare_q) {
        // q holds the raw rows of the q/k/v product: the head is normalised and rotated here, on its way into
        // the registers it stays in (a dead column prepares its group's first token and drops the result)
        prepare_head<D>(qf[b], q + (int64_t)token * q_stride + (int64_t)(active ? head : head0) * D, g, prep.q_weight, prep.weight_is_f32,
                        prep.eps, prep.cosv ? prep.cosv + (int64_t)token * (D / 2) : nullptr,
                        prep.sinv ? prep.sinv + (int64_t)token * (D / 2) : nullptr);
#pragma unroll
        for (int c = 0; c < DS; ++c) qf[b][c] = live[b] ? qf[b][c] : zero8;
      } else {
#pragma unroll
        for (int c = 0; c < DS; ++c)
          qf[b][c] = live[b] ? *(const bf16x8*)(q + (int64_t)token * q_stride + (int64_t)head * D + c * 32 + g * 8) : zero8;
      }
#pragma unroll
      for (int e = 0; e < DB; ++e) o[b][e] = floatx4{0.f, 0.f, 0.f, 0.f};
    }

    // scores: S[key, query] = K Q^T, unscaled (the scale enters with the exponent)
    auto scores = [&](int stage, floatx4 (&sc)[QB][2]) {
      const unsigned char* kt = key_tiles + stage * KBYTES + key_fragment;
#pragma unroll
      for (int b = 0; b < QB; ++b) sc[b][0] = sc[b][1] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int c = 0; c < DS; ++c) {
          const bf16x8 kfrag = *(const bf16x8*)(kt + h * 512 + c * 64);
#pragma unroll
          for (int b = 0; b < QB; ++b) sc[b][h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kfrag, qf[b][c], sc[b][h], 0, 0, 0);
        }
    };
    // weights: as in attention_prefill_bf16_kernel; sc[b][h][i] belongs to key tile * 32 + 8 m + 4 h + i
    auto weights_with_maximum = [&](int tile, floatx4 (&sc)[QB][2], auto masked, bf16x8 (&pf)[QB]) {
      constexpr bool MASKED = decltype(masked)::value;
      float alpha[QB];
      bool rescale = false;
#pragma unroll
      for (int b = 0; b < QB; ++b) {
        float tile_max = -INFINITY;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            if (MASKED) {
              const int key = tile * 32 + key_chunk * 8 + h * 4 + i;
              sc[b][h][i] = (key <= pos[b] && key >= lo[b]) ? sc[b][h][i] : -INFINITY;
            }
            tile_max = fmaxf(tile_max, sc[b][h][i]);
          }
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, WAVE));
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, WAVE));
        const float new_max = tile_max > run_max[b] + rescale_step ? tile_max : run_max[b];
        // a query whose window or position leaves it no key so far keeps its state
        const bool empty = MASKED && new_max == -INFINITY;
        alpha[b] = empty ? 1.f : fast_exp2((run_max[b] - new_max) * scale2);
        const float shift = empty ? 0.f : -new_max * scale2;
        run_max[b] = new_max;
        float tile_sum = 0.f;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float p = fast_exp2(fmaf(sc[b][h][i], scale2, shift));
            tile_sum += p;
            pf[b][h * 4 + i] = (bf16)p;
          }
        run_sum[b] = run_sum[b] * alpha[b] + tile_sum;
        rescale |= alpha[b] != 1.f;
      }
      if (__any(rescale)) {
#pragma unroll
        for (int b = 0; b < QB; ++b)
#pragma unroll
          for (int e = 0; e < DB; ++e) o[b][e] *= alpha[b];
      }
    };
    // The short way through the weights of the tile whose scores are in `sc`, and beside it the scores of the
    // tile after it (keys in `stage`) into `next`: the matrix cores work on the next tile's products while the
    // vector units turn this tile's scores into weights.  The two are independent and are written here one
    // product, one weight at a time, with a fence for the instruction scheduler after each pair, so that this
    // is the order the wave issues them in: a product keeps the matrix core busy for 16 cycles, in which the
    // three or four vector instructions of a weight cost nothing.  A head of 128 has as many products a tile
    // (8 for every 16 queries) as a lane has weights.  Returns false, and has changed nothing but pf and
    // next, if a weight sum says the reference point will not do.
    auto weights_beside_scores = [&](int stage, floatx4 (&sc)[QB][2], floatx4 (&next)[QB][2], bf16x8 (&pf)[QB]) -> bool {
      const unsigned char* kt = key_tiles + stage * KBYTES + key_fragment;
      constexpr int FRAGMENTS = 2 * DS, READ_AHEAD = 3;
      static_assert(FRAGMENTS * QB == QB * 8, "one weight for every product");
      bf16x8 kf[FRAGMENTS];
#pragma unroll
      for (int f = 0; f < READ_AHEAD; ++f) kf[f] = *(const bf16x8*)(kt + (f / DS) * 512 + (f % DS) * 64);
      float shift[QB], tile_sum[QB], weight[QB * 8];
#pragma unroll
      for (int b = 0; b < QB; ++b) {
        next[b][0] = next[b][1] = floatx4{0.f, 0.f, 0.f, 0.f};
        shift[b] = -run_max[b] * scale2;                         // +inf before the query's first tile: the sum then says "again"
        tile_sum[b] = 0.f;
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int n = 0; n < FRAGMENTS * QB; ++n) {
        const int f = n / QB, b = n % QB;
        if (b == 0 && f + READ_AHEAD < FRAGMENTS)
          kf[f + READ_AHEAD] = *(const bf16x8*)(kt + ((f + READ_AHEAD) / DS) * 512 + ((f + READ_AHEAD) % DS) * 64);
        next[b][f / DS] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[f], qf[b][f % DS], next[b][f / DS], 0, 0, 0);
        const int wb = n / 8, wh = (n / 4) % 2, wi = n % 4;      // the n-th weight of the lane
        weight[n] = fast_exp2(fmaf(sc[wb][wh][wi], scale2, shift[wb]));
        tile_sum[wb] += weight[n];
        if (n % 2 == 1) {
          pf[wb][wh * 4 + wi - 1] = (bf16)weight[n - 1];
          pf[wb][wh * 4 + wi] = (bf16)weight[n];
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      bool again = false;
#pragma unroll
      for (int b = 0; b < QB; ++b) again |= !(tile_sum[b] <= 0x1p60f);   // too large, infinite or not a number
      if (__any(again)) return false;
#pragma unroll
      for (int b = 0; b < QB; ++b) run_sum[b] += tile_sum[b];
      return true;
    };
    // values: O^T[dim, query] += V^T P
    auto values = [&](int stage, const bf16x8 (&pf)[QB]) {
      const unsigned char* vt = value_tiles + stage * VSTAGE + value_fragment;
#pragma unroll
      for (int e = 0; e < DB; ++e) {
        const bf16x8 vv = *(const bf16x8*)(vt + e * 512);
#pragma unroll
        for (int b = 0; b < QB; ++b) o[b][e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vv, pf[b], o[b][e], 0, 0, 0);
      }
    };

    // Tiles [whole_begin, whole_end) need no mask: every query of the group sees every key of theirs.
    int whole_begin = (lo_last + 31) / 32, whole_end = (pos_first + 1) / 32;
    if (whole_begin < first_tile) whole_begin = first_tile;
    if (whole_begin > last_tile + 1) whole_begin = last_tile + 1;
    if (whole_end > last_tile + 1) whole_end = last_tile + 1;
    if (whole_end < whole_begin) whole_end = whole_begin;

    // The walk.  Keys and values of tile t lie in stage (t - first_tile) % 3 of their rings.  A turn works on
    // tile t, whose scores the turn before has left in registers: it asks memory for the keys of t + 3 (their
    // stage was last read a turn ago, for the scores of t) and the values of t + 2 (likewise), computes the
    // scores of t + 1 beside the weights of t, adds the values of t, and before the barrier waits until only
    // what it asked for itself is still on its way: the keys of t + 2 and the values of t + 1 are then in LDS.
    __syncthreads();                                           // the stages of an earlier pass are done with
    floatx4 sa[QB][2], sb[QB][2];
    bf16x8 pf[QB];
    int pages_ahead[2];                                        // the pages of tile + 3 at the top of a turn
    const char* values_ahead[2];                               // where the values of tile + 2 lie
    if (first_tile <= last_tile) {
      int pages[2];
      const char *kbase[2], *vbase[2];
      pages_of(std::false_type{}, first_tile, pages);
      locate(std::false_type{}, first_tile, pages, kbase, vbase);
      fetch_keys(kbase, 0);
      fetch_values(vbase, 0);
      pages_of(std::false_type{}, first_tile + 1, pages);
      locate(std::false_type{}, first_tile + 1, pages, kbase, values_ahead);
      if (first_tile + 1 <= last_tile) fetch_keys(kbase, 1);
      int pending = 0;
      pages_of(std::false_type{}, first_tile + 2, pages);
      locate(std::false_type{}, first_tile + 2, pages, kbase, vbase);
      if (first_tile + 2 <= last_tile) fetch_keys(kbase, 2), pending += 2;
      if (first_tile + 1 <= last_tile) fetch_values(values_ahead, 1), pending += 2;
      values_ahead[0] = vbase[0], values_ahead[1] = vbase[1];
      pages_of(std::false_type{}, first_tile + 3, pages_ahead);
      if (pending == 4) fetched_then_barrier<4>();
      else if (pending == 2) fetched_then_barrier<2>();
      else fetched_then_barrier<0>();
      if (!IDLE_WAVES || active) scores(0, sa);
      asm volatile("s_barrier" ::: "memory");                  // everyone has read the first keys: their stage may be filled again
    }
    int tile = first_tile, stage = 0;                          // stage = (tile - first_tile) % 3
    // the turn's fetches, and how many they are; EVERY: tile + 3 is not past the last, so all of them happen
    auto ask_ahead = [&](auto every) -> int {
      constexpr bool EVERY = decltype(every)::value;
      int pending = 0;
      const char *kbase[2], *vbase[2];
      locate(std::true_type{}, tile + 3, pages_ahead, kbase, vbase);
      if (EVERY || tile + 3 <= last_tile) fetch_keys(kbase, stage), pending += 2;
      if (EVERY || tile + 2 <= last_tile) fetch_values(values_ahead, stage == 0 ? STAGES - 1 : stage - 1), pending += 2;
      values_ahead[0] = vbase[0], values_ahead[1] = vbase[1];
      pages_of(std::true_type{}, tile + 4, pages_ahead);        // wanted a turn from now
      return pending;
    };
    auto turn_over = [&](int pending) {
      if (pending == 4) fetched_then_barrier<4>();
      else if (pending == 2) fetched_then_barrier<2>();
      else fetched_then_barrier<0>();
      stage = stage == STAGES - 1 ? 0 : stage + 1;
      ++tile;
    };
    // Most turns take the short way and have three tiles behind them: the inner loop holds only those, with
    // every count fixed, so that nothing in it touches the accumulators but the matrix products.  A tile
    // that needs the mask, or whose weights came out too large, or one of the last three, leaves it and takes
    // the long way.  The scores of the tile at hand are in sa at the top of every turn.
    const int fast_begin = whole_begin, fast_end = whole_end < last_tile - 2 ? whole_end : last_tile - 2;
    // A wave without a head (a kv group whose heads are no multiple of the waves: IDLE_WAVES, a kernel of its own
    // so that the others keep their registers) only brings its share of the tiles in and keeps the workgroup's
    // barriers: one a tile, as the others.
    if (IDLE_WAVES && !active) {
      while (tile <= last_tile) turn_over(ask_ahead(std::false_type{}));
      continue;
    }
    for (;;) {
      bool asked = false;                                      // the turn's fetches have been asked for already
      // one way out of the inner loop only, at its top, before anything of the turn has happened to the accumulators
      for (;;) {
        if (asked || tile < fast_begin || tile >= fast_end) break;
        ask_ahead(std::true_type{});
        if (!weights_beside_scores(stage == STAGES - 1 ? 0 : stage + 1, sa, sb, pf)) {
          asked = true;
          continue;
        }
        values(stage, pf);
        turn_over(4);
#pragma unroll
        for (int b = 0; b < QB; ++b) sa[b][0] = sb[b][0], sa[b][1] = sb[b][1];
      }
      const bool unfinished = tile <= last_tile;
      if (!unfinished) break;
      const int pending = asked ? 4 : ask_ahead(std::false_type{});
      if (tile < last_tile) scores(stage == STAGES - 1 ? 0 : stage + 1, sb);
      if (tile >= whole_begin && tile < whole_end) weights_with_maximum(tile, sa, std::false_type{}, pf);
      else weights_with_maximum(tile, sa, std::true_type{}, pf);
      values(stage, pf);
      turn_over(pending);
#pragma unroll
      for (int b = 0; b < QB; ++b) sa[b][0] = sb[b][0], sa[b][1] = sb[b][1];
    }
#pragma unroll
    for (int b = 0; b < QB; ++b) {
      float total = run_sum[b];
      total += __shfl_xor(total, 16, WAVE);
      total += __shfl_xor(total, 32, WAVE);
      if (live[b] && splits > 1) {
        const int64_t slot = ((int64_t)(token0 + b * 16 + col) * nq + head) * splits + split;
#pragma unroll
        for (int e = 0; e < DB; ++e) *(floatx4*)(part_o + slot * D + e * 16 + g * 4) = o[b][e];
        if (g == 0) {
          part_ml[slot * 2] = run_max[b] * scale2;               // -inf stays -inf: no key seen
          part_ml[slot * 2 + 1] = total;
        }
      } else if (live[b]) {
        const float inv = 1.0f / total;
        bf16* dst = out + (int64_t)(token0 + b * 16 + col) * out_stride + (int64_t)head * D + g * 4;
#pragma unroll
        for (int e = 0; e < DB; ++e) {
          const bf16x4 packed = {(bf16)(o[b][e][0] * inv), (bf16)(o[b][e][1] * inv), (bf16)(o[b][e][2] * inv), (bf16)(o[b][e][3] * inv)};
          *(bf16x4*)(dst + e * 16) = packed;
        }
      }
    }
  }
}

// Compute units of the current device (asked once).
static int compute_units() {
  static int units = 0;
  if (!units) {
    int device = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&device) == hipSuccess && hipGetDeviceProperties(&prop, device) == hipSuccess) units = prop.multiProcessorCount;
    if (units <= 0) units = 256;
  }
  return units;
}

// Largest number of tokens in one query group of lrs_attention_prefill.
LRS_API int lrs_attention_prefill_group() { return 32; }

// The group size that serves a step of `tokens` tokens best, the longest context among them being `longest`
// (0: not known): groups of 16 while those of 32 would not give every compute unit its two workgroups several
// times over (measured on MI355X: a fresh prompt of up to 2,048 tokens is faster with 16, longer ones with 32);
// but groups of 32 already for 2,048 tokens behind as many or more, and for 1,024 behind three times as many: the
// walks are long then, and a wave with 32 queries does half as much beside its products for every key (2,048
// tokens after 2,048 / 6,144 / 30,720: 173 / 366 / 1,412 us with groups of 16, 142 / 272 / 1,071 with 32; 1,024
// after 7,168: 204 against 181 us; 512 after 7,680 stay with 16: 117 against 140 us).
LRS_API int lrs_attention_prefill_group_for(int tokens, int longest) {
  const int units = compute_units();
  if (tokens > 8 * units) return 32;
  if (tokens >= 8 * units && longest >= 2 * tokens) return 32;
  if (tokens >= 4 * units && longest >= 4 * tokens) return 32;
  return 16;
}

// Whether lrs_attention_prefill can be given the raw q rows of the q/k/v product (prepare != 0) for this head size.
LRS_API int lrs_attention_prefill_prepares(int d) { return d == 128; }

// Any step in bf16.  qblock_token0 / qblock_count [n_blocks]: first token and number of tokens
// (1..lrs_attention_prefill_group()) of each group of consecutive tokens of one request.
// splits > 1: every group's keys are divided between that many workgroups; needs part_o
// [tokens, nq, splits, d] and part_ml [tokens, nq, splits, 2] float32 and `tokens`, the step's size.
// prepare != 0 (heads of 128 only): q holds raw rows; every query head gets its RMSNorm (q_weight [d], or null for none)
// and the rotation of pairs (i, i + d/2) by the step's tables cosv / sinv [tokens, d/2] (null: none) on its way into the
// kernel's registers, as lrs_qk_prep would have left it in memory; the keys and values are in the pages already.
LRS_API int lrs_attention_prefill(void* out, int out_stride, const void* q, int q_stride, const void* k_pages,
                                  const void* v_pages, const int* block_table, int table_stride,
                                  const int* token_request, const int* positions, const int* qblock_token0,
                                  const int* qblock_count, int n_blocks, int max_count, int max_context, int nq,
                                  int nkv, int d, int page_size, float scale, int window, int tokens, int splits,
                                  float* part_o, float* part_ml, int prepare, const void* q_weight, int w_dtype, float eps,
                                  const float* cosv, const float* sinv, void* stream) {
  LRS_REQUIRE(n_blocks > 0 && nq > 0 && nkv > 0 && nq % nkv == 0, "attention_prefill: bad sizes blocks=%d nq=%d nkv=%d", n_blocks, nq, nkv);
  if (prepare) {
    LRS_REQUIRE(lrs_attention_prefill_prepares(d), "attention_prefill: only the kernel for heads of 128 prepares the queries itself, got head_dim %d", d);
    LRS_REQUIRE(q_weight == nullptr || eps > 0.f, "attention_prefill: eps must be positive");
    LRS_REQUIRE((cosv == nullptr) == (sinv == nullptr), "attention_prefill: cos and sin tables must come together");
    LRS_REQUIRE((uintptr_t)q_weight % 16 == 0 && (uintptr_t)cosv % 16 == 0 && (uintptr_t)sinv % 16 == 0,
                "attention_prefill: norm weight and rotation tables must be 16-byte aligned");
  }
  const DecodePrep prep{q_weight, nullptr, w_dtype == LRS_F32, eps, cosv, sinv, 0};
  LRS_REQUIRE(max_count >= 1 && max_count <= 32, "attention_prefill: query groups hold 1..32 tokens, got %d", max_count);
  LRS_REQUIRE(page_size % 16 == 0, "attention_prefill: page size %d is not a multiple of 16", page_size);
  LRS_REQUIRE(window >= 0, "attention_prefill: window must be >= 0 (0 = none)");
  LRS_REQUIRE(q_stride % 8 == 0 && ((uintptr_t)q % 16) == 0 && out_stride % 4 == 0 && ((uintptr_t)out % 8) == 0,
              "attention_prefill: q rows must be 16-byte and out rows 8-byte aligned");
  // four waves (with fewer heads in a kv group the spare waves still help to bring tiles in), more only below
  LRS_REQUIRE(splits >= 1 && splits <= 64 && (splits == 1 || (part_o && part_ml && tokens > 0)),
              "attention_prefill: splits=%d (1..64) need partial buffers and the number of tokens", splits);
  LRS_REQUIRE(splits == 1 || ((uintptr_t)part_o % 16) == 0, "attention_prefill: part_o must be 16-byte aligned");
  dim3 grid(n_blocks * nkv * splits), block(4 * WAVE);
  // workgroups that share a compute unit: see the kernel
  const int chunk = nkv >= compute_units() ? nkv : compute_units() / nkv * nkv;
  // LDS copy of the block table entries a workgroup walks: at most those of the longest context
  LRS_REQUIRE(max_context >= 1, "attention_prefill: max_context must be the longest context length of the step");
  const int span = window > 0 && window + 32 + 64 < max_context ? window + 32 + 64 : max_context;
  const size_t table_lds = sizeof(int) * (size_t)(span / page_size + 2);
  // (the kernel for heads of 128 reads the block table with scalar loads and keeps no copy)
  LRS_REQUIRE(d == 128 || table_lds <= 24 * 1024, "attention_prefill: a context of %d tokens needs more block table entries than fit LDS", max_context);
  hipStream_t s = (hipStream_t)stream;
#define LAUNCH2(D, QB)                                                                                               \
  attention_prefill_bf16_kernel<D, QB><<<grid, block, table_lds, s>>>((bf16*)out, out_stride, (const bf16*)q, q_stride, \
                                                              (const bf16*)k_pages, (const bf16*)v_pages, block_table, \
                                                              table_stride, token_request, positions, qblock_token0, \
                                                              qblock_count, n_blocks, chunk, nq, nkv, page_size, scale, window, \
                                                              splits, part_o, part_ml)
#define LAUNCH(D)                                \
  if (max_count <= 16) LAUNCH2(D, 1);            \
  else LAUNCH2(D, 2)
  switch (d) {
    case 32: LAUNCH(32); break;
    case 64: LAUNCH(64); break;
    case 96: LAUNCH(96); break;
    case 128:
      // head size 128 has a kernel of its own, whose tiles go from memory straight into LDS
      // A kv group of five to eight heads: a wave for every head and one walk over the keys instead of two, while
      // the launch is small (measured, 40 heads on 8: 512 tokens 28.9 -> 19.6 us, 512 tokens after 1,536 88 -> 54 us;
      // but 2,048 tokens 113 -> 129 us: a full chip does better with the smaller workgroups, three to a unit)
      {
        const bool many = nq / nkv > 4 && (int64_t)n_blocks * nkv * splits <= 2 * compute_units();
        if (many) block = dim3((nq / nkv < 8 ? nq / nkv : 8) * WAVE);
#define D128(QB, MANY, IDLE)                                                                                                      \
        attention_prefill_d128_bf16_kernel<QB, MANY, IDLE><<<grid, block, 0, s>>>(                                                    \
            (bf16*)out, out_stride, (const bf16*)q, q_stride, (const bf16*)k_pages, (const bf16*)v_pages, block_table, table_stride, \
            token_request, positions, qblock_token0, qblock_count, n_blocks, chunk, nq, nkv, page_size, scale, window, splits, part_o, part_ml, \
            prepare, prep)
#define D128_OF(QB)                                      \
        if (many && idle) D128(QB, true, true);          \
        else if (many) D128(QB, true, false);            \
        else if (idle) D128(QB, false, true);            \
        else D128(QB, false, false)
        const bool idle = (nq / nkv) % (int)(block.x / WAVE) != 0;   // some wave of some pass has no head
        if (max_count <= 16) { D128_OF(1); }
        else { D128_OF(2); }
#undef D128_OF
#undef D128
      }
      break;
    case 192: LAUNCH(192); break;
    default: return lrs_fail("attention_prefill: head_dim %d has no matrix-core kernel (32, 64, 96, 128, 192)", d);
  }
#undef LAUNCH
#undef LAUNCH2
  if (lrs_check_launch("attention_prefill")) return 1;
  if (splits > 1) {
    launch_attention_merge((bf16*)out, out_stride, part_o, part_ml, tokens, nq, d, splits, s);
    return lrs_check_launch("attention_merge");
  }
  return 0;
}

// Compute units of the device, for callers that size their launches by it.
LRS_API int lrs_compute_units() { return compute_units(); }

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
  const size_t lds = sizeof(float) * (d + d % 2 + THREADS) + (sizeof(int64_t) + sizeof(int)) * THREADS + 16;
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
