// Matrix products y = x W^T (+ bias) with W stored [out, in] as in the checkpoint.
//   x [M, K] row-major, W [N, K] row-major, both of dtype T (float or bf16).
// Output modes: store as T, store as float32, or add into a float32 matrix (the residual
// stream).  Accumulation is float32 in every kernel; the float32 kernels use plain FMAs and
// no matrix cores, so a float32 run is float32 throughout.  The order of the sum over K
// for one output element never depends on M, so a row's result does not depend on what
// else is in the batch.
#include "common.h"

#include <type_traits>

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

// ------------------------------------------------- float32 FMA kernel for at most 16 rows
// A decode step in float32: the tiled kernel above would fill one row of its 64 x 64 tiles in sixteen and walk K
// sixteen values at a time.  Here a workgroup of 256 threads owns 256 / MR weight rows and all (at most MR) rows
// of the input; a thread owns one output and adds its products up one after the other, k ascending from zero,
// which is exactly the sum the tiled kernel makes: the two give the same bits, so a row's result still does not
// depend on how many rows travel with it.  K is walked in slices of 64 through LDS (the weights as whole lines
// of 256 bytes, the next slice on its way into registers while this one is multiplied).  K % 64 == 0.
template <int MR>
__global__ __launch_bounds__(256) void gemm_f32_few_rows_kernel(void* __restrict__ out, int mode, const float* __restrict__ a,
                                                                 const float* __restrict__ w, const float* __restrict__ bias,
                                                                 int m, int n, int k, int lda, int ldc) {
  constexpr int CN = 256 / MR, BK = 64, PITCH = BK + 8;      // rows 288 bytes apart: 16-byte reads of consecutive rows at the full LDS rate
  constexpr int W_LOADS = CN * BK / 4 / 256, A_LOADS = (MR * BK / 4 + 255) / 256;
  static_assert(MR == 4 || MR == 8 || MR == 16, "4, 8 or 16 input rows a workgroup");
  __shared__ __attribute__((aligned(16))) float ws[2][CN * PITCH];
  __shared__ __attribute__((aligned(16))) float as[2][MR * PITCH];
  const int tid = threadIdx.x;
  const int n0 = blockIdx.x * CN;
  const int col = tid % CN, row = tid / CN;                   // this thread's output: weight row n0 + col, input row `row`
  // what this thread brings of a slice: 16 bytes of a weight row (and of an input row)
  const float* wsrc[W_LOADS];
  int wdst[W_LOADS];
#pragma unroll
  for (int i = 0; i < W_LOADS; ++i) {
    const int piece = tid + i * 256, r = piece / (BK / 4), c = piece % (BK / 4);
    const int gn = n0 + r < n ? n0 + r : n - 1;
    wsrc[i] = w + (int64_t)gn * k + c * 4;
    wdst[i] = r * PITCH + c * 4;
  }
  const float* asrc[A_LOADS];
  int adst[A_LOADS];
#pragma unroll
  for (int i = 0; i < A_LOADS; ++i) {
    const int piece = tid + i * 256, r = (piece / (BK / 4)) % MR, c = piece % (BK / 4);
    asrc[i] = a + (int64_t)(r < m ? r : m - 1) * lda + c * 4;
    adst[i] = r * PITCH + c * 4;
  }
  const bool brings_a = tid < MR * BK / 4 || A_LOADS > 1;
  floatx4 wreg[W_LOADS], areg[A_LOADS];
  auto load = [&](int k0) {
#pragma unroll
    for (int i = 0; i < W_LOADS; ++i) wreg[i] = *(const floatx4*)(wsrc[i] + k0);
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) areg[i] = *(const floatx4*)(asrc[i] + k0);
  };
  auto store = [&](int buf) {
#pragma unroll
    for (int i = 0; i < W_LOADS; ++i) *(floatx4*)(ws[buf] + wdst[i]) = wreg[i];
    if (brings_a) {
#pragma unroll
      for (int i = 0; i < A_LOADS; ++i) *(floatx4*)(as[buf] + adst[i]) = areg[i];
    }
  };
  float acc = 0.f;
  load(0);
  store(0);
  const int slices = k / BK;
  for (int slice = 0; slice < slices; ++slice) {
    __syncthreads();                                           // slice `slice` is in its buffer; the other buffer is read by nobody
    if (slice + 1 < slices) load((slice + 1) * BK);
    const float* wr = ws[slice & 1] + col * PITCH;
    const float* ar = as[slice & 1] + row * PITCH;
#pragma unroll
    for (int kk = 0; kk < BK; kk += 4) {
      const floatx4 wv = *(const floatx4*)(wr + kk), av = *(const floatx4*)(ar + kk);
      acc = fmaf(av[0], wv[0], acc);
      acc = fmaf(av[1], wv[1], acc);
      acc = fmaf(av[2], wv[2], acc);
      acc = fmaf(av[3], wv[3], acc);
    }
    if (slice + 1 < slices) store((slice + 1) & 1);
  }
  const int gn = n0 + col;
  if (row < m && gn < n) {
    float v = acc;
    if (bias) v += bias[gn];
    emit<float>(out, mode, (int64_t)row * ldc + gn, v);
  }
}

__device__ __forceinline__ float silu(float g) { return g / (1.0f + __expf(-g)); }

// ------------------------------------------------------- bf16 MFMA kernel
// 128x128 output tile per workgroup of 4 waves (2x2), each wave 64x64 as 2x2 MFMA
// 32x32x16 tiles.  K is walked in slices of 32 through LDS.  Needs K % 8 == 0 so that
// every 8-element chunk is a 16-byte aligned load; rows past M or N and chunks past K
// are zero-filled.
template <bool SWIGLU>
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
      if (SWIGLU) {
        // columns come in groups of 8 gate rows followed by the 8 up rows of the same features:
        // the up value of a gate column sits 8 lanes further on
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float up = __shfl(acc[i][j][r], (lane + 8) % WAVE, WAVE);
          const int gm = m0 + wm + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + r % 4;
          if (gn % 16 < 8 && gn + 8 < n && gm < m) {
            const float gate = acc[i][j][r];
            emit<bf16>(out, mode, (int64_t)gm * ldc + (gn / 16) * 8 + gn % 8, gate / (1.0f + __expf(-gate)) * up);
          }
        }
        continue;
      }
      if (gn >= n) continue;
      const float b = bias ? (float)bias[gn] : 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int gm = m0 + wm + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + r % 4;
        if (gm < m) emit<bf16>(out, mode, (int64_t)gm * ldc + gn, acc[i][j][r] + b);
      }
    }
}

// ------------------------------------------------- bf16 MFMA kernel for many rows
// 128 tokens x 256 weight rows per workgroup of four waves (2 x 2: a wave owns 64 tokens x 128 weight
// rows as 4 x 8 tiles of the 16x16x32 product), K walked in slices of 32.  Both operands pass through
// LDS, and memory writes them there itself (fetch_to_lds: no staging registers, no LDS write
// instructions): three stages of 24 KB, the slice two ahead asked for before a slice is multiplied, one
// barrier a slice, before which a wave waits for its own six fetches of the next slice.  Two workgroups
// share a compute unit.  Every fragment a wave reads from LDS feeds four or eight matrix instructions.
// Workgroups are numbered so that the 32 that share an XCD (and its L2) cover 4 x 8 tiles.  Needs
// K % 32 == 0, 16-byte aligned rows, no bias and matrices of fewer than 2^31 elements (the 128 x 128
// kernel above takes what this one does not).
// Before, a slice went through registers (asked for three slices ahead) and was written to LDS by the
// waves; measured then at 2,048 x 24,576 x 4,096: 469 us, without the loads from memory inside the loop
// 348 us, without the writes into LDS as well 252 us.  Weights straight from memory into registers (only
// activations through LDS) were slower: 513 us.
// Accumulator layout: weight row 4 * (lane / 16) + i, token lane % 16, i.e. four consecutive output
// columns of one token per lane.
constexpr int WIDE_BK = 32;   // measured on MI355X at 2,048 rows: slices of 32 (two workgroups a compute unit) beat slices of 64 (one) by a fifth
template <bool SWIGLU, int MODE>
__global__ __launch_bounds__(256, 2) void gemm_bf16_wide_kernel(void* __restrict__ out, const bf16* __restrict__ x,
                                                                const bf16* __restrict__ w, int m, int n, int k, int lda,
                                                                int ldc, int tiles_m, int tiles_n) {
  constexpr int BM = 128, BN = 256, BK = WIDE_BK, STAGES = 3;
  constexpr int XL = BM / 16 / 4, WL = BN / 16 / 4;           // blocks of 16 rows (1,024 bytes of a slice) per wave: 2 of x, 4 of w
  constexpr int STAGE_ELEMENTS = (BM + BN) * BK;
  __shared__ __attribute__((aligned(64))) bf16 slices[STAGES * STAGE_ELEMENTS];   // a stage: the tokens' slice, then the weights'
  const int tid = threadIdx.x, lane = tid % WAVE, wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
  const int r = lane & 15, g = lane >> 4;
  int id = blockIdx.x;
  const int tiles = tiles_m * tiles_n;
  if (tiles % 8 == 0) id = (id % 8) * (tiles / 8) + id / 8;        // consecutive workgroups go to different XCDs
  const int band = id / (4 * tiles_n), within = id % (4 * tiles_n);
  const int band_rows = tiles_m - band * 4 < 4 ? tiles_m - band * 4 : 4;
  const int m0 = (band * 4 + within % band_rows) * BM, n0 = (within / band_rows) * BN;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 128;           // this wave's corner inside the tile
  // Where chunk c (8 k) of tile row q lies in a stage: rows are 64 bytes, half a line of banks, packed
  // without padding; rows swap places in pairs in the upper half of every 16 and chunks are turned
  // round by the row number, so that the lanes LDS serves together (eight consecutive rows of a fragment,
  // chunks g and g + 1) each touch every bank once.  Element ((q ^ (q >> 3 & 1)) * 4 + (c ^ (q >> 1 & 3))) * 8;
  // only the low four bits of q enter the swaps, so a tile row 16 * j + q lies 16 * j * 32 elements further on.
  // A block of 16 rows is one fetch of one wave, whose lane l fills place l: it asks for the row and chunk
  // that belong there.  Rows past the matrix are read from its last row (and never written), slices past K
  // from the last slice (and not multiplied): no fetch in the loop is conditional.
  const int place_row = (lane >> 2) ^ ((lane >> 5) & 1);            // the row whose piece lies at place l = row' * 4 + chunk'
  const int place_chunk = (lane & 3) ^ ((place_row >> 1) & 3);
  unsigned xoff[XL], woff[WL];                                      // bytes from the matrix's first element
#pragma unroll
  for (int i = 0; i < XL; ++i) {
    const int row = m0 + 16 * (wave + 4 * i) + place_row;
    xoff[i] = (unsigned)(((row < m ? row : m - 1) * lda + place_chunk * 8) * 2);
  }
#pragma unroll
  for (int i = 0; i < WL; ++i) {
    const int row = n0 + 16 * (wave + 4 * i) + place_row;
    woff[i] = (unsigned)(((row < n ? row : n - 1) * k + place_chunk * 8) * 2);
  }
  const int frag = ((r ^ ((r >> 3) & 1)) * 4 + (g ^ ((r >> 1) & 3))) * 8;                    // where this lane's fragments come from
  floatx4 acc[8][4];
#pragma unroll
  for (int it = 0; it < 8; ++it)
#pragma unroll
    for (int jt = 0; jt < 4; ++jt) acc[it][jt] = floatx4{0.f, 0.f, 0.f, 0.f};
  const int steps = k / BK;
  const unsigned slices_address = (unsigned)(uintptr_t)(__attribute__((address_space(3))) bf16*)slices;
  auto fetch = [&](int kt, int stage) {                             // six fetches a wave
    const int at = (kt < steps ? kt : steps - 1) * BK * 2;
    const unsigned to = slices_address + (unsigned)(stage * STAGE_ELEMENTS * 2 + wave * 1024);
#pragma unroll
    for (int i = 0; i < XL; ++i) fetch_to_lds((const char*)x + at, xoff[i], to + (unsigned)(i * 4096));
#pragma unroll
    for (int i = 0; i < WL; ++i) fetch_to_lds((const char*)w + at, woff[i], to + (unsigned)(BM * BK * 2 + i * 4096));
  };
  auto multiply = [&](int stage) {
    const bf16* xs = slices + stage * STAGE_ELEMENTS;
    const bf16* ws = xs + BM * BK;
    bf16x8 xf[4];
#pragma unroll
    for (int jt = 0; jt < 4; ++jt) xf[jt] = *(const bf16x8*)(xs + frag + (wm + jt * 16) * BK);
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const bf16x8 wf = *(const bf16x8*)(ws + frag + (wn + it * 16) * BK);
#pragma unroll
      for (int jt = 0; jt < 4; ++jt) acc[it][jt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, xf[jt], acc[it][jt], 0, 0, 0);
    }
  };
  // Slice kt is multiplied from stage kt % 3 while slice kt + 1 arrives and slice kt + 2 is asked for (into
  // the stage that slice kt - 1 was multiplied from a barrier ago).  Before the barrier a wave waits until only
  // the six fetches it has just asked for are still on their way: slice kt + 1 is then in LDS.
  int m0_opaque = m0;
  fetch(0, 0);
  fetch(1, 1);
  fetched_then_barrier<6>();
  int stage = 0;
  for (int kt = 0; kt < steps; ++kt) {
    fetch(kt + 2, stage == 0 ? 2 : stage - 1);
    multiply(stage);
    fetched_then_barrier<6>();
    stage = stage == STAGES - 1 ? 0 : stage + 1;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");               // the fetches past K that nobody reads
  // nothing of the epilogue's addresses may be worked out (and kept in registers) before the loop above ends
  asm volatile("" : "+s"(ldc), "+s"(m0_opaque));
  // jt outside: one token row's address is worked out once and its 8 pieces of 4 columns follow 16 apart;
  // the fence after each piece keeps the compiler from working out all 32 addresses (64 registers) first
#pragma unroll
  for (int jt = 0; jt < 4; ++jt) {
    const int token = m0_opaque + wm + jt * 16 + r;
    const int64_t row_at = (int64_t)token * ldc;
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int tile0 = n0 + wn + it * 16, row0 = tile0 + 4 * g;     // this lane's four weight rows = output columns
      if (SWIGLU) {
        // a tile's 16 weight rows are 8 gate rows and the 8 up rows of the same features: the up
        // values of a lane's gate rows are held by the lane 32 further on
        floatx4 up;
#pragma unroll
        for (int i = 0; i < 4; ++i) up[i] = __shfl(acc[it][jt][i], (lane + 32) % WAVE, WAVE);
        if (g < 2 && token < m && tile0 + 15 < n) {
          const floatx4 gate = acc[it][jt];
          const bf16x4 y = {(bf16)(silu(gate[0]) * up[0]), (bf16)(silu(gate[1]) * up[1]), (bf16)(silu(gate[2]) * up[2]), (bf16)(silu(gate[3]) * up[3])};
          *(bf16x4*)((bf16*)out + row_at + tile0 / 2 + 4 * g) = y;
        }
      } else if (token < m && row0 < n) {
        floatx4 v = acc[it][jt];
        // An identity move across lanes: with a convergent operation on the accumulators here the
        // compiler keeps the loop above free of spills (222 registers); without one it spills about 300.
#pragma unroll
        for (int i = 0; i < 4; ++i)
          v[i] = __shfl(v[i], lane, WAVE);
        if constexpr (MODE == OUT_STORE) *(bf16x4*)((bf16*)out + row_at + row0) = bf16x4{(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
        else if constexpr (MODE == OUT_STORE_F32) *(floatx4*)((float*)out + row_at + row0) = v;
        else *(floatx4*)((float*)out + row_at + row0) = *(const floatx4*)((const float*)out + row_at + row0) + v;
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

// ------------------------------------------ bf16 MFMA kernel for many rows, slices of whole lines
// 256 tokens x BN weight rows per workgroup of eight waves, K walked in slices of 64, one workgroup a
// compute unit.  BN = 256 (2 x 4 waves: a wave owns 128 tokens x 64 weight rows as 8 x 4 tiles of the
// 16x16x32 product; two stages of 64 KB), BN = 192 (2 x 4 waves of 128 x 48; two stages of 56 KB) or
// BN = 128 (4 x 2 waves of 64 x 64; three stages of 48 KB): whichever leaves the compute units the least
// idle in the launch's last round (6,144 columns are 256 tiles of 192, one a unit).  Against the kernel above: a
// slice holds whole 128-byte lines of every row, so a fetch touches 8 lines instead of 16 halves (the address
// units in front of the L1 were busy 62 % of that kernel's time), and at BN = 256 a third less traffic from
// memory per product.  The slice after next (BN = 128) or the next (BN = 256) is asked for before a slice
// is multiplied.  K % 64 == 0; the kernel above takes the rest.
// Where chunk c (8 k, 16 bytes) of tile row q lies in a stage: rows are 128 bytes, eight to a block of
// 1,024 bytes (one fetch of one wave, whose lane l fills place l), and the chunks of a row are turned round
// by twice (q / 2) % 4, so that the lanes LDS serves together (eight consecutive rows, chunks g and g + 1)
// meet every bank once: place (q % 8) * 8 + (c ^ ((q >> 1 & 3) << 1)) of block q / 8.
template <int BN, bool SWIGLU, int MODE>
__global__ __launch_bounds__(512, 1) void gemm_bf16_lines_kernel(void* __restrict__ out, const bf16* __restrict__ x,
                                                                 const bf16* __restrict__ w, int m, int n, int k, int lda,
                                                                 int ldc, int tiles_m, int tiles_n, int splits) {
  static_assert(BN == 256 || BN == 192 || BN == 128, "256, 192 or 128 weight rows a workgroup");
  constexpr int BM = 256, BK = 64, STAGES = BN == 128 ? 3 : 2;
  constexpr int WAVES_N = BN == 128 ? 2 : 4;                   // waves side by side along the weight rows
  constexpr int IT = BN / WAVES_N / 16, JT = BM / (8 / WAVES_N) / 16;   // a wave's tiles: 4 x 8, 3 x 8 or 4 x 4
  constexpr int XL = BM / 8 / 8, WL = BN / 8 / 8;             // blocks of 8 rows per wave: 4 of x, 4, 3 or 2 of w
  constexpr int PENDING = STAGES == 2 ? 0 : XL + WL;          // fetches that may still be on their way at a barrier
  constexpr int STAGE_ELEMENTS = (BM + BN) * BK;
  __shared__ __attribute__((aligned(64))) bf16 slices[STAGES * STAGE_ELEMENTS];
  const int tid = threadIdx.x, lane = tid % WAVE, wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
  const int r = lane & 15, g = lane >> 4;
  const int tiles = tiles_m * tiles_n;
  const int split = blockIdx.x / tiles;                            // which part of K (the launch is tiles x splits)
  int id = blockIdx.x - split * tiles;
  if (tiles % 8 == 0) id = (id % 8) * (tiles / 8) + id / 8;        // consecutive workgroups go to different XCDs
  const int band = id / (4 * tiles_n), within = id % (4 * tiles_n);
  const int band_rows = tiles_m - band * 4 < 4 ? tiles_m - band * 4 : 4;
  const int m0 = (band * 4 + within % band_rows) * BM, n0 = (within / band_rows) * BN;
  const int wm = (wave / WAVES_N) * (JT * 16), wn = (wave % WAVES_N) * (IT * 16);   // this wave's corner inside the tile
  const int place_row = lane >> 3;                                  // the row whose piece lies at place l of a block
  const int place_chunk = (lane & 7) ^ (((place_row >> 1) & 3) << 1);
  unsigned xoff[XL], woff[WL];                                      // bytes from the matrix's first element
#pragma unroll
  for (int i = 0; i < XL; ++i) {
    const int row = m0 + 8 * (wave + 8 * i) + place_row;
    xoff[i] = (unsigned)(((row < m ? row : m - 1) * lda + place_chunk * 8) * 2);
  }
#pragma unroll
  for (int i = 0; i < WL; ++i) {
    const int row = n0 + 8 * (wave + 8 * i) + place_row;
    woff[i] = (unsigned)(((row < n ? row : n - 1) * k + place_chunk * 8) * 2);
  }
  // this lane's fragment of rows 16 j .. 16 j + 15, k half c: row r, chunk 4 c + g
  const int frag_row = (r >> 3) * 512 + (r & 7) * 64;               // elements; + 16 j * 64
  const int turn = ((r >> 1) & 3) << 1;
  const int frag0 = frag_row + ((g ^ turn) * 8), frag1 = frag_row + (((4 + g) ^ turn) * 8);
  floatx4 acc[IT][JT];
#pragma unroll
  for (int it = 0; it < IT; ++it)
#pragma unroll
    for (int jt = 0; jt < JT; ++jt) acc[it][jt] = floatx4{0.f, 0.f, 0.f, 0.f};
  // with K divided between workgroups, this one walks the slices step0 .. step0 + steps - 1 and leaves its sums
  // in part `split` of out [splits, m, ldc]
  const int steps_of_k = k / BK, steps_each = (steps_of_k + splits - 1) / splits, step0 = split * steps_each;
  const int steps = steps_of_k - step0 < steps_each ? steps_of_k - step0 : steps_each;
  const unsigned slices_address = (unsigned)(uintptr_t)(__attribute__((address_space(3))) bf16*)slices;
  auto fetch = [&](int kt, int stage) {                             // XL + WL fetches a wave
    const int at = (step0 + (kt < steps ? kt : steps - 1)) * BK * 2;
    const unsigned to = slices_address + (unsigned)(stage * STAGE_ELEMENTS * 2 + wave * 1024);
#pragma unroll
    for (int i = 0; i < XL; ++i) fetch_to_lds((const char*)x + at, xoff[i], to + (unsigned)(i * 8192));
#pragma unroll
    for (int i = 0; i < WL; ++i) fetch_to_lds((const char*)w + at, woff[i], to + (unsigned)(BM * BK * 2 + i * 8192));
  };
  auto multiply = [&](int stage) {
    const bf16* xs = slices + stage * STAGE_ELEMENTS;
    const bf16* ws = xs + BM * BK;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const int frag = c ? frag1 : frag0;
      bf16x8 xf[JT];
#pragma unroll
      for (int jt = 0; jt < JT; ++jt) xf[jt] = *(const bf16x8*)(xs + frag + (wm + jt * 16) * BK);
#pragma unroll
      for (int it = 0; it < IT; ++it) {
        const bf16x8 wf = *(const bf16x8*)(ws + frag + (wn + it * 16) * BK);
#pragma unroll
        for (int jt = 0; jt < JT; ++jt) acc[it][jt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, xf[jt], acc[it][jt], 0, 0, 0);
      }
    }
  };
  // Slice kt is multiplied from stage kt % STAGES while the slices after it arrive; a stage is filled again a
  // barrier after it was last read.  Before the barrier a wave waits until only the fetches it asked for in
  // this turn (none, with two stages) are still on their way: the next slice is then in LDS.
  int m0_opaque = m0;
  fetch(0, 0);
  if (STAGES == 3) fetch(1, 1);
  fetched_then_barrier<PENDING>();
  int stage = 0;
  for (int kt = 0; kt < steps; ++kt) {
    fetch(kt + STAGES - 1, stage == 0 ? STAGES - 1 : stage - 1);
    multiply(stage);
    fetched_then_barrier<PENDING>();
    stage = stage == STAGES - 1 ? 0 : stage + 1;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");               // the fetches past K that nobody reads
  asm volatile("" : "+s"(ldc), "+s"(m0_opaque));
#pragma unroll
  for (int jt = 0; jt < JT; ++jt) {
    const int token = m0_opaque + wm + jt * 16 + r;
    const int64_t row_at = ((int64_t)split * m + token) * ldc;
#pragma unroll
    for (int it = 0; it < IT; ++it) {
      const int tile0 = n0 + wn + it * 16, row0 = tile0 + 4 * g;     // this lane's four weight rows = output columns
      if (SWIGLU) {
        floatx4 up;
#pragma unroll
        for (int i = 0; i < 4; ++i) up[i] = __shfl(acc[it][jt][i], (lane + 32) % WAVE, WAVE);
        if (g < 2 && token < m && tile0 + 15 < n) {
          const floatx4 gate = acc[it][jt];
          const bf16x4 y = {(bf16)(silu(gate[0]) * up[0]), (bf16)(silu(gate[1]) * up[1]), (bf16)(silu(gate[2]) * up[2]), (bf16)(silu(gate[3]) * up[3])};
          *(bf16x4*)((bf16*)out + row_at + tile0 / 2 + 4 * g) = y;
        }
      } else if (token < m && row0 < n) {
        floatx4 v = acc[it][jt];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = __shfl(v[i], lane, WAVE);    // as in the kernel above: keeps the loop free of spills
        if constexpr (MODE == OUT_STORE) *(bf16x4*)((bf16*)out + row_at + row0) = bf16x4{(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
        else if constexpr (MODE == OUT_STORE_F32) *(floatx4*)((float*)out + row_at + row0) = v;
        else *(floatx4*)((float*)out + row_at + row0) = *(const floatx4*)((const float*)out + row_at + row0) + v;
      }
      __builtin_amdgcn_sched_barrier(0);
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
//
// NORM: the input is the float32 residual stream and the product is taken of its RMSNorm:
//   y[m, n] = rsqrt(mean_k h[m,k]^2 + eps) * sum_k (h[m,k] * g[k]) W[n,k]
// The row factor leaves the sum, so the B operand is bf16(h * g) and the factor is applied in
// the epilogue; the waves of a workgroup read all of K between them, so the sum of squares
// falls out of the loads they do anyway.  `rows` optionally picks the rows of h.
// SWIGLU: the 16 weight rows of a workgroup are 8 gate rows followed by the 8 up rows of the
// same features (the matrix is stored interleaved like that); the epilogue writes
// silu(gate) * up, 8 columns per workgroup, into out [M, N/2].
struct NormInput {
  const float* h;        // [*, K] float32, row stride lda
  const int* rows;       // optional: row of h for each of the m inputs
  const void* weight;    // [K] norm weight
  int weight_is_f32;
  float eps;
};

// A product between two RMSNorms of the residual stream can take the norm apart (at most 16 rows):
//   * the product that adds into the residual stream h also writes next_x = bf16(h_new * g), g the
//     weight of the norm that follows, and for each of its workgroups the sum of h_new^2 over the
//     workgroup's columns, next_sumsq [gridDim.x, m];
//   * the product that consumes the norm reads next_x as its input and multiplies row r of its
//     result by rsqrt(sum_p in_sumsq[p, r] / K + eps), the factor that is constant along K.
// The sums are added in a fixed order, so the result does not depend on the batch.
struct NormChain {
  const float* in_sumsq;   // consumer side: [in_parts, m], or null
  int in_parts;
  float in_eps;
  bf16* next_x;            // producer side: [m, n], or null
  float* next_sumsq;       // [gridDim.x, m]
  const void* next_weight; // [n]
  int next_weight_is_f32;
};


template <int MT, int RT, int WAVES, int UNROLL, bool NORM, bool SWIGLU, bool PARTIAL = false, bool LINES = false>
__global__ __launch_bounds__(WAVES * 64) void gemm_bf16_skinny_kernel(
    void* __restrict__ out, int mode, const bf16* __restrict__ x, NormInput norm,
    const bf16* __restrict__ w, const bf16* __restrict__ bias, int m, int n, int k, int lda, int ldc,
    float* __restrict__ split_sums, NormChain chain, int group_rows) {
  // RT: row tiles of 16 weight rows per workgroup; every activation fragment is used RT times.
  // group_rows (16 * RT unless PARTIAL): the weight rows a workgroup owns; fewer than its tiles hold
  // when that divides the matrix evenly between the compute units (rows past them are neither
  // loaded nor written).
  // gridDim.y > 1: K is also divided between workgroups; each then leaves its sums in
  // split_sums [gridDim.y, m, n] for gemm_split_finish_kernel instead of writing the output.
  // LINES: the weights come from memory as whole 128-byte lines (a load instruction brings 8 k chunks of
  // 8 rows; as fragments, 64 bytes of 16 rows, the same kilobyte touches 16 cache lines instead of 8, twice
  // the work for the address and tag units in front of the L1, which is what these kernels are short of) and take their places in the fragments through a patch of LDS of the
  // wave's own: two instructions fill 16 rows x 128 bytes, laid out as two panels (one per k step) of
  // 16 rows x 64 bytes with rows and chunks permuted so that writes and fragment reads meet no bank
  // conflicts; four steps go through the patch at a time.  No barrier: a wave's LDS instructions
  // execute in order.
  __shared__ bf16x8 patch_all[LINES ? WAVES : 1][2][128];
  // the activations likewise (8 tokens x 128 bytes an instruction, the second one only if there are more
  // than 8 tokens), through a patch of their own, two steps at a time
  __shared__ bf16x8 act_patch_all[LINES ? WAVES : 1][128];
  __shared__ floatx4 partial[WAVES][MT][WAVE];
  __shared__ float sumsq[WAVES][MT][16];
  __shared__ float chain_parts[WAVES * 4][16];   // in_sumsq, added up by WAVES * 4 threads per row
  __shared__ float chain_scale[16];
  __shared__ float chain_squares[16][RT * 16 + 1];
  const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * group_rows;
  const int n_end = n0 + group_rows < n ? n0 + group_rows : n;      // this workgroup's rows are [n0, n_end)
  const bf16* wp[RT];
  bool wrow[RT];
#pragma unroll
  for (int q = 0; q < RT; ++q) {
    wrow[q] = !PARTIAL || n0 + q * 16 + r < n_end;
    const int row = PARTIAL ? (wrow[q] ? n0 + q * 16 + r : n0) : (n0 + q * 16 + r < n ? n0 + q * 16 + r : n - 1);
    wp[q] = w + (int64_t)row * k + g * 8;
  }
  const bf16* wl[RT][2];
  bool wl_ok[RT][2];
  int wr_off[2], rd_off[2];
  bf16x8* const patch = &patch_all[LINES ? wave : 0][0][0];
  if constexpr (LINES) {
    auto place = [](int panel, int row, int chunk) -> int {
      return panel * 64 + ((row ^ ((row >> 3) & 1) ^ (panel & 1)) * 4 + (chunk ^ ((row >> 1) & 3)));
    };
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      wr_off[h] = place((lane % 8) / 4, 8 * h + lane / 8, lane % 4);
      rd_off[h] = place(h, r, g);
#pragma unroll
      for (int q = 0; q < RT; ++q) {
        const int row = n0 + q * 16 + 8 * h + lane / 8;
        wl_ok[q][h] = !PARTIAL || row < n_end;                 // PARTIAL: rows past the workgroup's own are the next one's
        wl[q][h] = w + (int64_t)(row < n ? row : n - 1) * k + (lane % 8) * 8;
      }
    }
  }
  const bf16* xl[2];
  bf16x8* const act_patch = &act_patch_all[LINES ? wave : 0][0];
  if constexpr (LINES) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int token = 8 * h + lane / 8;
      xl[h] = x + (int64_t)(token < m ? token : m - 1) * lda + (lane % 8) * 8;   // tokens past m: the last one's row, never written
    }
  }
  const bf16* xp[MT];
  const float* hp[MT];
  bool live[MT];
  float ss[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int token = t * 16 + r;
    live[t] = token < m;
    ss[t] = 0.f;
    if (NORM) {
      const int64_t src = live[t] ? (norm.rows ? norm.rows[token] : token) : 0;
      hp[t] = norm.h + src * lda + g * 8;
    } else {
      xp[t] = x + (int64_t)(live[t] ? token : 0) * lda + g * 8;
    }
  }
  floatx4 acc[RT][MT];
#pragma unroll
  for (int q = 0; q < RT; ++q)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[q][t] = floatx4{0.f, 0.f, 0.f, 0.f};
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  // B operand of one k step for token block t: 8 consecutive k of one token
  auto load_b = [&](int t, int step) -> bf16x8 {
    if (!live[t]) return zero;
    if (!NORM) return *(const bf16x8*)(xp[t] + step * 32);
    const floatx4 h0 = *(const floatx4*)(hp[t] + step * 32), h1 = *(const floatx4*)(hp[t] + step * 32 + 4);
    float gw[8];
    if (norm.weight_is_f32) {
      const floatx4 g0 = *(const floatx4*)((const float*)norm.weight + step * 32 + g * 8);
      const floatx4 g1 = *(const floatx4*)((const float*)norm.weight + step * 32 + g * 8 + 4);
#pragma unroll
      for (int i = 0; i < 4; ++i) { gw[i] = g0[i]; gw[4 + i] = g1[i]; }
    } else {
      const bf16x8 gb = *(const bf16x8*)((const bf16*)norm.weight + step * 32 + g * 8);
#pragma unroll
      for (int i = 0; i < 8; ++i) gw[i] = (float)gb[i];
    }
    bf16x8 b;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ss[t] = fmaf(h0[i], h0[i], ss[t]);
      ss[t] = fmaf(h1[i], h1[i], ss[t]);
      b[i] = (bf16)(h0[i] * gw[i]);
      b[4 + i] = (bf16)(h1[i] * gw[4 + i]);
    }
    return b;
  };

  const int all_steps = (k + 31) / 32;
  const int per_split = (all_steps + gridDim.y - 1) / gridDim.y;
  const int split_begin = blockIdx.y * per_split;
  const int split_end = split_begin + per_split < all_steps ? split_begin + per_split : all_steps;
  const int per_wave = (per_split + WAVES - 1) / WAVES;
  int s = split_begin + wave * per_wave;
  const int s_end = s + per_wave < split_end ? s + per_wave : split_end;
  const int full_end = k / 32 < s_end ? k / 32 : s_end;   // steps whose 32 k are all inside K
  // What the epilogue will need from memory is asked for now, before the weights stream, so that it
  // has long arrived by then: the partial sums of squares of the norm this product finishes, and
  // the residual values and norm weights of the columns this thread will update.
  const bool scaled_input = MT == 1 && !NORM && chain.in_sumsq != nullptr;
  const bool feeds_norm = MT == 1 && !SWIGLU && chain.next_x != nullptr && mode == OUT_ADD_F32 && gridDim.y == 1;
  constexpr int EARLY = 16;
  const bool sums_early = scaled_input && chain.in_parts <= WAVES * 4 * EARLY;
  float early_sums[EARLY];
  if (sums_early) {
    const int token = tid % 16, part = tid / 16;
#pragma unroll
    for (int j = 0; j < EARLY; ++j) {
      const int p = part + j * WAVES * 4;
      early_sums[j] = (token < m && p < chain.in_parts) ? chain.in_sumsq[(int64_t)p * m + token] : 0.f;
    }
  }
  float early_h[RT], early_w[RT];
  if (feeds_norm && tid < WAVE * 4) {
    const int l = tid / 4, i = tid % 4, token = l & 15;
#pragma unroll
    for (int q = 0; q < RT; ++q) {
      const int gn = n0 + q * 16 + 4 * (l >> 4) + i;
      const bool inside = token < m && gn < n_end;
      early_h[q] = inside ? ((const float*)out)[(int64_t)token * ldc + gn] : 0.f;
      early_w[q] = !inside ? 0.f : chain.next_weight_is_f32 ? ((const float*)chain.next_weight)[gn] : (float)((const bf16*)chain.next_weight)[gn];
    }
  }
  // U steps of 32 k, all their loads asked for before any is used
  auto steps_together = [&](int sb, auto count) {
    constexpr int U = decltype(count)::value;
    if constexpr (LINES && U % 4 == 0) {
      static_assert(MT == 1, "whole-line loads are for one block of tokens");
      bf16x8 raw[U][RT], rawb[U / 2][2];
      const bool second = m > 8;                       // the same for the whole grid
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int q = 0; q < RT; ++q) raw[u][q] = wl_ok[q][u & 1] ? *(const bf16x8*)(wl[q][u & 1] + (sb + (u & ~1)) * 32) : zero;
#pragma unroll
      for (int p = 0; p < U / 2; ++p) {
        rawb[p][0] = *(const bf16x8*)(xl[0] + (sb + 2 * p) * 32);
        rawb[p][1] = second ? *(const bf16x8*)(xl[1] + (sb + 2 * p) * 32) : zero;
      }
#pragma unroll
      for (int c4 = 0; c4 < U; c4 += 4) {
        bf16x8 b[4];
#pragma unroll
        for (int p = 0; p < 2; ++p) {                  // two steps of activations through their patch at a time
          act_patch[wr_off[0]] = rawb[c4 / 2 + p][0];
          act_patch[wr_off[1]] = rawb[c4 / 2 + p][1];
          b[2 * p] = act_patch[rd_off[0]];
          b[2 * p + 1] = act_patch[rd_off[1]];
        }
#pragma unroll
        for (int q = 0; q < RT; ++q) {
#pragma unroll
          for (int i = 0; i < 4; ++i) patch[(i >> 1) * 128 + wr_off[i & 1]] = raw[c4 + i][q];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const bf16x8 a = patch[(i >> 1) * 128 + rd_off[i & 1]];
            acc[q][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b[i], acc[q][0], 0, 0, 0);
          }
        }
      }
      return;
    }
    bf16x8 a[U][RT], b[U][MT];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int q = 0; q < RT; ++q) a[u][q] = !PARTIAL || wrow[q] ? *(const bf16x8*)(wp[q] + (sb + u) * 32) : zero;
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t) b[u][t] = load_b(t, sb + u);
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int q = 0; q < RT; ++q)
#pragma unroll
        for (int t = 0; t < MT; ++t)
          acc[q][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][q], b[u][t], acc[q][t], 0, 0, 0);
  };
  // Workgroups walk their K slices from different starting points (the order of a column's sum
  // depends on the column alone): all of them read the same activations, and in step they would
  // all ask the same few cache lines of the L2 at the same moment.
  const int batches = full_end > s ? (full_end - s) / UNROLL : 0;
  const int s_first = s;
  for (int j = 0; j < batches; ++j)
    steps_together(s_first + ((j + (int)blockIdx.x) % batches) * UNROLL, std::integral_constant<int, UNROLL>{});
  s = s_first + batches * UNROLL;
  // what is left of the whole steps, in shrinking groups (a step alone costs a trip to memory of its own)
  if constexpr (UNROLL > 4) {
    if (full_end - s >= 4) {
      steps_together(s, std::integral_constant<int, 4>{});
      s += 4;
    }
  }
  if constexpr (UNROLL > 2) {
    if (full_end - s >= 2) {
      steps_together(s, std::integral_constant<int, 2>{});
      s += 2;
    }
  }
  for (; s < s_end; ++s) {
    const bool inside = s * 32 + g * 8 < k;
    bf16x8 b[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) b[t] = inside ? load_b(t, s) : zero;
#pragma unroll
    for (int q = 0; q < RT; ++q) {
      const bf16x8 a = inside && (!PARTIAL || wrow[q]) ? *(const bf16x8*)(wp[q] + s * 32) : zero;
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[q][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b[t], acc[q][t], 0, 0, 0);
    }
  }
  if (NORM) {
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      float v = ss[t];
      v += __shfl_xor(v, 16, WAVE);
      v += __shfl_xor(v, 32, WAVE);
      if (g == 0) sumsq[wave][t][r] = v;
    }
  }
  if (scaled_input) {
    const int token = tid % 16, part = tid / 16;
    float v = 0.f;
    if (sums_early) {
#pragma unroll
      for (int j = 0; j < EARLY; ++j) v += early_sums[j];      // the order of the loop below
    } else if (token < m) {
      for (int p = part; p < chain.in_parts; p += WAVES * 4) v += chain.in_sumsq[(int64_t)p * m + token];
    }
    chain_parts[part][token] = v;
    __syncthreads();
    if (tid < 16) {
      float q = 0.f;
#pragma unroll
      for (int p = 0; p < WAVES * 4; ++p) q += chain_parts[p][tid];
      chain_scale[tid] = 1.0f / sqrtf(q / (float)k + chain.in_eps);
    }
  }
  // accumulator layout: token = t*16 + lane % 16, weight row = tile row 4 * (lane / 16) + i
  auto total = [&](int t, int l, int i) -> float {
    float v = 0.f;
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv) v += partial[wv][t][l][i];
    if (scaled_input) v *= chain_scale[l & 15];
    if (NORM) {
      float q = 0.f;
#pragma unroll
      for (int wv = 0; wv < WAVES; ++wv) q += sumsq[wv][t][l & 15];
      v *= 1.0f / sqrtf(q / (float)k + norm.eps);
    }
    return v;
  };
#pragma unroll
  for (int q = 0; q < RT; ++q) {
    if (q) __syncthreads();
#pragma unroll
    for (int t = 0; t < MT; ++t) partial[wave][t][lane] = acc[q][t];
    __syncthreads();
    const int nq0 = n0 + q * 16;
    if (gridDim.y > 1) {
      for (int e = tid; e < MT * WAVE * 4; e += WAVES * WAVE) {
        const int t = e / (WAVE * 4), l = (e / 4) % WAVE, i = e % 4;
        const int token = t * 16 + (l & 15), gn = nq0 + 4 * (l >> 4) + i;
        if (token < m && gn < n_end) split_sums[((int64_t)blockIdx.y * m + token) * n + gn] = total(t, l, i);
      }
    } else if (SWIGLU) {
      for (int e = tid; e < MT * 16 * 8; e += WAVES * WAVE) {
        const int t = e / 128, c = (e / 8) % 16, j = e % 8;
        const int token = t * 16 + c, feature = nq0 / 2 + j;
        if (token >= m || nq0 + 8 + j >= n) continue;
        const float gate = total(t, ((j / 4) << 4) | c, j % 4), up = total(t, ((2 + j / 4) << 4) | c, j % 4);
        emit<bf16>(out, mode, (int64_t)token * ldc + feature, silu(gate) * up);
      }
    } else {
      for (int e = tid; e < MT * WAVE * 4; e += WAVES * WAVE) {
        const int t = e / (WAVE * 4), l = (e / 4) % WAVE, i = e % 4;
        const int token = t * 16 + (l & 15), gn = nq0 + 4 * (l >> 4) + i;
        const bool inside = token < m && gn < n_end;
        if (feeds_norm && !inside) chain_squares[l & 15][q * 16 + 4 * (l >> 4) + i] = 0.f;
        if (!inside) continue;
        float v = total(t, l, i);
        if (bias) v += (float)bias[gn];
        if (feeds_norm) {                                        // MT == 1: e == tid, the element asked for early
          const float updated = early_h[q] + v;
          ((float*)out)[(int64_t)token * ldc + gn] = updated;
          chain.next_x[(int64_t)token * n + gn] = (bf16)(updated * early_w[q]);
          chain_squares[l & 15][q * 16 + 4 * (l >> 4) + i] = updated * updated;
        } else {
          emit<bf16>(out, mode, (int64_t)token * ldc + gn, v);
        }
      }
    }
  }
  if (feeds_norm) {
    __syncthreads();
    if (tid < m) {
      float q = 0.f;
#pragma unroll
      for (int c = 0; c < RT * 16; ++c) q += chain_squares[tid][c];
      chain.next_sumsq[(int64_t)blockIdx.x * m + tid] = q;
    }
  }
}

// Adds up what the K splits left in split_sums [splits, m, n], in split order, and writes the output
// with the same epilogues as the product kernels.
template <bool SWIGLU>
__global__ void gemm_split_finish_kernel(void* __restrict__ out, int mode, const float* __restrict__ split_sums,
                                         const bf16* __restrict__ bias, int m, int n, int ldc, int splits) {
  const int columns = SWIGLU ? n / 2 : n;
  if (!SWIGLU && !bias && n % 4 == 0 && ldc % 4 == 0 && (uintptr_t)out % 16 == 0) {
    // four columns a thread, 16 bytes a load
    const int quads = n / 4;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < (int64_t)m * quads; e += (int64_t)gridDim.x * blockDim.x) {
      const int token = e / quads, c = (e % quads) * 4;
      floatx4 v = {0.f, 0.f, 0.f, 0.f};
      for (int sp = 0; sp < splits; ++sp) v += *(const floatx4*)(split_sums + ((int64_t)sp * m + token) * n + c);
      const int64_t at = (int64_t)token * ldc + c;
      if (mode == OUT_STORE) *(bf16x4*)((bf16*)out + at) = bf16x4{(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
      else if (mode == OUT_STORE_F32) *(floatx4*)((float*)out + at) = v;
      else *(floatx4*)((float*)out + at) = *(const floatx4*)((const float*)out + at) + v;
    }
    return;
  }
  for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < (int64_t)m * columns; e += (int64_t)gridDim.x * blockDim.x) {
    const int token = e / columns, c = e % columns;
    const int gn = SWIGLU ? 16 * (c / 8) + c % 8 : c;
    float v = 0.f, up = 0.f;
    for (int sp = 0; sp < splits; ++sp) {
      v += split_sums[((int64_t)sp * m + token) * n + gn];
      if (SWIGLU) up += split_sums[((int64_t)sp * m + token) * n + gn + 8];
    }
    if (SWIGLU) v = silu(v) * up;
    else if (bias) v += (float)bias[gn];
    emit<bf16>(out, mode, (int64_t)token * ldc + c, v);
  }
}

// ------------------------------------------------- bf16 kernel for 17..128 rows
// (MT blocks of 16 tokens: 2, 3, 4, 6 or 8.)  Between the few-rows kernel (every wave reads its activations from L2 itself) and the many-rows
// kernel (both operands tiled through LDS): the weights are still streamed exactly once, as the MFMA A
// operand straight from memory into registers, but with several 16-token blocks the activations are
// as many bytes as the weights of a workgroup, so the waves of a workgroup (each with 16 weight rows
// of its own) share them through LDS.  K is walked in slices of 256: while a slice is multiplied,
// the weights of the next two slices are on their way into registers and the activations of the
// next slice lie in the other LDS buffer, loaded as whole 128-byte lines and laid out so that fragment reads
// meet no bank conflicts (see below).  gridDim.y > 1 divides K between
// workgroups; with split_sums given every workgroup leaves its sums there ([gridDim.y, m, n]) for a
// kernel that adds them up (gemm_split_finish_kernel, or the residual add and norm that follow).  K % 256 == 0.
// The input may be an RMSNorm that the kernel before began (see NormChain): x = bf16(h * norm weight) and partial
// sums of h^2 per row, sumsq [parts, m]; row r of the result (of every K split's sums alike: the factor is
// constant along K) is then multiplied by rsqrt(sum_p sumsq[p, r] / K + eps).
struct MidScale {
  const float* sumsq;   // null: the input is what it is
  int parts;
  float eps;
};

//
// EXTRA (4, 6 or 8 waves, up to 64 rows): the weight rows are dealt out in tiles of 16 so that every workgroup of the
// launch has WAVES or WAVES + 1 of them (the first `extras` workgroups the one more), which lets a launch be a whole
// multiple of the compute units whatever n is: the launch takes as long as the unit with the most to fetch.  The
// extra tile has no wave of its own: its k steps are dealt out over the waves (step s of a slice to wave s % WAVES:
// one each with eight waves, two with four, one or two with six), which multiply them by the activation fragments
// they hold anyway; the waves' partial sums meet in LDS at the end, are added in wave order and written by the
// first MT waves.
template <int MT, int WAVES, bool SWIGLU, bool EXTRA = false>
__global__ __launch_bounds__(WAVES * 64) void gemm_bf16_mid_kernel(
    void* __restrict__ out, int mode, const bf16* __restrict__ x, const bf16* __restrict__ w,
    int m, int n, int k, int lda, int ldc, float* __restrict__ split_sums, MidScale scale, int extras) {
  static_assert(!EXTRA || ((WAVES == 4 || WAVES == 6 || WAVES == 8) && MT <= 4), "the extra tile needs 4, 6 or 8 waves and at most 64 rows");
  constexpr int STEPS = 8;                         // k steps of 32 in a slice
  constexpr int XS = EXTRA ? (STEPS + WAVES - 1) / WAVES : 1;    // most steps of the extra tile that a wave multiplies in a slice
  constexpr int FRAGS = STEPS * MT;                // activation fragments of a slice
  constexpr int MINE = (FRAGS + WAVES - 1) / WAVES;  // of which a wave brings this many
  // LDS (dynamic: more than the 64 KB a static array may have): two buffers of activations, then a patch of
  // 4 KB for each wave through which its weights, loaded as whole 128-byte lines (8 k chunks of 8 rows an
  // instruction), take their places in the A fragments (see gemm_bf16_skinny_kernel, LINES).
  extern __shared__ __attribute__((aligned(16))) bf16x8 mid_lds[];
  const int tid = threadIdx.x, lane = tid % WAVE, wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
  const int r = lane & 15, g = lane >> 4;
  const int tile0 = EXTRA ? (int)blockIdx.x * WAVES + ((int)blockIdx.x < extras ? (int)blockIdx.x : extras) : (int)blockIdx.x * WAVES;
  const int row0 = (tile0 + wave) * 16;
  const bool has_extra = EXTRA && (int)blockIdx.x < extras;        // the same for every wave of the workgroup
  const int row_x = (tile0 + WAVES) * 16;                          // first row of the extra tile
  bf16x8* const patch = mid_lds + 2 * STEPS * MT * WAVE + wave * 256;
  const bf16* wl[2];
  int wr_off[2], rd_off[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    auto spot_of = [](int panel, int row, int chunk) -> int {
      return panel * 64 + ((row ^ ((row >> 3) & 1) ^ (panel & 1)) * 4 + (chunk ^ ((row >> 1) & 3)));
    };
    const int row = row0 + 8 * h + lane / 8;
    wl[h] = w + (int64_t)(row < n ? row : n - 1) * k + (lane % 8) * 8;
    wr_off[h] = spot_of((lane % 8) / 4, 8 * h + lane / 8, lane % 4);
    rd_off[h] = spot_of(h, r, g);
  }
  const int slices = k / 256;
  const int per_split = (slices + gridDim.y - 1) / gridDim.y;
  const int s0 = blockIdx.y * per_split;
  const int count = (s0 + per_split < slices ? s0 + per_split : slices) - s0;
  // Workgroups walk their slices from different starting points (round the ring): all of them read the
  // same activations, and in step they would all ask the same cache lines at the same moment.  The order
  // of a column's sum then depends on the column's workgroup alone.
  const int turn = count > 0 ? (int)(blockIdx.x % (unsigned)count) : 0;
  auto slice_at = [&](int c) -> int { const int v = c + turn; return s0 + (v >= count ? v - count : v); };
  // The activations of a slice come from memory as whole 128-byte lines: a load instruction brings 8 k
  // chunks (16 bytes each) of 8 tokens, FRAGS such pieces a slice, dealt out over the waves.  (Loaded as
  // B fragments, 64 bytes of 16 tokens an instruction, they cost a fifth of the kernel's time at 64 rows.)
  // In LDS a slice is 8 panels (one per k step) of MT blocks of 16 tokens; a token's row in a block is
  // its 4 chunks of that step, 64 bytes, and rows and chunks are permuted like this: rows swap places in
  // pairs in the upper half of a block, chunks are turned round by the row number, and odd panels swap
  // neighbouring rows once more.  A fragment read (lane = token % 16 + 16 * chunk) then touches every
  // bank once in each of its quarter-waves, and the 8 chunks of a token that one lane group of a load
  // writes fall into the two halves of a 128-byte bank line.  Address in 16-byte units:
  //   panel * MT * 64 + block * 64 + (row ^ (row >> 3 & 1) ^ (panel & 1)) * 4 + (chunk ^ (row >> 1 & 3))
  // Every load and every LDS write below is unconditional, so that the compiler can count the loads
  // in flight instead of waiting for all of them at a branch: a token past m reads the last token's
  // row (its columns of the result are never written), and where the pieces do not divide evenly
  // between the waves the spare turns bring the last piece once more (same data, same place).
  auto place = [&](int panel, int block, int row, int chunk) -> int {
    return panel * (MT * 64) + block * 64 + ((row ^ ((row >> 3) & 1) ^ (panel & 1)) * 4 + (chunk ^ ((row >> 1) & 3)));
  };
  const bf16* xp[MINE];
  bf16x8* spot[MINE];
  bf16x8* const lds = mid_lds;
#pragma unroll
  for (int i = 0; i < MINE; ++i) {
    const int piece = wave + i * WAVES < FRAGS ? wave + i * WAVES : FRAGS - 1;
    const int oct = piece % (2 * MT), line = piece / (2 * MT);              // 8 tokens, 128 bytes of the slice
    const int tok = oct * 8 + lane / 8, chunk = line * 8 + lane % 8;
    xp[i] = x + (int64_t)(tok < m ? tok : m - 1) * lda + chunk * 8;
    spot[i] = lds + place(chunk / 4, tok / 16, tok % 16, chunk % 4);
  }
  // the factors of a norm begun before this product: one thread a token adds up the parts now (the loads run
  // beside the weights') and keeps the factor; after the last slice they go through LDS to the lanes that need them
  float my_scale = 1.f;
  if (scale.sumsq && tid < m) {
    float q = 0.f;
    for (int p0 = 0; p0 < scale.parts; p0 += 8) {      // eight parts asked for at a time (usually all there are)
      float part[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) part[j] = p0 + j < scale.parts ? scale.sumsq[(int64_t)(p0 + j) * m + tid] : 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) q += part[j];
    }
    my_scale = 1.0f / sqrtf(q / (float)k + scale.eps);
  }
  floatx4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
  bf16x8 wa[STEPS], wb[STEPS], sa[MINE], sb[MINE];
  // the extra tile: this wave's steps of it as A fragments straight from memory (row = lane % 16, 8 k from 8 * (lane / 16))
  floatx4 acc_x[MT];
  bf16x8 xa[XS], xb[XS];
  const bf16* xl = w;
  if constexpr (EXTRA) {
#pragma unroll
    for (int t = 0; t < MT; ++t) acc_x[t] = floatx4{0.f, 0.f, 0.f, 0.f};
    xl = w + (int64_t)(row_x + r < n ? row_x + r : n - 1) * k + g * 8 + wave * 32;
  }
  auto load_x = [&](int slice, bf16x8 (&xf)[XS]) {
    if constexpr (EXTRA) {
      if (has_extra) {
#pragma unroll
        for (int j = 0; j < XS; ++j)
          if (STEPS % WAVES == 0 || wave + j * WAVES < STEPS) xf[j] = *(const bf16x8*)(xl + (int64_t)slice * 256 + j * (WAVES * 32));
      }
    }
  };
  // a[2 p + h]: line p (k steps 2 p and 2 p + 1) of rows 8 h .. 8 h + 7
  auto load_w = [&](int slice, bf16x8 (&a)[STEPS]) {
#pragma unroll
    for (int j = 0; j < STEPS; ++j) a[j] = *(const bf16x8*)(wl[j & 1] + (int64_t)slice * 256 + (j >> 1) * 64);
  };
  auto load_acts = [&](int slice, bf16x8 (&st)[MINE]) {
#pragma unroll
    for (int i = 0; i < MINE; ++i) st[i] = *(const bf16x8*)(xp[i] + (int64_t)slice * 256);
  };
  auto store_acts = [&](int buf, const bf16x8 (&st)[MINE]) {
#pragma unroll
    for (int i = 0; i < MINE; ++i) spot[i][buf * (STEPS * MT * WAVE)] = st[i];
  };
  // Multiplies the slice in LDS buffer `buf` by the weights in a[].  RELOAD: every a[j] is asked again,
  // for slice `next`, as soon as its products are issued (the scheduling barriers keep the compiler
  // from gathering these loads at the end, where they would leave the memory idle meanwhile).  The
  // activation fragments of a step are read from LDS while the step before is multiplied.
  const bf16x8* const frag_even = lds + place(0, 0, r, g);    // this lane's piece of a fragment in an even panel ...
  const bf16x8* const frag_odd = lds + place(1, 0, r, g) - MT * 64;   // ... and in an odd one, less the panel's own offset
  auto compute = [&](int buf, bf16x8 (&a)[STEPS], bf16x8 (&xf)[XS], auto reload, int next) {
    constexpr bool RELOAD = decltype(reload)::value;
    const bf16x8* const even = frag_even + buf * (STEPS * MT * WAVE);
    const bf16x8* const odd = frag_odd + buf * (STEPS * MT * WAVE);
    bf16x8 b[2][MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) b[0][t] = even[t * WAVE];
#pragma unroll
    for (int p = 0; p < STEPS / 2; ++p) {
      // two load instructions' worth (16 rows x 128 bytes) through the wave's patch: the A fragments of two steps
      bf16x8* const pp = patch + (p & 1) * 128;
      pp[wr_off[0]] = a[2 * p];
      pp[wr_off[1]] = a[2 * p + 1];
      const bf16x8 f0 = pp[rd_off[0]], f1 = pp[rd_off[1]];
      if constexpr (RELOAD) {
        a[2 * p] = *(const bf16x8*)(wl[0] + (int64_t)next * 256 + p * 64);
        a[2 * p + 1] = *(const bf16x8*)(wl[1] + (int64_t)next * 256 + p * 64);
      }
#pragma unroll
      for (int t = 0; t < MT; ++t) b[1][t] = odd[((2 * p + 1) * MT + t) * WAVE];
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f0, b[0][t], acc[t], 0, 0, 0);
      if constexpr (EXTRA) {       // step 2 p of the extra tile is the business of wave 2 p % WAVES
        if (has_extra && wave == (2 * p) % WAVES) {
#pragma unroll
          for (int t = 0; t < MT; ++t) acc_x[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xf[(2 * p) / WAVES], b[0][t], acc_x[t], 0, 0, 0);
        }
      }
      if (2 * p + 2 < STEPS) {
#pragma unroll
        for (int t = 0; t < MT; ++t) b[0][t] = even[((2 * p + 2) * MT + t) * WAVE];
      }
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f1, b[1][t], acc[t], 0, 0, 0);
      if constexpr (EXTRA) {
        if (has_extra && wave == (2 * p + 1) % WAVES) {
#pragma unroll
          for (int t = 0; t < MT; ++t) acc_x[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xf[(2 * p + 1) / WAVES], b[1][t], acc_x[t], 0, 0, 0);
        }
      }
      if constexpr (RELOAD) __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (RELOAD) load_x(next, xf);
  };
  const std::true_type again;
  const std::false_type last;
  // While slice c is multiplied, the weights of slice c + 1 are in registers or on their way and those of
  // slice c + 2 are asked for as the products of c are issued; the activations of slice c + 1 go from
  // staging registers into the LDS buffer that slice c - 1 has left, and those of the slices after it are on
  // their way into the staging registers: two sets of them in turn (slices c + 2 and c + 3) up to 64 rows, one
  // set (slice c + 2) beyond, where registers are short.
  // (six waves with an extra tile at 64 rows have no registers for the second set either)
  constexpr bool TWO_SETS = MT <= 4 && !(EXTRA && WAVES == 6 && MT == 4);
  int c = 0;
  if constexpr (TWO_SETS) {
    if (count > 0) {
      load_w(slice_at(0), wa);
      load_x(slice_at(0), xa);
      load_acts(slice_at(0), sa);
    }
    if (count > 1) {
      load_w(slice_at(1), wb);
      load_x(slice_at(1), xb);
      load_acts(slice_at(1), sb);
    }
    if (count > 0) store_acts(0, sa);
    if (count > 2) load_acts(slice_at(2), sa);
    // slice c: after the barrier LDS buffer c & 1 holds it and nobody reads the other buffer any more
    auto steady = [&](int c, bf16x8 (&a)[STEPS], bf16x8 (&xf)[XS], bf16x8 (&st)[MINE]) {
      __syncthreads();
      store_acts((c & 1) ^ 1, st);                       // slice c + 1
      load_acts(slice_at(c + 3), st);
      compute(c & 1, a, xf, again, slice_at(c + 2));
    };
    auto ending = [&](int c, bf16x8 (&a)[STEPS], bf16x8 (&xf)[XS], bf16x8 (&st)[MINE]) {
      __syncthreads();
      if (c + 1 < count) store_acts((c & 1) ^ 1, st);
      if (c + 3 < count) load_acts(slice_at(c + 3), st);
      if (c + 2 < count) compute(c & 1, a, xf, again, slice_at(c + 2));
      else compute(c & 1, a, xf, last, 0);
    };
    for (; c + 4 < count; c += 2) {            // no branch inside: slices up to c + 4 exist
      steady(c, wa, xa, sb);
      steady(c + 1, wb, xb, sa);
    }
    for (; c < count; c += 2) {                // the last one to four slices
      ending(c, wa, xa, sb);
      if (c + 1 >= count) break;
      ending(c + 1, wb, xb, sa);
    }
  } else {
    if (count > 0) {
      load_w(slice_at(0), wa);
      load_x(slice_at(0), xa);
      load_acts(slice_at(0), sa);
    }
    if (count > 1) {
      load_w(slice_at(1), wb);
      load_x(slice_at(1), xb);
    }
    if (count > 0) store_acts(0, sa);
    if (count > 1) load_acts(slice_at(1), sa);
    auto steady = [&](int c, bf16x8 (&a)[STEPS], bf16x8 (&xf)[XS]) {
      __syncthreads();
      store_acts((c & 1) ^ 1, sa);                       // slice c + 1
      load_acts(slice_at(c + 2), sa);
      compute(c & 1, a, xf, again, slice_at(c + 2));
    };
    auto ending = [&](int c, bf16x8 (&a)[STEPS], bf16x8 (&xf)[XS]) {
      __syncthreads();
      if (c + 1 < count) store_acts((c & 1) ^ 1, sa);
      if (c + 2 < count) {
        load_acts(slice_at(c + 2), sa);
        compute(c & 1, a, xf, again, slice_at(c + 2));
      } else {
        compute(c & 1, a, xf, last, 0);
      }
    };
    for (; c + 3 < count; c += 2) {            // no branch inside: slices up to c + 3 exist
      steady(c, wa, xa);
      steady(c + 1, wb, xb);
    }
    for (; c < count; c += 2) {                // the last one to three slices
      ending(c, wa, xa);
      if (c + 1 >= count) break;
      ending(c + 1, wb, xb);
    }
  }
  // accumulator layout: token = t * 16 + lane % 16, weight rows row0 + 4 * (lane / 16) + 0..3
  if (scale.sumsq) {
    float* const row_scales = (float*)mid_lds;     // the activation buffers have done their work
    __syncthreads();
    if (tid < m) row_scales[tid] = my_scale;
    __syncthreads();
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] *= row_scales[t * 16 + r < m ? t * 16 + r : 0];
  }
  // one block of 16 tokens of a tile of 16 weight rows that begins at row `first`: the wave's own, or the extra one
  auto emit_block = [&](int t, floatx4 v, int first) {
    const int token = t * 16 + r, gn = first + 4 * g;
    if (split_sums) {
      if (token < m && gn < n) *(floatx4*)(split_sums + ((int64_t)blockIdx.y * m + token) * n + gn) = v;
      return;
    }
    if constexpr (SWIGLU) {
      // the 16 rows of a tile are 8 gate rows and the 8 up rows of the same features: the up values
      // of a lane's gate rows sit 32 lanes further on
      floatx4 up;
#pragma unroll
      for (int i = 0; i < 4; ++i) up[i] = __shfl(v[i], (lane + 32) & 63, WAVE);
      if (g < 2 && token < m && first < n) {
        bf16x4 y;
#pragma unroll
        for (int i = 0; i < 4; ++i) y[i] = (bf16)(silu(v[i]) * up[i]);
        *(bf16x4*)((bf16*)out + (int64_t)token * ldc + first / 2 + 4 * g) = y;
      }
    } else if (token < m && gn < n) {
      if (mode == OUT_STORE) *(bf16x4*)((bf16*)out + (int64_t)token * ldc + gn) = bf16x4{(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
      else if (mode == OUT_STORE_F32) *(floatx4*)((float*)out + (int64_t)token * ldc + gn) = v;
      else *(floatx4*)((float*)out + (int64_t)token * ldc + gn) = *(const floatx4*)((const float*)out + (int64_t)token * ldc + gn) + v;
    }
  };
  if constexpr (EXTRA) {
    if (has_extra) {
      // the waves' partial sums of the extra tile, [wave][block][lane], behind the row factors at the head of LDS
      floatx4* const meet = (floatx4*)mid_lds + 64;
      __syncthreads();                               // nobody reads activations any more (and the row factors are written)
#pragma unroll
      for (int t = 0; t < MT; ++t) meet[(wave * MT + t) * WAVE + lane] = acc_x[t];
      __syncthreads();
      if (wave < MT) {
        floatx4 v = meet[wave * WAVE + lane];
        for (int other = 1; other < WAVES; ++other) v += meet[(other * MT + wave) * WAVE + lane];
        if (scale.sumsq) v *= ((const float*)mid_lds)[wave * 16 + r < m ? wave * 16 + r : 0];
        emit_block(wave, v, row_x);
      }
    }
  }
#pragma unroll
  for (int t = 0; t < MT; ++t) emit_block(t, acc[t], row0);
}

// Choices a caller may make for the products (measurements and tests; a step carries its runner's).  They
// travel with every call as one word, so that nothing about them is kept in the library:
//   bit 0      the kernel for 17..128 rows may be used (else such products take the kernels for other row counts)
//   bit 1      the few-rows kernel loads its weights as whole 128-byte lines where the shape allows
//   bits 4-7   workgroup shape of the kernel for 17..128 rows: 4, 5, 6 or 8 waves (0: chosen here)
//   bits 8-12  its number of K splits, 1..16 (0: chosen here)
//   bits 13-14 its weight rows dealt out evenly over a whole multiple of the compute units, some workgroups with a
//              tile more than the others (see the kernel, EXTRA): 0: where it pays (chosen here), 1: never, 2: wherever
//              the shape allows
struct GemmTune {
  bool mid, lines;
  int waves, splits, even;
};
constexpr int TUNE_DEFAULT = 3;
static bool tune_ok(int word) {
  const int waves = (word >> 4) & 15, splits = (word >> 8) & 31, even = (word >> 13) & 3;
  return word >= 0 && (word >> 15) == 0 && (waves == 0 || waves == 4 || waves == 5 || waves == 6 || waves == 8) && splits <= 16 && even <= 2;
}
static GemmTune tune_of(int word) { return GemmTune{(word & 1) != 0, (word & 2) != 0, (word >> 4) & 15, (word >> 8) & 31, (word >> 13) & 3}; }

// Row tiles per workgroup: more of them means each activation fragment read from L2 serves more
// weight rows, which matters once there are several token blocks; fewer means more workgroups.
template <int MT, int RT, bool NORM, bool SWIGLU>
static void launch_skinny_rt(void* out, int mode, const bf16* a, NormInput norm, const bf16* w, const bf16* bias,
                             int m, int n, int k, int lda, int ldc, hipStream_t s, GemmTune tune, float* split_sums = nullptr, int splits = 1,
                             NormChain chain = NormChain{}, int group_rows = 16 * RT) {
  const int groups = (n + group_rows - 1) / group_rows;
  constexpr int UNROLL = (NORM ? 4 : 8) / (MT * RT > 4 ? 4 : (MT * RT > 1 ? 2 : 1));
  if (group_rows != 16 * RT) {
    if constexpr (MT == 1 && RT == 2 && !NORM && !SWIGLU) {
      if (tune.lines && splits == 1 && k % 64 == 0 && (k / 32) % 16 == 0 && UNROLL % 4 == 0)
        gemm_bf16_skinny_kernel<MT, RT, 8, UNROLL, NORM, SWIGLU, true, true><<<dim3(groups, 1), 8 * 64, 0, s>>>(out, mode, a, norm, w, bias, m, n, k, lda, ldc, split_sums, chain, group_rows);
      else
        gemm_bf16_skinny_kernel<MT, RT, 8, UNROLL, NORM, SWIGLU, true><<<dim3(groups, splits), 8 * 64, 0, s>>>(out, mode, a, norm, w, bias, m, n, k, lda, ldc, split_sums, chain, group_rows);
    }
  } else if (groups <= 2048) {
    if constexpr (MT == 1 && !NORM && UNROLL % 4 == 0) {
      if (tune.lines && splits == 1 && k % 64 == 0 && (k / 32) % 16 == 0) {   // every wave starts at an even step
        gemm_bf16_skinny_kernel<MT, RT, 8, UNROLL, NORM, SWIGLU, false, true><<<dim3(groups, 1), 8 * 64, 0, s>>>(out, mode, a, norm, w, bias, m, n, k, lda, ldc, split_sums, chain, group_rows);
        return;
      }
    }
    gemm_bf16_skinny_kernel<MT, RT, 8, UNROLL, NORM, SWIGLU><<<dim3(groups, splits), 8 * 64, 0, s>>>(out, mode, a, norm, w, bias, m, n, k, lda, ldc, split_sums, chain, group_rows);
  }
  else
    gemm_bf16_skinny_kernel<MT, RT, 4, UNROLL, NORM, SWIGLU><<<dim3(groups, splits), 4 * 64, 0, s>>>(out, mode, a, norm, w, bias, m, n, k, lda, ldc, split_sums, chain, group_rows);
  if (splits > 1) {
    const int64_t total = (int64_t)m * (SWIGLU ? n / 2 : n);
    const int blocks = (int)((total + 255) / 256 < 1024 ? (total + 255) / 256 : 1024);
    gemm_split_finish_kernel<SWIGLU><<<blocks, 256, 0, s>>>(out, mode, split_sums, bias, m, n, ldc, splits);
  }
}

LRS_API int lrs_compute_units();

// Weight rows per workgroup for a product of at most 16 rows and n output columns that is narrow
// enough for one row tile per workgroup (n < 16384, no gated epilogue).  16, unless that leaves the
// compute units unevenly loaded (n = 5120: 320 workgroups for 256 units, a quarter of them with twice
// the work): then the rows are dealt out evenly over a whole multiple of the units, between 16 and 32
// a workgroup (two tiles, the second partly empty).  Measured on MI355X at 8 rows: 6144 columns
// 16.7 -> 14.5 us, 5120 columns (K 5120 and 17408) 19.9 -> 15.9 and 56.0 -> 39.6 us.  0: 16 rows.
static int even_group_rows(int n) {
  const int units = lrs_compute_units(), tiles = (n + 15) / 16;
  if (units <= 0 || tiles <= units || tiles % units == 0) return 0;
  const int rows = (n + units * (tiles / units) - 1) / (units * (tiles / units));
  return rows <= 32 ? rows : 0;
}

// Device memory for the sums of K splits.  A caller brings its own (`workspace`, at least lrs_gemm_workspace_bytes()
// bytes: every runner has one, so that two runners on two streams of one GPU do not write over each other's sums
// between a product and the kernel that finishes it); a caller that brings none gets one that the process keeps, made
// on first use, and must then keep all its products on one stream.  Which of the two an entry point uses is a matter
// of that call alone: UseSpace notes it for the launches the call makes on its thread.
static float* g_split_sums = nullptr;
constexpr size_t SPLIT_SUMS_BYTES = 64u << 20;
static float* own_split_sums() {
  if (!g_split_sums && hipMalloc((void**)&g_split_sums, SPLIT_SUMS_BYTES) != hipSuccess) g_split_sums = nullptr;
  return g_split_sums;
}
struct SplitSpace {
  float* sums;
  size_t bytes;
};
static thread_local SplitSpace t_split_space = {nullptr, 0};
struct UseSpace {
  SplitSpace before;
  UseSpace(void* workspace, int64_t bytes) : before(t_split_space) {
    t_split_space = workspace ? SplitSpace{(float*)workspace, (size_t)bytes} : SplitSpace{own_split_sums(), SPLIT_SUMS_BYTES};
  }
  ~UseSpace() { t_split_space = before; }
};
static float* split_sums_buffer() { return t_split_space.sums; }
static size_t split_sums_bytes() { return t_split_space.sums ? t_split_space.bytes : 0; }
static bool workspace_ok(const void* workspace, int64_t bytes) {
  return workspace == nullptr || (bytes >= (int64_t)SPLIT_SUMS_BYTES && (uintptr_t)workspace % 16 == 0);
}
LRS_API int64_t lrs_gemm_workspace_bytes() { return (int64_t)SPLIT_SUMS_BYTES; }

// The kernel for 17..128 rows: which of its workgroup shapes and how many K splits.  Unless the caller's
// choices say otherwise: the shape and split that fill a whole multiple of the compute units best, then the
// fewest splits.
LRS_API int lrs_compute_units();

// What a launch of `groups` workgroups of `wv` tiles (16 weight rows each) costs: with every unit busy a compute unit
// gets some 35-45 GB/s from the L2s (a workgroup all alone on the chip 70-75), so the launch takes as long as the
// unit with the most to fetch: the tiles of its workgroups
// and, for each of them, the activations once (`blocks` blocks of 16 tokens: as many bytes as that many tiles).
static int mid_cost(int groups, int wv, int blocks, int units) { return (groups + units - 1) / units * (wv + blocks); }

static void choose_mid_shape(int n, int k, GemmTune tune, int& waves, int& splits, int blocks = 4) {
  const int want_waves = tune.waves, want_splits = tune.splits;
  const int units = lrs_compute_units() > 0 ? lrs_compute_units() : 256, slices = k / 256;
  auto tiles_of = [&](int wv) { return (n + 16 * wv - 1) / (16 * wv); };
  auto fill_of = [&](int groups) { return (double)groups / ((groups + units - 1) / units * units); };
  if (want_waves && want_splits) {
    waves = want_waves, splits = want_splits;
    return;
  }
  // Measured on MI355X (32..64 rows).  A matrix with enough rows to give every compute unit a workgroup is not
  // divided along K; of the workgroup shapes the one that costs least by mid_cost(): 24,576 rows are 256 workgroups
  // of six waves (one round of the chip; 39 us at 64 rows, eight waves 192 workgroups: a third slower); 34,816 rows
  // 436 of five (two rounds of 80 rows: 83 us at 64 rows; 363 of six 88, 544 of four 93, 272 of eight 100); 51,200
  // rows 400 of eight (110 us; 640 of five 121, 800 of four 124, 534 of six 131).  Eight waves only while that is
  // at most two rounds: walking many slices in many rounds they were slower than six (the LM head).  Ties go to
  // six, five, four, eight in that order.
  if ((!want_splits || want_splits == 1) && tiles_of(6) >= units && (!want_waves || want_waves == 4 || want_waves == 5 || want_waves == 6)) {
    splits = 1;
    waves = want_waves;
    if (!want_waves) {
      const int order[4] = {6, 5, 4, 8};
      int best = 0;
      for (int i = 0; i < 4; ++i) {
        const int wv = order[i], groups = tiles_of(wv);
        if (wv == 8 && groups > 2 * units) continue;
        const int cost = mid_cost(groups, wv, blocks, units);
        if (best == 0 || cost < best) best = cost, waves = wv;
      }
    }
    return;
  }
  // A narrower matrix: K is divided so that tiles x splits fills the units once (at least two slices a
  // workgroup, at most 8 splits).  Of the choices within 3 % of the fullest: the one with the most waves
  // among those whose workgroups still walk four slices or more (down: 8 waves x 8 splits, 6 slices each),
  // else the one with the fewest waves (o_proj: 4 waves x 4 splits); then the fewest splits.
  struct Choice { int waves, splits, len; double fill; };
  Choice all[32];
  int count = 0;
  double fullest = -1.0;
  const int shapes[4] = {4, 5, 6, 8};
  for (int wi = 0; wi < 4; ++wi) {
    const int wv = shapes[wi];
    if (want_waves && wv != want_waves) continue;
    for (int sp = 1; sp <= 8; ++sp) {
      if (want_splits && sp != want_splits) continue;
      if (sp > 1 && slices / sp < 2) continue;
      const int groups = tiles_of(wv) * sp;
      const double fill = groups <= units ? (double)groups / units : fill_of(groups) - 0.25;   // a second round costs more than its share
      all[count++] = Choice{wv, sp, slices / sp, fill};
      if (fill > fullest) fullest = fill;
    }
  }
  if (count == 0) {
    waves = want_waves ? want_waves : 4, splits = want_splits ? want_splits : 1;
    return;
  }
  const Choice* pick = nullptr;
  for (int i = 0; i < count; ++i) {
    const Choice& c = all[i];
    if (c.fill < fullest - 0.03) continue;
    if (!pick) { pick = &c; continue; }
    const bool c_long = c.len >= 4, p_long = pick->len >= 4;
    if (c_long != p_long) { if (c_long) pick = &c; continue; }
    if (c.waves != pick->waves) { if ((c.waves > pick->waves) == c_long) pick = &c; continue; }
    if (c.splits < pick->splits) pick = &c;
  }
  waves = pick->waves, splits = pick->splits;
}

// An even deal of the weight rows for a matrix that is not divided along K (see the kernel, EXTRA): workgroups of 4,
// 6 or 8 tiles of 16 rows, `groups` of them (a whole multiple of the compute units), the first `extras` with a tile
// more.  What a launch costs is taken to be what its busiest compute unit fetches, in tiles: the tiles of its
// workgroups and, for each of them, the activations once (mid_cost()), and one tile more where there are extras.  Taken
// where that is a tenth less than for the plain shape (measured on MI355X: 34,816 x 5,120 as 256 workgroups of 8 or 9
// tiles against 436 of 5: 66 / 68 / 71 us at 32 / 48 / 64 rows against 72 / 77 / 83; 51,200 x 5,120 as 768 of 4 or 5
// is no better than 400 of 8: 107 / 104 / 113 against 100 / 105 / 110, and is not taken).  Returns false if there is
// no such deal or it does not pay.
static bool choose_mid_even(int n, int blocks, GemmTune tune, int plain_waves, int& waves, int& groups, int& extras) {
  if (tune.even == 1 || blocks > 4) return false;
  const int units = lrs_compute_units() > 0 ? lrs_compute_units() : 256, tiles = (n + 15) / 16;
  const int plain_cost = mid_cost((tiles + plain_waves - 1) / plain_waves, plain_waves, blocks, units);
  int best = 0;
  for (int rounds = 1; rounds <= 8; ++rounds) {
    const int g = units * rounds, wv = tiles / g;
    if (wv != 4 && wv != 6 && wv != 8) continue;
    if (tune.waves && tune.waves != wv) continue;
    const int more = tiles - g * wv;                        // 0 .. g - 1 workgroups with a tile more
    const int cost = rounds * (wv + blocks) + (more + units - 1) / units;
    if (best == 0 || cost < best) best = cost, waves = wv, groups = g, extras = more;
  }
  if (best == 0) return false;
  return tune.even == 2 || 10 * best <= 9 * plain_cost;
}

// The shape the kernel for 17..128 rows takes for a matrix of n rows and k columns at 49..64 rows (for tests and
// reports; lrs_gemm_mid_deal() says it for any number of rows).
LRS_API int lrs_gemm_mid_shape(int n, int k, int tune, int* waves, int* splits) {
  LRS_REQUIRE(n > 0 && k > 0 && k % 256 == 0 && waves && splits, "gemm_mid_shape: needs n > 0 and K %% 256 == 0, got n=%d k=%d", n, k);
  LRS_REQUIRE(tune_ok(tune), "gemm_mid_shape: unknown choices %d", tune);
  choose_mid_shape(n, k, tune_of(tune), *waves, *splits);
  return 0;
}

// How the kernel for 17..128 rows deals out a matrix of n rows and k columns for a product of m rows: waves a
// workgroup, K splits, workgroups along n, and how many of those have a tile of 16 rows more than `waves` (0: the
// plain deal, every workgroup 16 * waves rows).
LRS_API int lrs_gemm_mid_deal(int m, int n, int k, int tune, int* waves, int* splits, int* groups, int* extras) {
  LRS_REQUIRE(m > 16 && m <= 128 && n > 0 && k > 0 && k % 256 == 0 && waves && splits && groups && extras,
              "gemm_mid_deal: needs 17..128 rows, n > 0 and K %% 256 == 0, got m=%d n=%d k=%d", m, n, k);
  LRS_REQUIRE(tune_ok(tune), "gemm_mid_deal: unknown choices %d", tune);
  const int blocks = m <= 32 ? 2 : m <= 48 ? 3 : m <= 64 ? 4 : m <= 96 ? 6 : 8;
  choose_mid_shape(n, k, tune_of(tune), *waves, *splits, blocks);
  *groups = (n + 16 * *waves - 1) / (16 * *waves);
  *extras = 0;
  int even_waves = 0, even_groups = 0, more = 0;
  if (*splits == 1 && choose_mid_even(n, blocks, tune_of(tune), *waves, even_waves, even_groups, more))
    *waves = even_waves, *groups = even_groups, *extras = more;
  return 0;
}

// keep_sums: the sums of the K splits (of the one split, if K is not divided) stay in the split buffer for
// the caller's own finishing kernel; returns their number, or 0 if the buffer cannot hold them.
template <int MT, bool SWIGLU>
static int launch_mid_mt(void* out, int mode, const bf16* a, const bf16* w, int m, int n, int k, int lda, int ldc, hipStream_t s, GemmTune tune, bool keep_sums, MidScale scale) {
  int waves = 4, splits = 1;
  choose_mid_shape(n, k, tune, waves, splits, MT);
  float* sums = splits > 1 || keep_sums ? split_sums_buffer() : nullptr;
  if ((splits > 1 || keep_sums) && (!sums || (size_t)splits * m * n * sizeof(float) > split_sums_bytes())) {
    if (keep_sums) return 0;
    splits = 1, sums = nullptr;
  }
  dim3 grid((n + 16 * waves - 1) / (16 * waves), splits);
  int extras = 0;
  bool even = false;
  if constexpr (MT <= 4) {
    int even_waves = 0, even_groups = 0;
    if (splits == 1 && choose_mid_even(n, MT, tune, waves, even_waves, even_groups, extras)) {
      even = true;
      waves = even_waves;
      grid = dim3(even_groups, 1);
    }
  }
  // dynamic LDS: two activation buffers of 8 x MT KB and 4 KB a wave; more than 64 KB has to be asked for once
#define MID_LAUNCH(WV, EXTRA)                                                                                       \
  do {                                                                                                              \
    constexpr int bytes = (2 * 8 * MT * 64 + WV * 256) * 16;                                                        \
    static bool asked = false;                                                                                      \
    if (!asked) {                                                                                                   \
      (void)hipFuncSetAttribute((const void*)gemm_bf16_mid_kernel<MT, WV, SWIGLU, EXTRA>, hipFuncAttributeMaxDynamicSharedMemorySize, bytes); \
      asked = true;                                                                                                 \
    }                                                                                                               \
    gemm_bf16_mid_kernel<MT, WV, SWIGLU, EXTRA><<<grid, WV * 64, bytes, s>>>(out, mode, a, w, m, n, k, lda, ldc, sums, scale, extras);    \
  } while (0)
  if constexpr (MT <= 4) {
    if (even && waves == 4) MID_LAUNCH(4, true);
    else if (even && waves == 6) MID_LAUNCH(6, true);
    else if (even) MID_LAUNCH(8, true);
  }
  if (even) {
  } else if (waves == 4) MID_LAUNCH(4, false);
  else if (waves == 5) MID_LAUNCH(5, false);
  else if (waves == 6) MID_LAUNCH(6, false);
  else MID_LAUNCH(8, false);
#undef MID_LAUNCH
  if (splits > 1 && !keep_sums) {
    const int64_t total = (int64_t)m * (SWIGLU ? n / 2 : n);
    const int blocks = (int)((total + 255) / 256 < 1024 ? (total + 255) / 256 : 1024);
    gemm_split_finish_kernel<SWIGLU><<<blocks, 256, 0, s>>>(out, mode, sums, nullptr, m, n, ldc, splits);
  }
  return splits;
}

template <bool SWIGLU>
static int launch_mid(void* out, int mode, const bf16* a, const bf16* w, int m, int n, int k, int lda, int ldc, hipStream_t s, GemmTune tune,
                      bool keep_sums = false, MidScale scale = MidScale{nullptr, 0, 0.f}) {
  if (m <= 32) return launch_mid_mt<2, SWIGLU>(out, mode, a, w, m, n, k, lda, ldc, s, tune, keep_sums, scale);
  if (m <= 48) return launch_mid_mt<3, SWIGLU>(out, mode, a, w, m, n, k, lda, ldc, s, tune, keep_sums, scale);
  if (m <= 64) return launch_mid_mt<4, SWIGLU>(out, mode, a, w, m, n, k, lda, ldc, s, tune, keep_sums, scale);
  if (m <= 96) return launch_mid_mt<6, SWIGLU>(out, mode, a, w, m, n, k, lda, ldc, s, tune, keep_sums, scale);
  return launch_mid_mt<8, SWIGLU>(out, mode, a, w, m, n, k, lda, ldc, s, tune, keep_sums, scale);
}

template <int MT, bool NORM, bool SWIGLU>
static void launch_skinny(void* out, int mode, const bf16* a, NormInput norm, const bf16* w, const bf16* bias,
                          int m, int n, int k, int lda, int ldc, hipStream_t s, GemmTune tune, NormChain chain = NormChain{}) {
  if (MT > 1 && !NORM) {
    // several token blocks: 64 weight rows per workgroup, so that an activation fragment read from
    // L2 serves four weight fragments, and K divided between workgroups until there are enough
    // of them to fill the chip
    const int groups = (n + 63) / 64;
    int splits = (383 + groups) / groups;
    if (splits > 8) splits = 8;
    while (splits > 1 && k / splits < 512) --splits;
    float* sums = splits > 1 ? split_sums_buffer() : nullptr;
    if (splits > 1 && (!sums || (size_t)splits * m * n * sizeof(float) > split_sums_bytes())) splits = 1;
    launch_skinny_rt<MT, (MT > 1 ? 4 : 1), NORM, SWIGLU>(out, mode, a, norm, w, bias, m, n, k, lda, ldc, s, tune, sums, splits);
    return;
  }
  if (MT == 1 && !NORM && n >= 16384) {  // measured: two row tiles and four waves stream wide matrices a little faster
    if (tune.lines && k % 64 == 0 && (k / 32) % 8 == 0)
      gemm_bf16_skinny_kernel<1, 2, 4, 4, NORM, SWIGLU, false, true><<<dim3((n + 31) / 32, 1), 4 * 64, 0, s>>>(out, mode, a, norm, w, bias, m, n, k, lda, ldc, nullptr, chain, 32);
    else
      gemm_bf16_skinny_kernel<1, 2, 4, 4, NORM, SWIGLU><<<dim3((n + 31) / 32, 1), 4 * 64, 0, s>>>(out, mode, a, norm, w, bias, m, n, k, lda, ldc, nullptr, chain, 32);
  }
  else if (MT == 1 && !NORM && !SWIGLU && even_group_rows(n) > 0) {
    if constexpr (MT == 1 && !NORM && !SWIGLU)
      launch_skinny_rt<1, 2, false, false>(out, mode, a, norm, w, bias, m, n, k, lda, ldc, s, tune, nullptr, 1, chain, even_group_rows(n));
  } else if (MT == 1 || n <= 32 * 128)
    launch_skinny_rt<MT, 1, NORM, SWIGLU>(out, mode, a, norm, w, bias, m, n, k, lda, ldc, s, tune, nullptr, 1, chain);
  else if (n < 64 * 256)
    launch_skinny_rt<MT, 2, NORM, SWIGLU>(out, mode, a, norm, w, bias, m, n, k, lda, ldc, s, tune);
  else
    launch_skinny_rt<MT, (MT > 1 ? 4 : 1), NORM, SWIGLU>(out, mode, a, norm, w, bias, m, n, k, lda, ldc, s, tune);
}

template <bool NORM, bool SWIGLU>
static void launch_skinny_m(void* out, int mode, const bf16* a, NormInput norm, const bf16* w, const bf16* bias,
                            int m, int n, int k, int lda, int ldc, hipStream_t s, GemmTune tune) {
  if (m <= 16) launch_skinny<1, NORM, SWIGLU>(out, mode, a, norm, w, bias, m, n, k, lda, ldc, s, tune);
  else if (m <= 32) launch_skinny<2, NORM, SWIGLU>(out, mode, a, norm, w, bias, m, n, k, lda, ldc, s, tune);
  else if (m <= 48) launch_skinny<3, NORM, SWIGLU>(out, mode, a, norm, w, bias, m, n, k, lda, ldc, s, tune);
  else launch_skinny<4, NORM, SWIGLU>(out, mode, a, norm, w, bias, m, n, k, lda, ldc, s, tune);
}

// Allocates the device memory the K-split products need, so that no later call has to (a call
// under graph capture must not allocate).  Safe to call more than once.
LRS_API int lrs_gemm_prepare() {
  if (!own_split_sums()) return lrs_fail("gemm_prepare: could not allocate %zu bytes for split sums", SPLIT_SUMS_BYTES);
  return 0;
}

// Most rows the few-rows kernel takes (and with it the fused RMSNorm input).  From 17 rows on the kernel for
// 17..128 rows (or, where a shape does not suit it, the vendor library) is faster, so callers send larger
// products there unless they are told otherwise.
LRS_API int lrs_gemm_skinny_capacity() { return 64; }

// How many partial sums of squares a product of n output columns leaves for the norm that follows it
// (the number of workgroups of the few-rows kernel for that width).
LRS_API int lrs_gemm_norm_chain_parts(int n) {
  if (n >= 16384) return (n + 31) / 32;
  const int rows = even_group_rows(n);
  return rows > 0 ? (n + rows - 1) / rows : (n + 15) / 16;
}

// The few-rows bf16 product (M <= 16) with an RMSNorm of the residual stream taken apart around it;
// see NormChain.  in_sumsq != null: `a` is bf16(h * g) and row r of the result is scaled by
// rsqrt(sum_p in_sumsq[p, r] / K + in_eps).  next_x != null (mode must add into the float32
// residual, no swiglu): also writes next_x [M, N] = bf16(out_new * next_weight) and next_sumsq
// [lrs_gemm_norm_chain_parts(N), M].
LRS_API int lrs_gemm_norm_chain(void* out, int mode, const void* a, const void* w, const void* bias, int m, int n, int k,
                                int lda, int ldc, int swiglu, const float* in_sumsq, int in_parts, float in_eps,
                                void* next_x, float* next_sumsq, const void* next_weight, int next_weight_dtype,
                                int tune, void* stream) {
  LRS_REQUIRE(m > 0 && m <= 16 && n > 0 && k > 0, "gemm_norm_chain: takes 1..16 rows and positive sizes, got m=%d n=%d k=%d", m, n, k);
  LRS_REQUIRE(tune_ok(tune), "gemm_norm_chain: unknown choices %d", tune);
  LRS_REQUIRE(lda >= k && ldc >= (swiglu ? n / 2 : n), "gemm_norm_chain: strides lda=%d ldc=%d too small for k=%d n=%d", lda, ldc, k, n);
  LRS_REQUIRE(mode >= OUT_STORE && mode <= OUT_ADD_F32, "gemm_norm_chain: unknown output mode %d", mode);
  LRS_REQUIRE(k % 8 == 0 && lda % 8 == 0 && ((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0),
              "gemm_norm_chain: needs 16-byte aligned rows (k=%d lda=%d)", k, lda);
  LRS_REQUIRE(!swiglu || (n % 16 == 0 && bias == nullptr && mode == OUT_STORE), "gemm_norm_chain: swiglu needs n %% 16 == 0, no bias and a stored output (n=%d)", n);
  LRS_REQUIRE(in_sumsq == nullptr || (in_parts > 0 && in_eps > 0.f), "gemm_norm_chain: in_parts and in_eps must be positive");
  LRS_REQUIRE(next_x == nullptr || (mode == OUT_ADD_F32 && !swiglu && next_sumsq && next_weight),
              "gemm_norm_chain: the output for the next norm needs a product that adds into the float32 residual stream");
  const NormChain chain{in_sumsq, in_parts, in_eps, (bf16*)next_x, next_sumsq, next_weight, next_weight_dtype == LRS_F32};
  const NormInput none{nullptr, nullptr, nullptr, 0, 0.f};
  hipStream_t s = (hipStream_t)stream;
  if (swiglu) launch_skinny<1, false, true>(out, mode, (const bf16*)a, none, (const bf16*)w, nullptr, m, n, k, lda, ldc, s, tune_of(tune), chain);
  else launch_skinny<1, false, false>(out, mode, (const bf16*)a, none, (const bf16*)w, (const bf16*)bias, m, n, k, lda, ldc, s, tune_of(tune), chain);
  return lrs_check_launch("gemm_norm_chain");
}

static bool mid_shape_ok(const void* a, const void* w, int m, int n, int k, int lda) {
  return m > 16 && m <= 128 && n > 0 && k > 0 && k % 256 == 0 && n % 16 == 0 && lda >= k && lda % 8 == 0 && ((uintptr_t)a % 16 == 0) &&
         ((uintptr_t)w % 16 == 0);
}

// The product of 17..128 rows whose input is a norm that the kernel before began: a = bf16(h * norm weight)
// [M, K], in_sumsq [in_parts, M] partial sums of h^2; row r of the result is multiplied by
// rsqrt(sum_p in_sumsq[p, r] / K + in_eps).  swiglu as in lrs_gemm.
LRS_API int lrs_gemm_mid_scaled(void* out, int mode, const void* a, const void* w, int m, int n, int k, int lda, int ldc,
                                int swiglu, const float* in_sumsq, int in_parts, float in_eps, int tune, void* workspace,
                                int64_t workspace_bytes, void* stream) {
  LRS_REQUIRE(tune_ok(tune), "gemm_mid_scaled: unknown choices %d", tune);
  LRS_REQUIRE(workspace_ok(workspace, workspace_bytes), "gemm_mid_scaled: a workspace must be 16-byte aligned and hold lrs_gemm_workspace_bytes() bytes");
  const UseSpace space(workspace, workspace_bytes);
  LRS_REQUIRE(mid_shape_ok(a, w, m, n, k, lda), "gemm_mid_scaled: takes 17..128 rows, K %% 256 == 0, N %% 16 == 0, 16-byte aligned rows (m=%d n=%d k=%d lda=%d)", m, n, k, lda);
  LRS_REQUIRE(mode >= OUT_STORE && mode <= OUT_ADD_F32 && ldc >= (swiglu ? n / 2 : n) && ldc % 4 == 0 && (uintptr_t)out % 16 == 0,
              "gemm_mid_scaled: unknown output mode %d, or an output that is not 16-byte aligned (ldc=%d)", mode, ldc);
  LRS_REQUIRE(!swiglu || mode == OUT_STORE, "gemm_mid_scaled: swiglu needs a stored output");
  LRS_REQUIRE(in_sumsq != nullptr && in_parts > 0 && in_eps > 0.f, "gemm_mid_scaled: needs the partial sums of squares, their number and eps");
  const MidScale scale{in_sumsq, in_parts, in_eps};
  if (swiglu) launch_mid<true>(out, mode, (const bf16*)a, (const bf16*)w, m, n, k, lda, ldc, (hipStream_t)stream, tune_of(tune), false, scale);
  else launch_mid<false>(out, mode, (const bf16*)a, (const bf16*)w, m, n, k, lda, ldc, (hipStream_t)stream, tune_of(tune), false, scale);
  return lrs_check_launch("gemm_mid_scaled");
}

// Defined beside the norm kernels: x [rows, hidden] += the sum over `splits` of sums[split, rows, hidden]; next_x =
// bf16(x * weight); next_sumsq [lrs_norm_begin_parts(hidden), rows] = partial sums of x^2.
extern "C" int lrs_split_add_norm_begin(float* x, const float* sums, int splits, const void* weight, int w_dtype, void* next_x,
                                        float* next_sumsq, int n_rows, int hidden, void* stream);

// A product of 17..128 rows that adds into the float32 residual stream and begins the RMSNorm that follows:
// residual [M, N] += a [M, K] w[N, K]^T; next_x [M, N] = bf16(residual * norm_weight); next_sumsq
// [lrs_norm_begin_parts(N), M] = partial sums of residual^2, for the product that finishes the norm
// (lrs_gemm_mid_scaled) or for scale_rows.  The kernel that adds the K splits' sums spreads over rows x 1,024
// columns, where a whole norm would have one workgroup a row.
LRS_API int lrs_gemm_mid_add_norm_begin(float* residual, const void* a, const void* w, const void* norm_weight, int norm_weight_dtype,
                                        void* next_x, float* next_sumsq, int m, int n, int k, int lda, int tune, void* workspace,
                                        int64_t workspace_bytes, void* stream) {
  LRS_REQUIRE(tune_ok(tune), "gemm_mid_add_norm_begin: unknown choices %d", tune);
  LRS_REQUIRE(workspace_ok(workspace, workspace_bytes), "gemm_mid_add_norm_begin: a workspace must be 16-byte aligned and hold lrs_gemm_workspace_bytes() bytes");
  const UseSpace space(workspace, workspace_bytes);
  LRS_REQUIRE(mid_shape_ok(a, w, m, n, k, lda) && ((uintptr_t)residual % 16 == 0), "gemm_mid_add_norm_begin: takes 17..128 rows, K %% 256 == 0, N %% 16 == 0, 16-byte aligned rows (m=%d n=%d k=%d lda=%d)", m, n, k, lda);
  LRS_REQUIRE(next_x && next_sumsq && norm_weight, "gemm_mid_add_norm_begin: needs the norm weight and the two outputs for the next norm");
  const int splits = launch_mid<false>(nullptr, OUT_STORE, (const bf16*)a, (const bf16*)w, m, n, k, lda, n, (hipStream_t)stream, tune_of(tune), true);
  LRS_REQUIRE(splits > 0, "gemm_mid_add_norm_begin: the buffer for the sums of the K splits cannot hold %d x %d values", m, n);
  if (int rc = lrs_check_launch("gemm_mid_add_norm_begin")) return rc;
  return lrs_split_add_norm_begin(residual, split_sums_buffer(), splits, norm_weight, norm_weight_dtype, next_x, next_sumsq, m, n, stream);
}

// Defined beside qk_prep: see there.
extern "C" int lrs_qk_prep_from_sums(void* qkv, int dtype, int tokens, int row_stride, int nq, int nkv, int d, const void* q_weight,
                                     const void* k_weight, int w_dtype, float eps, const float* cosv, const float* sinv,
                                     int rot_half, void* k_pages, void* v_pages, const int* slots, int page_size,
                                     const float* sums, int splits, void* stream);

// The q/k/v product of 17..128 rows (its input possibly a norm begun before it: in_sumsq as in lrs_gemm_mid_scaled, or
// null) and what follows it: per-head norm and rotation of q and k, q into qkv [M, row_stride], k and v into the
// pages.  The kernel that prepares the heads adds up the K splits' sums itself.
LRS_API int lrs_gemm_mid_qk_prep(void* qkv, int row_stride, const void* a, const void* w, int m, int k, int lda,
                                 const float* in_sumsq, int in_parts, float in_eps, int nq, int nkv, int d,
                                 const void* q_weight, const void* k_weight, int w_dtype, float eps, const float* cosv,
                                 const float* sinv, int rot_half, void* k_pages, void* v_pages, const int* slots,
                                 int page_size, int tune, void* workspace, int64_t workspace_bytes, void* stream) {
  const int n = (nq + 2 * nkv) * d;
  LRS_REQUIRE(tune_ok(tune), "gemm_mid_qk_prep: unknown choices %d", tune);
  LRS_REQUIRE(workspace_ok(workspace, workspace_bytes), "gemm_mid_qk_prep: a workspace must be 16-byte aligned and hold lrs_gemm_workspace_bytes() bytes");
  const UseSpace space(workspace, workspace_bytes);
  LRS_REQUIRE(mid_shape_ok(a, w, m, n, k, lda), "gemm_mid_qk_prep: takes 17..128 rows, K %% 256 == 0, N %% 16 == 0, 16-byte aligned rows (m=%d n=%d k=%d lda=%d)", m, n, k, lda);
  LRS_REQUIRE(in_sumsq == nullptr || (in_parts > 0 && in_eps > 0.f), "gemm_mid_qk_prep: in_parts and in_eps must be positive");
  const MidScale scale{in_sumsq, in_parts, in_eps};
  const int splits = launch_mid<false>(nullptr, OUT_STORE, (const bf16*)a, (const bf16*)w, m, n, k, lda, n, (hipStream_t)stream, tune_of(tune), true, scale);
  LRS_REQUIRE(splits > 0, "gemm_mid_qk_prep: the buffer for the sums of the K splits cannot hold %d x %d values", m, n);
  if (int rc = lrs_check_launch("gemm_mid_qk_prep")) return rc;
  return lrs_qk_prep_from_sums(qkv, LRS_BF16, m, row_stride, nq, nkv, d, q_weight, k_weight, w_dtype, eps, cosv, sinv, rot_half, k_pages,
                               v_pages, slots, page_size, split_sums_buffer(), splits, stream);
}

// Which tile width the kernel for many rows with slices of whole lines would take for this product, or 0 if
// it does not take it: K a multiple of 64 and a tile of 256 x 128 for every compute unit; then the width
// (256, 192 or 128 weight rows) whose launch takes the fewest rounds of the chip times its width, the wider
// of two that tie (less traffic per product).
LRS_API int lrs_gemm_lines_width(int m, int n, int k) {
  const int units = lrs_compute_units() > 0 ? lrs_compute_units() : 256;
  const int big_m = (m + 255) / 256;
  if (m <= 0 || n <= 0 || k <= 0 || k % 64 != 0 || big_m * ((n + 127) / 128) < units) return 0;
  int width = 0;
  int64_t best = 0;
  for (int candidate : {256, 192, 128}) {
    const int across = (n + candidate - 1) / candidate;
    const int64_t cost = (int64_t)((big_m * across + units - 1) / units) * candidate;
    if (!width || cost < best) width = candidate, best = cost;
  }
  return width;
}

// Into how many parts that kernel divides K for a product with too few tiles of 256 x 128 to go round the
// compute units, or 0 if it does not take the product that way (then lrs_gemm_lines_width says whether it takes
// it whole): the number of parts, from 1 (just the tiles, if they fill half the units) to 8, that fills the
// units best in one round, every part with 8 slices of 64 or more, and the parts' sums within the split buffer.
LRS_API int lrs_gemm_lines_splits(int m, int n, int k) {
  const int units = lrs_compute_units() > 0 ? lrs_compute_units() : 256;
  if (m <= 128 || n <= 0 || k <= 0 || k % 64 != 0) return 0;
  const int tiles = ((m + 255) / 256) * ((n + 127) / 128), steps = k / 64;
  if (tiles >= units) return 0;
  int splits = 0;
  for (int parts = 1; parts <= 8 && tiles * parts <= units; ++parts) {
    const int each = (steps + parts - 1) / parts;
    if (parts > 1 && (each < 8 || (parts - 1) * each >= steps || (size_t)parts * m * n * sizeof(float) > SPLIT_SUMS_BYTES)) continue;
    splits = parts;
  }
  return splits && 2 * tiles * splits >= units ? splits : 0;
}

// Whether that divided form is the faster way for a product that could also go to the vendor library.  Measured
// on MI355X at 256..1024 rows with the layer sizes of the 8B and 14B models, against the library's first choice:
// products with a long K (the feed-forward's second: K three times N or more) take 0.4 to 0.9 of the library's
// time at every such row count (14B at 512 rows: 102 against 171 us; 8B: 61 against 82); square and wide ones only
// up to 256 rows, when every part still has 12 slices (14B q/k/v 41 against 54 us, o_proj 35 against 49; with 8
// slices a part, 8B o_proj, 31 against 23).  Elsewhere the library is as fast or faster.
LRS_API int lrs_gemm_lines_split_pays(int m, int n, int k) {
  const int splits = lrs_gemm_lines_splits(m, n, k);
  if (splits < 1 || n % 4 != 0) return 0;
  if (k >= 2 * n) return 1;
  return m <= 256 && splits >= 2 && (k / 64 + splits - 1) / splits >= 12;
}

// Defined beside the norm kernels: x += the sum of the splits' sums, then out = RMSNorm(x), one pass over the rows.
extern "C" int lrs_split_add_rmsnorm(void* out, int out_dtype, float* x, const float* sums, int splits, const void* weight,
                                     int w_dtype, int n_rows, int hidden, float eps, void* stream);

// A product of more than 128 bf16 rows that adds into the float32 residual stream, and the RMSNorm that follows, as two
// kernels: residual [M, N] += a [M, K] w[N, K]^T; normed [M, N] = RMSNorm(residual) with norm_weight and eps.  The
// product is the many-rows kernel with slices of whole lines, its K divided between workgroups as lrs_gemm_lines_splits
// says (which must take the shape); its sums stay in the workspace, and the kernel that adds them up also adds the
// residual, writes it back and normalises the row: no kernel of its own for the add, none for the norm.
LRS_API int lrs_gemm_lines_add_rmsnorm(float* residual, const void* a, const void* w, int m, int n, int k, int lda,
                                       const void* norm_weight, int norm_weight_dtype, float eps, void* normed, int normed_dtype,
                                       void* workspace, int64_t workspace_bytes, void* stream) {
  LRS_REQUIRE(m > 128 && n > 0 && k > 0 && lda >= k, "gemm_lines_add_rmsnorm: takes more than 128 rows and positive sizes, got m=%d n=%d k=%d lda=%d", m, n, k, lda);
  LRS_REQUIRE(workspace_ok(workspace, workspace_bytes), "gemm_lines_add_rmsnorm: a workspace must be 16-byte aligned and hold lrs_gemm_workspace_bytes() bytes");
  const UseSpace space(workspace, workspace_bytes);
  const int splits = lrs_gemm_lines_splits(m, n, k);
  LRS_REQUIRE(splits >= 1, "gemm_lines_add_rmsnorm: the divided product does not take m=%d n=%d k=%d (see lrs_gemm_lines_splits)", m, n, k);
  LRS_REQUIRE(k % WIDE_BK == 0 && lda % 8 == 0 && n % 4 == 0 && ((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0) && ((uintptr_t)residual % 16 == 0) &&
                  (int64_t)m * lda < (1ll << 31) && (int64_t)n * k < (1ll << 31),
              "gemm_lines_add_rmsnorm: needs 16-byte aligned rows and sizes below 2^31 elements (m=%d n=%d k=%d lda=%d)", m, n, k, lda);
  float* sums = split_sums_buffer();
  LRS_REQUIRE(sums != nullptr && (size_t)splits * m * n * sizeof(float) <= split_sums_bytes(), "gemm_lines_add_rmsnorm: no room for the sums of %d K splits of %d x %d", splits, m, n);
  LRS_REQUIRE(residual && normed && norm_weight && eps > 0.f, "gemm_lines_add_rmsnorm: needs the residual stream, the norm's weight, a positive eps and the output");
  const int big_m = (m + 255) / 256, tiles_w = (n + 127) / 128;
  gemm_bf16_lines_kernel<128, false, OUT_STORE_F32><<<big_m * tiles_w * splits, 512, 0, (hipStream_t)stream>>>(
      sums, (const bf16*)a, (const bf16*)w, m, n, k, lda, n, big_m, tiles_w, splits);
  if (int rc = lrs_check_launch("gemm_lines_add_rmsnorm")) return rc;
  return lrs_split_add_rmsnorm(normed, normed_dtype, residual, sums, splits, norm_weight, norm_weight_dtype, m, n, eps, stream);
}

// out [M, N] (row stride ldc) = a [M, K] (row stride lda) times w[N, K]^T.
//   norm_weight != null: `a` is the float32 residual stream [*, K]; its rows (picked through
//     `rows` if given) are RMS-normalised with norm_weight and eps on the way in.  bf16 weights,
//     at most 64 rows.
//   swiglu != 0: w holds gate and up rows interleaved in groups of 8 and out is [M, N/2] with
//     silu(gate) * up.  bf16, K % 8 == 0, no bias.
//   workspace: device memory of lrs_gemm_workspace_bytes() bytes for the sums of K splits, the caller's own; null: the
//     one the process keeps, which every caller that brings none shares (products on one stream only then).
LRS_API int lrs_gemm(void* out, int mode, const void* a, const void* w, const void* bias, int dtype,
                     int m, int n, int k, int lda, int ldc, const int* rows, const void* norm_weight,
                     int norm_weight_dtype, float eps, int swiglu, int tune_word, void* workspace, int64_t workspace_bytes,
                     void* stream) {
  LRS_REQUIRE(m > 0 && n > 0 && k > 0, "gemm: sizes m=%d n=%d k=%d must be positive", m, n, k);
  LRS_REQUIRE(workspace_ok(workspace, workspace_bytes), "gemm: a workspace must be 16-byte aligned and hold lrs_gemm_workspace_bytes() bytes");
  const UseSpace space(workspace, workspace_bytes);
  LRS_REQUIRE(tune_ok(tune_word), "gemm: unknown choices %d", tune_word);
  const GemmTune tune = tune_of(tune_word);
  LRS_REQUIRE(lda >= k && ldc >= (swiglu ? n / 2 : n), "gemm: strides lda=%d ldc=%d too small for k=%d n=%d", lda, ldc, k, n);
  LRS_REQUIRE(mode >= OUT_STORE && mode <= OUT_ADD_F32, "gemm: unknown output mode %d", mode);
  hipStream_t s = (hipStream_t)stream;
  const bool normed = norm_weight != nullptr;
  const bool aligned = k % 8 == 0 && lda % 8 == 0 && ((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0);
  if (normed || swiglu) {
    LRS_REQUIRE(dtype == LRS_BF16 && aligned, "gemm: fused norm / swiglu need bf16 weights and 16-byte aligned rows (k=%d lda=%d)", k, lda);
    LRS_REQUIRE(!swiglu || (n % 16 == 0 && bias == nullptr && mode == OUT_STORE), "gemm: swiglu needs n %% 16 == 0, no bias and a stored output (n=%d)", n);
    LRS_REQUIRE(!normed || m <= 64, "gemm: the fused norm input takes at most 64 rows, got %d", m);
    LRS_REQUIRE(!normed || eps > 0.f, "gemm: eps must be positive");
  }
  LRS_REQUIRE(normed || rows == nullptr, "gemm: a row gather needs the fused norm input");
  if (dtype == LRS_F32 && m <= 16 && k % 64 == 0 && lda % 4 == 0 && ((uintptr_t)a % 16) == 0 && ((uintptr_t)w % 16) == 0) {
    // a decode step in float32: the same sums as the tiled kernel below makes, from a kernel made for few rows
    if (m <= 4) gemm_f32_few_rows_kernel<4><<<(n + 63) / 64, 256, 0, s>>>(out, mode, (const float*)a, (const float*)w, (const float*)bias, m, n, k, lda, ldc);
    else if (m <= 8) gemm_f32_few_rows_kernel<8><<<(n + 31) / 32, 256, 0, s>>>(out, mode, (const float*)a, (const float*)w, (const float*)bias, m, n, k, lda, ldc);
    else gemm_f32_few_rows_kernel<16><<<(n + 15) / 16, 256, 0, s>>>(out, mode, (const float*)a, (const float*)w, (const float*)bias, m, n, k, lda, ldc);
  } else if (dtype == LRS_F32) {
    dim3 grid((n + 63) / 64, (m + 63) / 64);
    gemm_tiled_kernel<float><<<grid, 256, 0, s>>>(out, mode, (const float*)a, (const float*)w,
                                                  (const float*)bias, m, n, k, lda, ldc);
  } else if (dtype == LRS_BF16) {
    const bool mid = aligned && m > 16 && m <= 128 && !normed && !bias && tune.mid && k % 256 == 0 && n % 16 == 0 && ldc % 4 == 0 &&
                     (uintptr_t)out % 16 == 0;
    if (aligned && (m <= 64 || mid)) {
      const bf16 *wp = (const bf16*)w, *bp = (const bf16*)bias;
      const NormInput norm{(const float*)a, rows, norm_weight, norm_weight_dtype == LRS_F32, eps};
      const bf16* ap = normed ? nullptr : (const bf16*)a;
      if (mid) {
        if (swiglu) launch_mid<true>(out, mode, ap, wp, m, n, k, lda, ldc, s, tune);
        else launch_mid<false>(out, mode, ap, wp, m, n, k, lda, ldc, s, tune);
      } else if (normed && swiglu) launch_skinny_m<true, true>(out, mode, ap, norm, wp, bp, m, n, k, lda, ldc, s, tune);
      else if (normed) launch_skinny_m<true, false>(out, mode, ap, norm, wp, bp, m, n, k, lda, ldc, s, tune);
      else if (swiglu) launch_skinny_m<false, true>(out, mode, ap, norm, wp, bp, m, n, k, lda, ldc, s, tune);
      else launch_skinny_m<false, false>(out, mode, ap, norm, wp, bp, m, n, k, lda, ldc, s, tune);
    } else if (aligned && k % WIDE_BK == 0 && n % 4 == 0 && ldc % 4 == 0 && (uintptr_t)out % 16 == 0 && !bias &&
               (int64_t)m * lda < (1ll << 31) && (int64_t)n * k < (1ll << 31)) {
      const int big_m = (m + 255) / 256, splits = lrs_gemm_lines_splits(m, n, k);
      const int width = splits ? 128 : lrs_gemm_lines_width(m, n, k), tiles_w = width ? (n + width - 1) / width : 0;
#define LINES(BN, SW, MODE, OUT, LDC, SPLITS) \
  gemm_bf16_lines_kernel<BN, SW, MODE><<<big_m * tiles_w * SPLITS, 512, 0, s>>>(OUT, (const bf16*)a, (const bf16*)w, m, n, k, lda, LDC, big_m, tiles_w, SPLITS)
      if (splits > 1) {
        // K divided between workgroups: their sums go to the split buffer, and the kernel that adds them up
        // writes the output with the epilogue that was asked for
        float* sums = split_sums_buffer();
        LRS_REQUIRE(sums != nullptr, "gemm: no memory for the sums of %d K splits", splits);
        LINES(128, false, OUT_STORE_F32, sums, n, splits);
        const int64_t total = (int64_t)m * (swiglu ? n / 2 : n);
        const int blocks = (int)((total + 1023) / 1024 < 2048 ? (total + 1023) / 1024 : 2048);
        if (swiglu) gemm_split_finish_kernel<true><<<blocks, 256, 0, s>>>(out, mode, sums, nullptr, m, n, ldc, splits);
        else gemm_split_finish_kernel<false><<<blocks, 256, 0, s>>>(out, mode, sums, nullptr, m, n, ldc, splits);
      } else if (width) {
#define LINES_OF(BN)                                                           \
        if (swiglu) LINES(BN, true, OUT_STORE, out, ldc, 1);                    \
        else if (mode == OUT_STORE) LINES(BN, false, OUT_STORE, out, ldc, 1);   \
        else if (mode == OUT_STORE_F32) LINES(BN, false, OUT_STORE_F32, out, ldc, 1); \
        else LINES(BN, false, OUT_ADD_F32, out, ldc, 1)
        if (width == 256) { LINES_OF(256); }
        else if (width == 192) { LINES_OF(192); }
        else { LINES_OF(128); }
#undef LINES_OF
#undef LINES
      } else {
        const int tiles_m = (m + 127) / 128, tiles_n = (n + 255) / 256;
#define WIDE(SW, MODE) gemm_bf16_wide_kernel<SW, MODE><<<tiles_m * tiles_n, 256, 0, s>>>(out, (const bf16*)a, (const bf16*)w, m, n, k, lda, ldc, tiles_m, tiles_n)
        if (swiglu) WIDE(true, OUT_STORE);
        else if (mode == OUT_STORE) WIDE(false, OUT_STORE);
        else if (mode == OUT_STORE_F32) WIDE(false, OUT_STORE_F32);
        else WIDE(false, OUT_ADD_F32);
#undef WIDE
      }
    } else if (aligned) {
      dim3 grid((n + 127) / 128, (m + 127) / 128);
      if (swiglu)
        gemm_bf16_mfma_kernel<true><<<grid, 256, 0, s>>>(out, mode, (const bf16*)a, (const bf16*)w, (const bf16*)bias, m, n, k, lda, ldc);
      else
        gemm_bf16_mfma_kernel<false><<<grid, 256, 0, s>>>(out, mode, (const bf16*)a, (const bf16*)w, (const bf16*)bias, m, n, k, lda, ldc);
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
