// True float32 product for many rows on the matrix cores:  C[M, N] = A[M, K] W[N, K]^T (+ bias[N]).
// v_mfma_f32_32x32x2_f32 takes float32 inputs and adds float32 products into float32 sums: no reduced-precision
// mode exists for it.  It has twice the rate of the vector units' fused multiply-add, which the tiled kernel in
// gemm_f32.hip uses (and nearly exhausts: 73 of 79 TFLOP/s without packed instructions).
//
//  * A block makes 256 x 128 results with 8 multiplying waves (4 x 2, each 64 x 64: four 32 x 32 tiles, 64
//    accumulators a lane) and has two more waves that only load; up to 128 rows of A, 128 x 128 results with 4.
//  * K may be split over blocks (partial sums [split][M][N] that the consuming kernel adds in split order), for
//    products whose tiles alone would leave most of the chip idle.
//  * A stage is 32 columns of K: 256 rows of A and 128 rows of W, 128 bytes each, loaded straight from memory into
//    LDS (global_load_lds_dwordx4: a wave's instruction takes 8 rows), piece p of row r at place p ^ ((r >> 1) & 7):
//    a fragment read takes 16 rows at a time, rows two apart lie on the same banks, and turned by r / 2 the 16 rows'
//    pieces fall on all 64 banks once.  Three stages lie in LDS; one barrier a stage.
//  * Loading and multiplying are different waves' work because of the compiler: it makes a wave that has sent a load
//    into LDS wait for ALL its loads before its next LDS read, which would end the overlap of a stage's loads with the
//    stage before.  A wave that only reads LDS, or only loads into it, gets no such wait.
//  * A lane (row l % 32, half l / 32) reads 16 bytes of its row: the columns 8 c + 4 half + 0..3 of chunk c, which
//    feed four products as the k of its half.  Which two columns of K meet in one product does not matter to the
//    sum, only that A and W pair them alike.
//  * Every element of C is the sum over k in one fixed order, whatever M, the row's place in the batch or its tile.
// Takes K a multiple of 32 with at least 2 stages a split and 16-byte aligned A, W and C; any M and N.
#include "common.h"

typedef float f32x16 __attribute__((ext_vector_type(16)));

#define FM_COLS 128                                        // rows of W (columns of C) a block
#define FM_STAGE 32                                        // columns of K a stage: rows of 128 bytes
#define FM_RING 3

// The loads of one of the two loading waves: COUNT instructions a stage (8 rows each) from `source`, whose rows
// first .. first + 8 COUNT - 1 (clamped to `last`: rows past the end repeat it, their results are not stored) go to
// `to` in every stage's place.
template <int COUNT, int SLOT>
__device__ __forceinline__ void fm_load_loop(const float* source, int first, int last, int K, int stages,
                                             unsigned char* lds, uint32_t to, int lane) {
  const int rl = lane >> 3;                                // lane = (row lane / 8, place lane % 8), which gets piece place ^ (row / 2 % 8)
  const char* from[COUNT];
#pragma unroll
  for (int i = 0; i < COUNT; ++i)
    from[i] = reinterpret_cast<const char*>(source + (size_t)min(first + 8 * i + rl, last) * K) +
              (((lane & 7) ^ ((4 * i + (rl >> 1)) & 7)) << 4);
  auto load = [&](int stage) __attribute__((always_inline)) {
    unsigned char* slot = lds + (stage % FM_RING) * SLOT + to;
    const size_t at = (size_t)stage * (FM_STAGE * 4);
#pragma unroll
    for (int i = 0; i < COUNT; ++i)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(from[i] + at),
                                       (__attribute__((address_space(3))) void*)(slot + i * 1024), 16, 0, 0);
  };
#pragma unroll
  for (int s = 0; s < FM_RING - 1; ++s)
    if (s < stages) load(s);
  for (int stage = 0; stage < stages; ++stage) {
    // all but the newest stage's loads have landed (near the end: all); after the barrier everybody is done with the
    // stage before, whose place the next loads take
    if (stage + FM_RING - 2 < stages) asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((FM_RING - 2) * COUNT) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    if (stage + FM_RING - 1 < stages) load(stage + FM_RING - 1);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// ROWS: rows of A a block, 256 or 128; ROWS / 32 waves multiply and two more load.  gridDim.z splits of K, each of
// `stages` stages; split z writes C + z M N (bias: one split only).
template <int ROWS>
__global__ void __launch_bounds__((ROWS / 32 + 2) * QIL_WAVE, 1)
gemm_f32_mfma_kernel(const float* __restrict__ A, const float* __restrict__ W, const float* __restrict__ bias,
                     float* __restrict__ C, int M, int N, int K, int stages) {
  constexpr int WAVES = ROWS / 32, SLOT = (ROWS + FM_COLS) * 128;   // bytes of a stage: A's rows, then W's
  extern __shared__ __align__(1024) unsigned char lds[];
  const int lane = threadIdx.x & (QIL_WAVE - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / QIL_WAVE);
  const int m0 = blockIdx.x * ROWS, n0 = blockIdx.y * FM_COLS;
  const size_t k_begin = (size_t)blockIdx.z * stages * FM_STAGE;
  C += (size_t)blockIdx.z * M * N;

  if (wave == WAVES) {                                     // ---- the wave that loads A
    fm_load_loop<ROWS / 8, SLOT>(A + k_begin, m0, M - 1, K, stages, lds, 0, lane);
    return;
  }
  if (wave == WAVES + 1) {                                 // ---- the wave that loads W
    fm_load_loop<FM_COLS / 8, SLOT>(W + k_begin, n0, N - 1, K, stages, lds, ROWS * 128, lane);
    return;
  }

  // ---- the waves that multiply: rows 64 (wave / 2) .. of A's tile, rows 64 (wave % 2) .. of W's
  const int l32 = lane & 31, half = lane >> 5;
  const int wm = wave >> 1, wn = wave & 1;
  uint32_t read_at[4];                                     // chunk c of this lane's row: piece 2 c + half, at place piece ^ (row / 2 % 8)
#pragma unroll
  for (int c = 0; c < 4; ++c) read_at[c] = l32 * 128 + (((2 * c + half) ^ ((l32 >> 1) & 7)) << 4);
  const uint32_t a_rows = (wm * 64) * 128, w_rows = ROWS * 128 + (wn * 64) * 128;

  f32x16 acc[2][2];                                        // [tile of W's rows][tile of A's rows]
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  for (int stage = 0; stage < stages; ++stage) {
    asm volatile("s_barrier" ::: "memory");                // the stage has landed (the loading waves waited for it)
    const unsigned char* slot = lds + (stage % FM_RING) * SLOT;
    float4 af[2][2], wf[2][2];                             // [chunk in flight][tile]
    auto fragments = [&](int c) __attribute__((always_inline)) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        af[c & 1][t] = *reinterpret_cast<const float4*>(slot + a_rows + t * 4096 + read_at[c]);
        wf[c & 1][t] = *reinterpret_cast<const float4*>(slot + w_rows + t * 4096 + read_at[c]);
      }
    };
    fragments(0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      if (c + 1 < 4) fragments(c + 1);                     // the next chunk's reads run under these products
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int tw = 0; tw < 2; ++tw)
#pragma unroll
          for (int ta = 0; ta < 2; ++ta) {
            const float a = j == 0 ? af[c & 1][ta].x : j == 1 ? af[c & 1][ta].y : j == 2 ? af[c & 1][ta].z : af[c & 1][ta].w;
            const float w = j == 0 ? wf[c & 1][tw].x : j == 1 ? wf[c & 1][tw].y : j == 2 ? wf[c & 1][tw].z : wf[c & 1][tw].w;
            acc[tw][ta] = __builtin_amdgcn_mfma_f32_32x32x2f32(w, a, acc[tw][ta], 0, 0, 0);
          }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // acc[tw][ta][e]: row m0 + 64 wm + 32 ta + l32, column n0 + 64 wn + 32 tw + 8 (e / 4) + 4 half + e % 4
  const bool whole = N % 4 == 0;                            // four columns at a time where rows of C stay 16-byte aligned
#pragma unroll
  for (int ta = 0; ta < 2; ++ta) {
    const int m = m0 + wm * 64 + ta * 32 + l32;
    if (m >= M) continue;
#pragma unroll
    for (int tw = 0; tw < 2; ++tw)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = n0 + wn * 64 + tw * 32 + 8 * g + 4 * half;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc[tw][ta][4 * g + e] + (bias && n + e < N ? bias[n + e] : 0.f);
        if (whole && n + 3 < N) {
          *reinterpret_cast<float4*>(C + (size_t)m * N + n) = make_float4(v[0], v[1], v[2], v[3]);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < N) C[(size_t)m * N + n + e] = v[e];
        }
      }
  }
}

// 1 if qil_gemm_f32_mfma takes these sizes in this many splits (the operands' alignment is checked by the call).
extern "C" int qil_gemm_f32_mfma_takes(int M, int N, int K, int splits) {
  return M >= 1 && N >= 1 && splits >= 1 && splits <= 64 && K % (FM_STAGE * splits) == 0 &&
         K / (FM_STAGE * splits) >= FM_RING - 1 && (N + FM_COLS - 1) / FM_COLS <= 65535;
}

// Blocks of the product before K is split.
extern "C" long qil_gemm_f32_mfma_blocks(int M, int N) {
  return (long)((M + (M <= 128 ? 127 : 255)) / (M <= 128 ? 128 : 256)) * ((N + FM_COLS - 1) / FM_COLS);
}

// Splits of K for a product whose consumer takes partial sums: as many as bring the blocks to about 256 (at most 32,
// whole stages, 4 or more a split); 1 if the tiles alone fill most of the chip.
extern "C" int qil_gemm_f32_mfma_splits(int M, int N, int K) {
  const long blocks = qil_gemm_f32_mfma_blocks(M, N);
  if (blocks >= 160 || K % FM_STAGE) return 1;
  const int stages = K / FM_STAGE;
  int best = 1;
  for (int c = 2; c <= 32 && blocks * c <= 320; ++c)
    if (stages % c == 0 && stages / c >= 4) best = c;
  return best;
}

template <int ROWS>
static int fm_launch(const float* A, const float* W, const float* bias, float* C, int M, int N, int K, int splits,
                     hipStream_t s) {
  const size_t lds = (size_t)FM_RING * (ROWS + FM_COLS) * 128;
  auto kernel = gemm_f32_mfma_kernel<ROWS>;
  static bool granted = false;                             // per instantiation
  if (!granted) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
    granted = true;
  }
  dim3 grid((M + ROWS - 1) / ROWS, (N + FM_COLS - 1) / FM_COLS, splits);
  hipLaunchKernelGGL(kernel, grid, dim3((ROWS / 32 + 2) * QIL_WAVE), lds, s, A, W, bias, C, M, N, K, K / FM_STAGE / splits);
  QIL_RETURN_LAUNCH_STATUS();
}

// C float32 [splits][M][N] = partial sums of A W^T over the splits' ranges of K (+ bias: one split only).
extern "C" int qil_gemm_f32_mfma(const float* A, const float* W, const float* bias, float* C, int M, int N, int K,
                                 int splits, hipStream_t s) {
  if (M == 0 || N == 0) return 0;
  if (!qil_gemm_f32_mfma_takes(M, N, K, splits) || (bias && splits > 1) ||
      (((uintptr_t)A | (uintptr_t)W | (uintptr_t)C) % 16))
    return -1;
  return M <= 128 ? fm_launch<128>(A, W, bias, C, M, N, K, splits, s) : fm_launch<256>(A, W, bias, C, M, N, K, splits, s);
}
