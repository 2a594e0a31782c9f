// bfloat16 matrix product on the matrix cores for few rows (decode, selected logit rows):
//   C[M, N] = A[M, K] W[N, K]^T (+ bias[N]),  float32 accumulation.
// Both operands have K contiguous (qil/model.py:32-40).  The product is bound by streaming W once
// from HBM, so the kernel is shaped to keep as many loads in flight as the chip can hold:
//
//   * a block owns 16 rows of W (16 output columns), 16 * MT rows of A and one of `splits` ranges
//     of K; its waves split that range into contiguous pieces, and every wave issues the loads
//     of four 32-wide k steps before the first v_mfma_f32_16x16x32_bf16 that uses them;
//   * with few columns (N / 16 blocks would leave CUs idle) K is split over blocks as well:
//     the block writes a float32 partial result C[split, M, N], and the kernel that consumes
//     the product (norm, rotary/store, SiLU gate) adds the partials in split order.  Sums are
//     therefore made in a fixed order: the waves' in wave order, the splits' in split order;
//   * with splits == 1 the result may be rounded to bfloat16 here (and take the bias).
//
// Fragment layout of v_mfma_f32_16x16x32_bf16 (wave64): lane l supplies A[l % 16][8 (l / 16) .. +7]
// and B[8 (l / 16) .. +7][l % 16]; it receives D[4 (l / 16) + i][l % 16], i < 4.  A and W rows are
// both loaded with the same k assignment, so only the D layout matters for correctness.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void store_out(float* p, float v) { *p = v; }
__device__ __forceinline__ void store_out(bf16_t* p, float v) { *p = f32_to_bf16(v); }

// Eight consecutive bf16 of a row starting at k, zero where the row or k is out of range.
template <bool ALIGNED>
__device__ __forceinline__ uint4 load_frag(const bf16_t* __restrict__ base, int row, int rows, int k, int K) {
  uint4 raw = make_uint4(0, 0, 0, 0);
  if (row < rows && k < K) {
    const bf16_t* p = base + (size_t)row * K + k;
    if (ALIGNED) {
      raw = *reinterpret_cast<const uint4*>(p);
    } else {
      uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (k + e < K) w[e >> 1] |= (uint32_t)p[e] << ((e & 1) * 16);
      raw = make_uint4(w[0], w[1], w[2], w[3]);
    }
  }
  return raw;
}

#define GEMM_UNROLL 4

template <int MT, int WAVES, bool ALIGNED, typename OUT>
__global__ void __launch_bounds__(WAVES * QIL_WAVE)
gemm_bf16_stream_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, const float* __restrict__ bias,
                        OUT* __restrict__ C, int M, int N, int K, int steps_per_split) {
  __shared__ float partial[WAVES][MT][256];
  const int lane = threadIdx.x & (QIL_WAVE - 1), wave = threadIdx.x / QIL_WAVE;
  const int r = lane & 15, kb = lane >> 4;
  const int n0 = blockIdx.x * 16, m0 = blockIdx.y * 16 * MT, split = blockIdx.z;

  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};

  // this block's k steps, cut into contiguous pieces for the waves
  const int steps = (K + 31) / 32;
  const int s0 = split * steps_per_split, s1 = min(steps, s0 + steps_per_split);
  const int per_wave = (s1 - s0 + WAVES - 1) / WAVES;
  const int w0 = s0 + wave * per_wave, w1 = min(s1, w0 + per_wave);
  for (int step = w0; step < w1; step += GEMM_UNROLL) {
    uint4 b[GEMM_UNROLL], a[GEMM_UNROLL][MT];
#pragma unroll
    for (int u = 0; u < GEMM_UNROLL; ++u) {
      const int k = (step + u < w1) ? (step + u) * 32 + kb * 8 : K;      // K: out of range, loads nothing
      b[u] = load_frag<ALIGNED>(W, n0 + r, N, k, K);
#pragma unroll
      for (int t = 0; t < MT; ++t) a[u][t] = load_frag<ALIGNED>(A, m0 + t * 16 + r, M, k, K);
    }
#pragma unroll
    for (int u = 0; u < GEMM_UNROLL; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a[u][t]),
                                                         __builtin_bit_cast(bf16x8, b[u]), acc[t], 0, 0, 0);
  }
  // lane holds D[4 kb + i][r]; park it as [m][n] so the final pass is contiguous in n
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) partial[wave][t][(4 * kb + i) * 16 + r] = acc[t][i];
  __syncthreads();
  OUT* out = C + (size_t)split * M * N;
  for (int idx = threadIdx.x; idx < MT * 256; idx += WAVES * QIL_WAVE) {
    const int t = idx >> 8, cell = idx & 255;
    const int m = m0 + t * 16 + (cell >> 4), n = n0 + (cell & 15);
    if (m >= M || n >= N) continue;
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) total += partial[w][t][cell];
    store_out(out + (size_t)m * N + n, total + (bias ? bias[n] : 0.f));
  }
}

template <int MT, int WAVES, typename OUT>
static void launch_stream(const bf16_t* A, const bf16_t* W, const float* bias, OUT* C, int M, int N, int K, int splits,
                          hipStream_t s) {
  const int steps = (K + 31) / 32;
  const int steps_per_split = (steps + splits - 1) / splits;
  dim3 grid((N + 15) / 16, (M + 16 * MT - 1) / (16 * MT), splits);
  const bool aligned = (K % 8 == 0) && (((uintptr_t)A | (uintptr_t)W) % 16 == 0);
  if (aligned)
    hipLaunchKernelGGL((gemm_bf16_stream_kernel<MT, WAVES, true, OUT>), grid, dim3(WAVES * QIL_WAVE), 0, s, A, W, bias,
                       C, M, N, K, steps_per_split);
  else
    hipLaunchKernelGGL((gemm_bf16_stream_kernel<MT, WAVES, false, OUT>), grid, dim3(WAVES * QIL_WAVE), 0, s, A, W, bias,
                       C, M, N, K, steps_per_split);
}

template <typename OUT>
static void dispatch_stream(const bf16_t* A, const bf16_t* W, const float* bias, OUT* C, int M, int N, int K,
                            int splits, hipStream_t s) {
  // Row tiles: 16, 32 or 64 rows of A per pass over W.  Waves per block: as many as have at least
  // one unrolled group of k steps each.
  const int steps = ((K + 31) / 32 + splits - 1) / splits;
  const int waves = steps >= 8 * GEMM_UNROLL ? 8 : steps >= 4 * GEMM_UNROLL ? 4 : 2;
#define QIL_STREAM_CASE(MT)                                                              \
  if (waves == 8) launch_stream<MT, 8, OUT>(A, W, bias, C, M, N, K, splits, s);          \
  else if (waves == 4) launch_stream<MT, 4, OUT>(A, W, bias, C, M, N, K, splits, s);     \
  else launch_stream<MT, 2, OUT>(A, W, bias, C, M, N, K, splits, s)
  if (M <= 16) { QIL_STREAM_CASE(1); }
  else if (M <= 32) { QIL_STREAM_CASE(2); }
  else { QIL_STREAM_CASE(4); }
#undef QIL_STREAM_CASE
}

// How many ways to split K so that the launch has enough waves for the chip, given the columns.
extern "C" int qil_gemm_bf16_splits(int M, int N, int K) {
  const int tiles = ((N + 15) / 16) * ((M + 63) / 64);
  const int steps = (K + 31) / 32;
  int splits = 1;
  // aim at >= 1024 blocks; keep at least 8 k steps (256 columns of K) per split
  while (tiles * splits < 1024 && splits < 16 && steps / (splits * 2) >= 8) splits *= 2;
  return splits;
}

// out_dtype QIL_BF16: C bfloat16 [M, N], splits must be 1.  QIL_F32: C float32 [splits, M, N], the
// value being the sum over the first axis; bias (if any) requires splits == 1.
extern "C" int qil_gemm_bf16(const void* A, const void* W, const float* bias, void* C, int M, int N, int K,
                             int out_dtype, int splits, hipStream_t s) {
  if (M == 0 || N == 0) return 0;
  if (K < 1 || splits < 1 || splits > 65535 || (splits > 1 && (out_dtype != QIL_F32 || bias))) return -1;
  if (out_dtype == QIL_F32)
    dispatch_stream<float>((const bf16_t*)A, (const bf16_t*)W, bias, (float*)C, M, N, K, splits, s);
  else
    dispatch_stream<bf16_t>((const bf16_t*)A, (const bf16_t*)W, bias, (bf16_t*)C, M, N, K, splits, s);
  QIL_RETURN_LAUNCH_STATUS();
}
