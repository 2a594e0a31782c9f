// bfloat16 matrix product on the matrix cores: C[M, N] = A[M, K] W[N, K]^T (+ bias[N]), float32
// accumulation, C in bfloat16 or float32.  Both operands have K contiguous (qil/model.py:32-40).
//
// Weight-streaming kernel for few rows (decode, selected logit rows): a block owns 16 rows of W (16
// output columns) and 16 * MT rows of A; its waves split K in interleaved steps of 32, so together
// they stream each W row contiguously, and every wave issues v_mfma_f32_16x16x32_bf16 with the W
// fragment reused across the MT row tiles.  The waves' partial sums meet in LDS and are added in
// wave order, so a result does not depend on timing.  W is read from HBM once per 16 * MT rows of A.
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
__device__ __forceinline__ bf16x8 load_frag(const bf16_t* __restrict__ base, int row, int rows, int k, int K) {
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
  return __builtin_bit_cast(bf16x8, raw);
}

template <int MT, int WAVES, bool ALIGNED, typename OUT>
__global__ void __launch_bounds__(WAVES * QIL_WAVE)
gemm_bf16_stream_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, const float* __restrict__ bias,
                        OUT* __restrict__ C, int M, int N, int K) {
  __shared__ float partial[WAVES][MT][256];
  const int lane = threadIdx.x & (QIL_WAVE - 1), wave = threadIdx.x / QIL_WAVE;
  const int r = lane & 15, kb = lane >> 4;
  const int n0 = blockIdx.x * 16, m0 = blockIdx.y * 16 * MT;

  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};

  const int steps = (K + 31) / 32;
  for (int step = wave; step < steps; step += WAVES) {
    const int k = step * 32 + kb * 8;
    const bf16x8 b = load_frag<ALIGNED>(W, n0 + r, N, k, K);
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const bf16x8 a = load_frag<ALIGNED>(A, m0 + t * 16 + r, M, k, K);
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[t], 0, 0, 0);
    }
  }
  // lane holds D[4 kb + i][r]; park it as [m][n] so the final pass is contiguous in n
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) partial[wave][t][(4 * kb + i) * 16 + r] = acc[t][i];
  __syncthreads();
  for (int idx = threadIdx.x; idx < MT * 256; idx += WAVES * QIL_WAVE) {
    const int t = idx >> 8, cell = idx & 255;
    const int m = m0 + t * 16 + (cell >> 4), n = n0 + (cell & 15);
    if (m >= M || n >= N) continue;
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) total += partial[w][t][cell];
    store_out(C + (size_t)m * N + n, total + (bias ? bias[n] : 0.f));
  }
}

template <int MT, int WAVES, typename OUT>
static void launch_stream(const bf16_t* A, const bf16_t* W, const float* bias, OUT* C, int M, int N, int K,
                          hipStream_t s) {
  dim3 grid((N + 15) / 16, (M + 16 * MT - 1) / (16 * MT));
  const bool aligned = (K % 8 == 0) && (((uintptr_t)A | (uintptr_t)W) % 16 == 0);
  if (aligned)
    hipLaunchKernelGGL((gemm_bf16_stream_kernel<MT, WAVES, true, OUT>), grid, dim3(WAVES * QIL_WAVE), 0, s, A, W, bias,
                       C, M, N, K);
  else
    hipLaunchKernelGGL((gemm_bf16_stream_kernel<MT, WAVES, false, OUT>), grid, dim3(WAVES * QIL_WAVE), 0, s, A, W, bias,
                       C, M, N, K);
}

template <typename OUT>
static void dispatch_stream(const bf16_t* A, const bf16_t* W, const float* bias, OUT* C, int M, int N, int K,
                            hipStream_t s) {
  // Short K leaves little to split: fewer waves.  Row tiles: 16, 32 or 64 rows of A per pass over W.
  if (K <= 512) {
    if (M <= 16) launch_stream<1, 2, OUT>(A, W, bias, C, M, N, K, s);
    else if (M <= 32) launch_stream<2, 2, OUT>(A, W, bias, C, M, N, K, s);
    else launch_stream<4, 2, OUT>(A, W, bias, C, M, N, K, s);
  } else {
    if (M <= 16) launch_stream<1, 8, OUT>(A, W, bias, C, M, N, K, s);
    else if (M <= 32) launch_stream<2, 8, OUT>(A, W, bias, C, M, N, K, s);
    else launch_stream<4, 8, OUT>(A, W, bias, C, M, N, K, s);
  }
}

// out_dtype: QIL_BF16 or QIL_F32.
extern "C" int qil_gemm_bf16(const void* A, const void* W, const float* bias, void* C, int M, int N, int K,
                             int out_dtype, hipStream_t s) {
  if (M == 0 || N == 0) return 0;
  if (K < 1) return -1;
  if (out_dtype == QIL_F32)
    dispatch_stream<float>((const bf16_t*)A, (const bf16_t*)W, bias, (float*)C, M, N, K, s);
  else
    dispatch_stream<bf16_t>((const bf16_t*)A, (const bf16_t*)W, bias, (bf16_t*)C, M, N, K, s);
  QIL_RETURN_LAUNCH_STATUS();
}
