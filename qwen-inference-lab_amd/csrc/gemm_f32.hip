// True float32 matrix product for the 32-bit path: C[M, N] = A[M, K] W[N, K]^T (+ bias[N]).
//
// Inputs, products and sums are IEEE float32 FMA on the vector units: no matrix-core mode, no
// reduced-precision inputs, no split of K across threads, so every element of C is one thread's
// sequential sum over k and does not depend on M, on the row's place in the batch or on the tile
// it falls into.  Both operands have K contiguous (nn.Linear layout, qil/model.py:32-40).
// 64 x 64 x 16 tiles in LDS, 256 threads, 4 x 4 outputs a thread.
#include "common.h"

#define SG_BM 64
#define SG_BN 64
#define SG_BK 16
#define SG_PAD 4

template <bool VEC>
__global__ void __launch_bounds__(256)
sgemm_nt_kernel(const float* __restrict__ A, const float* __restrict__ W, const float* __restrict__ bias,
                float* __restrict__ C, int M, int N, int K) {
  __shared__ float As[SG_BK][SG_BM + SG_PAD];
  __shared__ float Ws[SG_BK][SG_BN + SG_PAD];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * SG_BM, n0 = blockIdx.x * SG_BN;
  const int load_row = tid >> 2, load_k = (tid & 3) * 4;      // 64 rows x 4 quads of k
  const int ty = tid >> 4, tx = tid & 15;

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += SG_BK) {
    float a[4], w[4];
    const int am = m0 + load_row, wn = n0 + load_row, kk = k0 + load_k;
    if (VEC && am < M && kk + 3 < K) {
      const float4 v = *reinterpret_cast<const float4*>(A + (size_t)am * K + kk);
      a[0] = v.x; a[1] = v.y; a[2] = v.z; a[3] = v.w;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = (am < M && kk + i < K) ? A[(size_t)am * K + kk + i] : 0.f;
    }
    if (VEC && wn < N && kk + 3 < K) {
      const float4 v = *reinterpret_cast<const float4*>(W + (size_t)wn * K + kk);
      w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) w[i] = (wn < N && kk + i < K) ? W[(size_t)wn * K + kk + i] : 0.f;
    }
    __syncthreads();                       // previous tile fully consumed
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      As[load_k + i][load_row] = a[i];
      Ws[load_k + i][load_row] = w[i];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < SG_BK; ++k) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = Ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) C[(size_t)m * N + n] = acc[i][j] + (bias ? bias[n] : 0.f);
    }
  }
}

// Few rows (decode): one wave per output column, lanes stride over K; each (m, n) is still a fixed
// order sum: lane partials in k order, then the wave's butterfly.
#define SV_ROWS 8
__global__ void __launch_bounds__(256)
sgemv_rows_kernel(const float* __restrict__ A, const float* __restrict__ W, const float* __restrict__ bias,
                  float* __restrict__ C, int M, int N, int K, int m0) {
  const int lane = threadIdx.x & (QIL_WAVE - 1);
  const int n = blockIdx.x * (blockDim.x / QIL_WAVE) + threadIdx.x / QIL_WAVE;
  if (n >= N) return;
  const float* w = W + (size_t)n * K;
  float acc[SV_ROWS];
#pragma unroll
  for (int r = 0; r < SV_ROWS; ++r) acc[r] = 0.f;
  const int rows = min(SV_ROWS, M - m0);
  for (int k = lane; k < K; k += QIL_WAVE) {
    const float wv = w[k];
#pragma unroll
    for (int r = 0; r < SV_ROWS; ++r)
      if (r < rows) acc[r] = fmaf(A[(size_t)(m0 + r) * K + k], wv, acc[r]);
  }
#pragma unroll
  for (int r = 0; r < SV_ROWS; ++r) {
    const float total = wave_sum(acc[r]);
    if (lane == 0 && r < rows) C[(size_t)(m0 + r) * N + n] = total + (bias ? bias[n] : 0.f);
  }
}

extern "C" int qil_gemm_f32(const float* A, const float* W, const float* bias, float* C, int M, int N, int K,
                            hipStream_t s) {
  if (M == 0 || N == 0) return 0;
  if (K < 1) return -1;
  if (M <= 2 * SV_ROWS) {
    const int waves = 4;
    for (int m0 = 0; m0 < M; m0 += SV_ROWS)
      hipLaunchKernelGGL(sgemv_rows_kernel, dim3((N + waves - 1) / waves), dim3(waves * QIL_WAVE), 0, s, A, W, bias, C,
                         M, N, K, m0);
    QIL_RETURN_LAUNCH_STATUS();
  }
  dim3 grid((N + SG_BN - 1) / SG_BN, (M + SG_BM - 1) / SG_BM);
  const bool vec = (K % 4 == 0) && (((uintptr_t)A | (uintptr_t)W) % 16 == 0);
  if (vec) hipLaunchKernelGGL(sgemm_nt_kernel<true>, grid, dim3(256), 0, s, A, W, bias, C, M, N, K);
  else     hipLaunchKernelGGL(sgemm_nt_kernel<false>, grid, dim3(256), 0, s, A, W, bias, C, M, N, K);
  QIL_RETURN_LAUNCH_STATUS();
}
