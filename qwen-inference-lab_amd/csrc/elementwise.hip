// Embedding gather, RMSNorm fused with the residual add, SiLU gate, bias add.
// T is the model's element type (float or bfloat16); the residual stream is float32.
#include "common.h"

// stream[n, :] = float(table[token[n], :])                      (qil/model.py:126)
template <typename T>
__global__ void embed_kernel(const int* __restrict__ tokens, const T* __restrict__ table,
                             float* __restrict__ stream, int width) {
  const int n = blockIdx.x;
  const T* row = table + (size_t)tokens[n] * width;
  float* out = stream + (size_t)n * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) out[i] = ld(row + i);
}

// One block per output row.
//   x = stream[r] (+ delta[r]);  if (update) stream[r] = x;
//   out[m] = round_T(round_T(x * rsqrt(mean(x^2) + eps)) * weight)   (qil/model.py:15-23)
// r = rows ? rows[m] : m.  Statistics, the sum and the weight product are float32.
template <typename T>
__global__ void add_rmsnorm_kernel(float* __restrict__ stream, const T* __restrict__ delta,
                                   const int* __restrict__ rows, const float* __restrict__ weight,
                                   T* __restrict__ out, int width, float eps, int update) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  const size_t r = rows ? (size_t)rows[m] : (size_t)m;
  float* x = stream + r * width;
  const T* d = delta ? delta + r * width : nullptr;
  float sum = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = x[i];
    if (d) {
      v += ld(d + i);
      if (update) x[i] = v;
    }
    sum += v * v;
  }
  sum = block_sum(sum, scratch);
  const float rstd = rsqrtf(sum / (float)width + eps);
  T* y = out + (size_t)m * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = x[i];
    if (d && !update) v += ld(d + i);
    st(y + i, round_to<T>(v * rstd) * weight[i]);
  }
}

// out[n, i] = silu(gate_up[n, i]) * gate_up[n, inner + i], silu(z) = z * sigmoid(z)   (qil/model.py:71)
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int inner, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t n = idx / inner;
  const int i = (int)(idx - n * inner);
  const float g = ld(gate_up + n * 2 * (size_t)inner + i);
  const float u = ld(gate_up + n * 2 * (size_t)inner + inner + i);
  st(out + idx, (g / (1.f + expf(-g))) * u);
}

// x[n, i] += bias[i]
template <typename T>
__global__ void add_bias_kernel(T* __restrict__ x, const float* __restrict__ bias, int width, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  st(x + idx, ld(x + idx) + bias[idx % width]);
}

extern "C" {

int qil_embed(const int* tokens, const void* table, float* stream, int n, int width, int dtype, hipStream_t s) {
  if (n == 0) return 0;
  const int threads = width >= 1024 ? 256 : 64;
  if (dtype == QIL_F32)
    hipLaunchKernelGGL(embed_kernel<float>, dim3(n), dim3(threads), 0, s, tokens, (const float*)table, stream, width);
  else
    hipLaunchKernelGGL(embed_kernel<bf16_t>, dim3(n), dim3(threads), 0, s, tokens, (const bf16_t*)table, stream, width);
  QIL_RETURN_LAUNCH_STATUS();
}

int qil_add_rmsnorm(float* stream, const void* delta, const int* rows, const float* weight, void* out,
                    int n_out, int width, float eps, int update, int dtype, hipStream_t s) {
  if (n_out == 0) return 0;
  const int threads = width >= 2048 ? 512 : width >= 512 ? 256 : 64;
  if (dtype == QIL_F32)
    hipLaunchKernelGGL(add_rmsnorm_kernel<float>, dim3(n_out), dim3(threads), 0, s, stream, (const float*)delta,
                       rows, weight, (float*)out, width, eps, update);
  else
    hipLaunchKernelGGL(add_rmsnorm_kernel<bf16_t>, dim3(n_out), dim3(threads), 0, s, stream, (const bf16_t*)delta,
                       rows, weight, (bf16_t*)out, width, eps, update);
  QIL_RETURN_LAUNCH_STATUS();
}

int qil_silu_mul(const void* gate_up, void* out, int n, int inner, int dtype, hipStream_t s) {
  const size_t total = (size_t)n * inner;
  if (total == 0) return 0;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (dtype == QIL_F32)
    hipLaunchKernelGGL(silu_mul_kernel<float>, dim3(blocks), dim3(256), 0, s, (const float*)gate_up, (float*)out, inner, total);
  else
    hipLaunchKernelGGL(silu_mul_kernel<bf16_t>, dim3(blocks), dim3(256), 0, s, (const bf16_t*)gate_up, (bf16_t*)out, inner, total);
  QIL_RETURN_LAUNCH_STATUS();
}

int qil_add_bias(void* x, const float* bias, int n, int width, int dtype, hipStream_t s) {
  const size_t total = (size_t)n * width;
  if (total == 0) return 0;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (dtype == QIL_F32)
    hipLaunchKernelGGL(add_bias_kernel<float>, dim3(blocks), dim3(256), 0, s, (float*)x, bias, width, total);
  else
    hipLaunchKernelGGL(add_bias_kernel<bf16_t>, dim3(blocks), dim3(256), 0, s, (bf16_t*)x, bias, width, total);
  QIL_RETURN_LAUNCH_STATUS();
}

}  // extern "C"
