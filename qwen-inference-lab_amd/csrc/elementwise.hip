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

// The same for rows of bfloat16 whose width is a multiple of 8, 16-byte aligned: one thread, eight elements.
__global__ void embed_bf16x8_kernel(const int* __restrict__ tokens, const bf16_t* __restrict__ table,
                                    float* __restrict__ stream, int width) {
  const int n = blockIdx.x;
  const bf16_t* row = table + (size_t)tokens[n] * width;
  float* out = stream + (size_t)n * width;
  for (int i = threadIdx.x * 8; i < width; i += blockDim.x * 8) {
    const uint4 raw = *reinterpret_cast<const uint4*>(row + i);
    *reinterpret_cast<float4*>(out + i) = make_float4(__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u),
                                                      __uint_as_float(raw.y << 16), __uint_as_float(raw.y & 0xffff0000u));
    *reinterpret_cast<float4*>(out + i + 4) = make_float4(__uint_as_float(raw.z << 16), __uint_as_float(raw.z & 0xffff0000u),
                                                          __uint_as_float(raw.w << 16), __uint_as_float(raw.w & 0xffff0000u));
  }
}

__device__ __forceinline__ float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4(const bf16_t* p) {
  const uint2 raw = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u),
                     __uint_as_float(raw.y << 16), __uint_as_float(raw.y & 0xffff0000u));
}
__device__ __forceinline__ void store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void store4(bf16_t* p, float4 v) {
  *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16(v.x, v.y), pack_bf16(v.z, v.w));
}

// A sub-layer's output arrives either in the model's type T (one array) or as float32 partial sums
// of a K-split matrix product, [splits][rows][width], which the consumer adds in split order.
// Loads go out eight at a time before the first is used; the additions stay in split order.
template <typename TD>
__device__ __forceinline__ float load_sum(const TD* __restrict__ base, size_t index, int splits, size_t stride) {
  float v = 0.f;
  for (int s0 = 0; s0 < splits; s0 += 8) {
    float part[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) part[u] = s0 + u < splits ? ld(base + (s0 + u) * stride + index) : 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u) v += part[u];
  }
  return v;
}
template <typename TD>
__device__ __forceinline__ float4 load_sum4(const TD* __restrict__ base, size_t index, int splits, size_t stride) {
  float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int s0 = 0; s0 < splits; s0 += 8) {
    float4 part[8];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      part[u] = s0 + u < splits ? load4(base + (s0 + u) * stride + index) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int u = 0; u < 8; ++u) { v.x += part[u].x; v.y += part[u].y; v.z += part[u].z; v.w += part[u].w; }
  }
  return v;
}
// One block per output row.
//   x = stream[r] (+ delta[r]);  if (update) stream[r] = x;
//   out[m] = round_T(round_T(x * rsqrt(mean(x^2) + eps)) * weight)   (qil/model.py:15-23)
// r = rows ? rows[m] : m.  Statistics, the sum and the weight product are float32.
template <typename TD, typename T>
__global__ void add_rmsnorm_kernel(float* __restrict__ stream, const TD* __restrict__ delta, int splits,
                                   size_t split_stride, const int* __restrict__ rows,
                                   const float* __restrict__ weight, T* __restrict__ out, int width, float eps,
                                   int update) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  const size_t r = rows ? (size_t)rows[m] : (size_t)m;
  float* x = stream + r * width;
  float sum = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = x[i];
    if (delta) {
      v += load_sum(delta, r * width + i, splits, split_stride);
      if (update) x[i] = v;
    }
    sum += v * v;
  }
  sum = block_sum(sum, scratch);
  const float rstd = rsqrtf(sum / (float)width + eps);
  T* y = out + (size_t)m * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = x[i];
    if (delta && !update) v += load_sum(delta, r * width + i, splits, split_stride);
    st(y + i, round_to<T>(v * rstd) * weight[i]);
  }
}

// The same for width % 4 == 0 and width <= 4 * J * THREADS: every access is a 16-byte (8-byte for
// bfloat16) vector, all loads (stream, delta or its partial sums, weight) are issued before the first
// is used, and the row stays in registers between the statistics and the output.
template <typename TD, typename T, int THREADS, int J>
__global__ void __launch_bounds__(THREADS)
add_rmsnorm_vec_kernel(float* __restrict__ stream, const TD* __restrict__ delta, int splits, size_t split_stride,
                       const int* __restrict__ rows, const float* __restrict__ weight, T* __restrict__ out, int width,
                       float eps, int update) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  const size_t r = rows ? (size_t)rows[m] : (size_t)m;
  float* x = stream + r * width;
  float4 cache[J], w[J], d[J];
#pragma unroll
  for (int j = 0; j < J; ++j) {
    const int i = (threadIdx.x + j * THREADS) * 4;
    const bool live = i < width;
    cache[j] = live ? load4(x + i) : make_float4(0.f, 0.f, 0.f, 0.f);
    w[j] = live ? load4(weight + i) : make_float4(0.f, 0.f, 0.f, 0.f);
    d[j] = (live && delta) ? load_sum4(delta, r * width + i, splits, split_stride) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < J; ++j) {
    const int i = (threadIdx.x + j * THREADS) * 4;
    float4 v = cache[j];
    v.x += d[j].x; v.y += d[j].y; v.z += d[j].z; v.w += d[j].w;
    if (delta && update && i < width) store4(x + i, v);
    cache[j] = v;
    sum += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
  }
  sum = block_sum(sum, scratch);
  const float rstd = rsqrtf(sum / (float)width + eps);
  T* y = out + (size_t)m * width;
#pragma unroll
  for (int j = 0; j < J; ++j) {
    const int i = (threadIdx.x + j * THREADS) * 4;
    if (i < width) {
      const float4 v = cache[j];
      store4(y + i, make_float4(round_to<T>(v.x * rstd) * w[j].x, round_to<T>(v.y * rstd) * w[j].y,
                                round_to<T>(v.z * rstd) * w[j].z, round_to<T>(v.w * rstd) * w[j].w));
    }
  }
}

// out[n, i] = silu(gate[n, i]) * up[n, i], silu(z) = z * sigmoid(z)   (qil/model.py:71).  The two halves of a row of
// gate_up [n, 2 inner] are stacked (gate columns first: gate i at i, up i at inner + i) or interleaved in tiles of 16
// columns (gate tile, up tile, gate tile, ...: gate i at 32 (i / 16) + i % 16, up i 16 further; inner % 16 == 0).
__device__ __forceinline__ size_t gate_column(int i, int interleaved) {
  return interleaved ? (size_t)(i >> 4) * 32 + (i & 15) : (size_t)i;
}
template <typename TD, typename T>
__global__ void silu_mul_kernel(const TD* __restrict__ gate_up, int splits, size_t split_stride, T* __restrict__ out,
                                int inner, size_t total, int interleaved) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t n = idx / inner;
  const int i = (int)(idx - n * inner);
  const size_t at = n * 2 * (size_t)inner + gate_column(i, interleaved);
  const float g = load_sum(gate_up, at, splits, split_stride);
  const float u = load_sum(gate_up, at + (interleaved ? 16 : inner), splits, split_stride);
  st(out + idx, (g / (1.f + expf(-g))) * u);
}

// Four outputs a thread, vector loads and stores; inner % 4 == 0.
template <typename TD, typename T>
__global__ void silu_mul_vec_kernel(const TD* __restrict__ gate_up, int splits, size_t split_stride,
                                    T* __restrict__ out, int inner, size_t total4, int interleaved) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total4) return;
  const int per_row = inner / 4;
  const size_t n = idx / per_row;
  const int i = (int)(idx - n * per_row) * 4;
  const size_t at = n * 2 * (size_t)inner + gate_column(i, interleaved);
  const float4 g = load_sum4(gate_up, at, splits, split_stride);
  const float4 u = load_sum4(gate_up, at + (interleaved ? 16 : inner), splits, split_stride);
  store4(out + n * (size_t)inner + i, make_float4((g.x / (1.f + expf(-g.x))) * u.x, (g.y / (1.f + expf(-g.y))) * u.y,
                                                  (g.z / (1.f + expf(-g.z))) * u.z, (g.w / (1.f + expf(-g.w))) * u.w));
}

// bfloat16 in and out, eight outputs a thread: 16-byte loads and stores (inner % 8 == 0).
__global__ void silu_mul_bf16x8_kernel(const bf16_t* __restrict__ gate_up, bf16_t* __restrict__ out, int inner,
                                       size_t total8, int interleaved) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total8) return;
  const int per_row = inner / 8;
  const size_t n = idx / per_row;
  const int i = (int)(idx - n * per_row) * 8;
  float g[8], u[8], y[8];
  const size_t at = n * 2 * (size_t)inner + gate_column(i, interleaved);
  ld8(gate_up + at, g);
  ld8(gate_up + at + (interleaved ? 16 : inner), u);
#pragma unroll
  for (int e = 0; e < 8; ++e) y[e] = (g[e] / (1.f + expf(-g[e]))) * u[e];
  *reinterpret_cast<uint4*>(out + n * (size_t)inner + i) =
      make_uint4(pack_bf16(y[0], y[1]), pack_bf16(y[2], y[3]), pack_bf16(y[4], y[5]), pack_bf16(y[6], y[7]));
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
  else if (width % 8 == 0 && (((uintptr_t)table | (uintptr_t)stream) % 16) == 0)
    hipLaunchKernelGGL(embed_bf16x8_kernel, dim3(n), dim3(width >= 2048 ? 256 : 64), 0, s, tokens, (const bf16_t*)table,
                       stream, width);
  else
    hipLaunchKernelGGL(embed_kernel<bf16_t>, dim3(n), dim3(threads), 0, s, tokens, (const bf16_t*)table, stream, width);
  QIL_RETURN_LAUNCH_STATUS();
}

// delta: null, or the sub-layer output to add: delta_dtype QIL_BF16 (one array, splits == 1) or QIL_F32
// ([splits][delta_rows][width] partial sums).  out_dtype: type of `out`.
int qil_add_rmsnorm(float* stream, const void* delta, int delta_dtype, int splits, int delta_rows, const int* rows,
                    const float* weight, void* out, int n_out, int width, float eps, int update, int out_dtype,
                    hipStream_t s) {
  if (n_out == 0) return 0;
  if (splits < 1 || (delta_dtype == QIL_BF16 && splits != 1)) return -1;
  const size_t stride = (size_t)delta_rows * width;
  const bool vec = width % 4 == 0 && width <= 8192 &&
                   (((uintptr_t)stream | (uintptr_t)delta | (uintptr_t)weight | (uintptr_t)out) % 16 == 0);
#define QIL_NORM_VEC(TD, T, THREADS, J)                                                                             \
  hipLaunchKernelGGL((add_rmsnorm_vec_kernel<TD, T, THREADS, J>), dim3(n_out), dim3(THREADS), 0, s, stream,          \
                     (const TD*)delta, splits, stride, rows, weight, (T*)out, width, eps, update)
#define QIL_NORM_CASE(TD, T)                                                                                         \
  do {                                                                                                               \
    if (vec && width <= 256) QIL_NORM_VEC(TD, T, 64, 1);                                                             \
    else if (vec && width <= 1024) QIL_NORM_VEC(TD, T, 256, 1);                                                      \
    else if (vec && width <= 2048) QIL_NORM_VEC(TD, T, 512, 1);                                                      \
    else if (vec && width <= 4096) QIL_NORM_VEC(TD, T, 512, 2);                                                      \
    else if (vec) QIL_NORM_VEC(TD, T, 1024, 2);                                                                      \
    else                                                                                                             \
      hipLaunchKernelGGL((add_rmsnorm_kernel<TD, T>), dim3(n_out), dim3(width >= 2048 ? 512 : width >= 512 ? 256 : 64), \
                         0, s, stream, (const TD*)delta, splits, stride, rows, weight, (T*)out, width, eps, update); \
  } while (0)
  if (out_dtype == QIL_F32) {
    if (delta_dtype != QIL_F32) return -1;
    QIL_NORM_CASE(float, float);
  } else if (delta_dtype == QIL_F32) {
    QIL_NORM_CASE(float, bf16_t);
  } else {
    QIL_NORM_CASE(bf16_t, bf16_t);
  }
#undef QIL_NORM_CASE
#undef QIL_NORM_VEC
  QIL_RETURN_LAUNCH_STATUS();
}

// gate_up: in_dtype QIL_BF16 [n, 2 inner] or QIL_F32 [splits][n][2 inner] partial sums.
int qil_silu_mul(const void* gate_up, int in_dtype, int splits, void* out, int n, int inner, int out_dtype,
                 int interleaved, hipStream_t s) {
  const size_t total = (size_t)n * inner;
  if (total == 0) return 0;
  if (splits < 1 || (in_dtype == QIL_BF16 && splits != 1) || (interleaved && inner % 16)) return -1;
  const size_t stride = (size_t)n * 2 * inner;
  if (in_dtype == QIL_BF16 && out_dtype == QIL_BF16 && inner % 8 == 0 && (((uintptr_t)gate_up | (uintptr_t)out) % 16 == 0)) {
    const size_t work8 = total / 8;
    hipLaunchKernelGGL(silu_mul_bf16x8_kernel, dim3((unsigned)((work8 + 255) / 256)), dim3(256), 0, s,
                       (const bf16_t*)gate_up, (bf16_t*)out, inner, work8, interleaved);
    QIL_RETURN_LAUNCH_STATUS();
  }
  const bool vec = inner % 4 == 0 && (((uintptr_t)gate_up | (uintptr_t)out) % 16 == 0);
  const size_t work = vec ? total / 4 : total;
  const unsigned blocks = (unsigned)((work + 255) / 256);
#define QIL_SILU_CASE(TD, T)                                                                                          \
  do {                                                                                                                \
    if (vec)                                                                                                          \
      hipLaunchKernelGGL((silu_mul_vec_kernel<TD, T>), dim3(blocks), dim3(256), 0, s, (const TD*)gate_up, splits,      \
                         stride, (T*)out, inner, work, interleaved);                                                  \
    else                                                                                                              \
      hipLaunchKernelGGL((silu_mul_kernel<TD, T>), dim3(blocks), dim3(256), 0, s, (const TD*)gate_up, splits, stride,  \
                         (T*)out, inner, total, interleaved);                                                         \
  } while (0)
  if (out_dtype == QIL_F32) {
    if (in_dtype != QIL_F32) return -1;
    QIL_SILU_CASE(float, float);
  } else if (in_dtype == QIL_F32) {
    QIL_SILU_CASE(float, bf16_t);
  } else {
    QIL_SILU_CASE(bf16_t, bf16_t);
  }
#undef QIL_SILU_CASE
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
