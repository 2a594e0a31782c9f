// Fused per-head RMSNorm of q and k, rotary encoding, and the write of k and v into the pages.
//
// qkv[N, (heads + 2 kv_heads) * d]: head h of q at columns [h d, (h+1) d), then the k heads, then the
// v heads.  One wave per (token, head).  All arithmetic is float32 and a value is rounded to T once,
// when it is stored (the reference rounds after the norm, of cos and sin, and after every product:
// qil/model.py:15-23,42-46,52-55).
//   q heads: norm -> rotate -> stored back in place
//   k heads: norm -> rotate -> stored into k_cache at the token's slot
//   v heads: copied into v_cache at the token's slot
// Cache layout [pages, kv_heads, page_size, d]; slot = page * page_size + offset (qil/cache.py:79-82).
// Rotation pairs (i, i + rot/2), i < rot/2 (qil/model.py:42-46); elements from rot on pass unrotated.
#include "common.h"

#define QIL_MAX_HEAD_DIM 512

template <typename T>
__global__ void qk_norm_rope_store_kernel(
    T* __restrict__ qkv, const float* __restrict__ q_weight, const float* __restrict__ k_weight,
    const float* __restrict__ cos_table, const float* __restrict__ sin_table, const int* __restrict__ positions,
    const int* __restrict__ slots, T* __restrict__ k_cache, T* __restrict__ v_cache,
    int heads, int kv_heads, int d, int rot, int page_size, float eps) {
  __shared__ float vec[QIL_MAX_HEAD_DIM];
  const int n = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int total_heads = heads + 2 * kv_heads;
  T* src = qkv + ((size_t)n * total_heads + head) * d;
  const bool is_q = head < heads, is_k = !is_q && head < heads + kv_heads;
  if (!is_q && slots == nullptr) return;                 // a reader of another entry's cache writes no k/v

  T* dst = src;
  if (!is_q) {
    const int kvh = is_k ? head - heads : head - heads - kv_heads;
    const int slot = slots[n];
    const size_t page = slot / page_size, offset = slot % page_size;
    dst = (is_k ? k_cache : v_cache) + ((page * kv_heads + kvh) * page_size + offset) * d;
  }
  if (!is_q && !is_k) {                                  // v: plain copy
    for (int i = lane; i < d; i += QIL_WAVE) dst[i] = src[i];
    return;
  }

  const float* weight = is_q ? q_weight : k_weight;
  float sum = 0.f;
  for (int i = lane; i < d; i += QIL_WAVE) {
    const float v = ld(src + i);
    vec[i] = v;
    sum += v * v;
  }
  if (weight) {
    sum = wave_sum(sum);
    const float rstd = rsqrtf(sum / (float)d + eps);
    for (int i = lane; i < d; i += QIL_WAVE) vec[i] = round_to<T>(vec[i] * rstd) * weight[i];
  }
  __syncthreads();
  const int half = rot / 2;
  const float* c = cos_table ? cos_table + (size_t)positions[n] * half : nullptr;
  const float* s = sin_table ? sin_table + (size_t)positions[n] * half : nullptr;
  for (int i = lane; i < d; i += QIL_WAVE) {
    float v = vec[i];
    if (c && i < rot) {
      if (i < half) v = vec[i] * c[i] - vec[i + half] * s[i];
      else          v = vec[i - half] * s[i - half] + vec[i] * c[i - half];
    }
    st(dst + i, v);
  }
}

extern "C" int qil_qk_norm_rope_store(
    void* qkv, const float* q_weight, const float* k_weight, const float* cos_table, const float* sin_table,
    const int* positions, const int* slots, void* k_cache, void* v_cache, int n, int heads, int kv_heads,
    int d, int rot, int page_size, float eps, int dtype, hipStream_t s) {
  if (n == 0) return 0;
  if (d > QIL_MAX_HEAD_DIM || rot > d || (rot & 1)) return -1;
  dim3 grid(n, heads + 2 * kv_heads);
  if (dtype == QIL_F32)
    hipLaunchKernelGGL(qk_norm_rope_store_kernel<float>, grid, dim3(QIL_WAVE), 0, s, (float*)qkv, q_weight, k_weight,
                       cos_table, sin_table, positions, slots, (float*)k_cache, (float*)v_cache, heads, kv_heads, d,
                       rot, page_size, eps);
  else
    hipLaunchKernelGGL(qk_norm_rope_store_kernel<bf16_t>, grid, dim3(QIL_WAVE), 0, s, (bf16_t*)qkv, q_weight, k_weight,
                       cos_table, sin_table, positions, slots, (bf16_t*)k_cache, (bf16_t*)v_cache, heads, kv_heads, d,
                       rot, page_size, eps);
  QIL_RETURN_LAUNCH_STATUS();
}
