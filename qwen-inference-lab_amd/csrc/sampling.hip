// Next-token choice from float32 logits: greedy argmax or a seeded temperature draw.
//
// One block per row.  A row with a non-finite logit is flagged (the engine raises, as the reference
// does at qil/engine.py:96-99).  Greedy takes the largest logit, the lowest index on ties (what
// argmax returns, qil/engine.py:100).  With temperature T > 0 the draw is the Gumbel-max form of
// sampling from softmax(logits / T): argmax_i (logit_i / T - log(-log(u_i))), u_i a counter-based
// uniform in (0, 1) keyed by (seed, output index, i), so a request's draws depend neither on the
// batch it sits in nor on how its work was cut.
#include "common.h"

__device__ __forceinline__ uint32_t mix32(uint32_t x) {
  x ^= x >> 16; x *= 0x7feb352du;
  x ^= x >> 15; x *= 0x846ca68bu;
  x ^= x >> 16;
  return x;
}

__device__ __forceinline__ float gumbel(uint32_t seed, uint32_t counter, uint32_t i) {
  const uint32_t x = mix32(i * 0x9e3779b1u + seed * 0x85ebca77u + counter * 0xc2b2ae3du);
  const float u = ((float)(x >> 8) + 0.5f) * (1.0f / 16777216.0f);
  return -logf(-logf(u));
}

#define SAMPLE_THREADS 512

__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(const float* __restrict__ logits, const float* __restrict__ temperatures,
              const int* __restrict__ seeds, const int* __restrict__ counters, int* __restrict__ tokens,
              int* __restrict__ finite, int vocab) {
  __shared__ float best_value[SAMPLE_THREADS / QIL_WAVE];
  __shared__ int best_index[SAMPLE_THREADS / QIL_WAVE];
  __shared__ int bad[SAMPLE_THREADS / QIL_WAVE];
  const int row = blockIdx.x;
  const float* x = logits + (size_t)row * vocab;
  const float temperature = temperatures[row];
  const uint32_t seed = (uint32_t)seeds[row], counter = (uint32_t)counters[row];
  float value = -INFINITY;
  int index = 0x7fffffff, broken = 0;
  for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS) {
    const float v = x[i];
    if (!isfinite(v)) broken = 1;
    const float score = temperature > 0.f ? v / temperature + gumbel(seed, counter, (uint32_t)i) : v;
    if (score > value) { value = score; index = i; }          // strided ascending: first maximum kept
  }
  for (int o = QIL_WAVE / 2; o > 0; o >>= 1) {
    const float other = __shfl_xor(value, o, QIL_WAVE);
    const int other_index = __shfl_xor(index, o, QIL_WAVE);
    broken |= __shfl_xor(broken, o, QIL_WAVE);
    if (other > value || (other == value && other_index < index)) { value = other; index = other_index; }
  }
  const int lane = threadIdx.x & (QIL_WAVE - 1), wave = threadIdx.x / QIL_WAVE;
  if (lane == 0) { best_value[wave] = value; best_index[wave] = index; bad[wave] = broken; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < SAMPLE_THREADS / QIL_WAVE; ++w) {
      broken |= bad[w];
      if (best_value[w] > value || (best_value[w] == value && best_index[w] < index)) {
        value = best_value[w];
        index = best_index[w];
      }
    }
    tokens[row] = index == 0x7fffffff ? 0 : index;
    finite[row] = broken ? 0 : 1;
  }
}

extern "C" int qil_sample(const float* logits, const float* temperatures, const int* seeds, const int* counters,
                          int* tokens, int* finite, int rows, int vocab, hipStream_t s) {
  if (rows == 0) return 0;
  hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, s, logits, temperatures, seeds, counters,
                     tokens, finite, vocab);
  QIL_RETURN_LAUNCH_STATUS();
}
