// Next-token choice from float32 logits: greedy argmax or a seeded temperature draw.
//
// One block per row.  A row with a non-finite logit is flagged (the engine raises, as the reference
// does at qil/engine.py:96-99).  Greedy takes the largest logit, the lowest index on ties (what
// argmax returns, qil/engine.py:100).  With temperature T > 0 the draw is the Gumbel-max form of
// sampling from softmax(logits / T): argmax_i (logit_i / T - log(-log(u_i))), u_i a counter-based
// uniform in (0, 1) keyed by (seed, output index, i), so a request's draws depend neither on the
// batch it sits in nor on how its work was cut.
#include "common.h"
#include "sampling.h"
#include <mutex>

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

#define SAMPLE_THREADS 256
#define SAMPLE_CHUNK 4096          // vocabulary entries per first-stage block

struct Best { float value; int index; int broken; };

// Larger value wins; on equal values the lower index (argmax's tie rule, qil/engine.py:100).
__device__ __forceinline__ void take(Best& a, float value, int index) {
  if (value > a.value || (value == a.value && index < a.index)) { a.value = value; a.index = index; }
}

__device__ __forceinline__ Best block_best(Best mine, float* values, int* indices, int* bad) {
  for (int o = QIL_WAVE / 2; o > 0; o >>= 1) {
    const float v = __shfl_xor(mine.value, o, QIL_WAVE);
    const int i = __shfl_xor(mine.index, o, QIL_WAVE);
    mine.broken |= __shfl_xor(mine.broken, o, QIL_WAVE);
    take(mine, v, i);
  }
  const int lane = threadIdx.x & (QIL_WAVE - 1), wave = threadIdx.x / QIL_WAVE;
  if (lane == 0) { values[wave] = mine.value; indices[wave] = mine.index; bad[wave] = mine.broken; }
  __syncthreads();
  if (threadIdx.x == 0)
    for (int w = 1; w < (int)(blockDim.x / QIL_WAVE); ++w) {
      mine.broken |= bad[w];
      take(mine, values[w], indices[w]);
    }
  return mine;                       // complete in thread 0
}

// Stage 1: grid (chunks, rows).  Each block scans SAMPLE_CHUNK logits of one row.
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_scan_kernel(const float* __restrict__ logits, const float* __restrict__ temperatures,
                   const int* __restrict__ seeds, const int* __restrict__ counters, float* __restrict__ chunk_value,
                   int* __restrict__ chunk_index, int* __restrict__ chunk_bad, int vocab, int chunks) {
  __shared__ float values[SAMPLE_THREADS / QIL_WAVE];
  __shared__ int indices[SAMPLE_THREADS / QIL_WAVE], bad[SAMPLE_THREADS / QIL_WAVE];
  const int chunk = blockIdx.x, row = blockIdx.y;
  const float* x = logits + (size_t)row * vocab;
  const float temperature = temperatures[row];
  const uint32_t seed = (uint32_t)seeds[row], counter = (uint32_t)counters[row];
  Best mine = {-INFINITY, 0x7fffffff, 0};
  const int stop = min(vocab, (chunk + 1) * SAMPLE_CHUNK);
  for (int i = chunk * SAMPLE_CHUNK + threadIdx.x; i < stop; i += SAMPLE_THREADS) {
    const float v = x[i];
    if (!isfinite(v)) mine.broken = 1;
    take(mine, temperature > 0.f ? v / temperature + gumbel(seed, counter, (uint32_t)i) : v, i);
  }
  mine = block_best(mine, values, indices, bad);
  if (threadIdx.x == 0) {
    const size_t cell = (size_t)row * chunks + chunk;
    chunk_value[cell] = mine.value; chunk_index[cell] = mine.index; chunk_bad[cell] = mine.broken;
  }
}

// Stage 2: one block per row over the chunks' winners.
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_pick_kernel(const float* __restrict__ chunk_value, const int* __restrict__ chunk_index,
                   const int* __restrict__ chunk_bad, int* __restrict__ tokens, int* __restrict__ finite, int chunks) {
  __shared__ float values[SAMPLE_THREADS / QIL_WAVE];
  __shared__ int indices[SAMPLE_THREADS / QIL_WAVE], bad[SAMPLE_THREADS / QIL_WAVE];
  const int row = blockIdx.x;
  Best mine = {-INFINITY, 0x7fffffff, 0};
  for (int c = threadIdx.x; c < chunks; c += SAMPLE_THREADS) {
    const size_t cell = (size_t)row * chunks + c;
    mine.broken |= chunk_bad[cell];
    take(mine, chunk_value[cell], chunk_index[cell]);
  }
  mine = block_best(mine, values, indices, bad);
  if (threadIdx.x == 0) {
    tokens[row] = mine.index == 0x7fffffff ? 0 : mine.index;
    finite[row] = mine.broken ? 0 : 1;
  }
}

extern "C" {

// Bytes of scratch for `rows` rows: per chunk a value, an index and a flag.
size_t qil_sample_workspace(int rows, int vocab) {
  return (size_t)rows * ((vocab + SAMPLE_CHUNK - 1) / SAMPLE_CHUNK) * 12;
}

// The two launches of a draw over scratch memory that holds, per (row, chunk) cell, a value, an index and a flag.
static int launch_sample(const float* logits, const float* temperatures, const int* seeds, const int* counters,
                         int* tokens, int* finite, void* scratch_memory, int rows, int vocab, hipStream_t s) {
  const int chunks = (vocab + SAMPLE_CHUNK - 1) / SAMPLE_CHUNK;
  float* values = (float*)scratch_memory;
  int* indices = (int*)(values + (size_t)rows * chunks);
  int* bad = indices + (size_t)rows * chunks;
  hipLaunchKernelGGL(sample_scan_kernel, dim3(chunks, rows), dim3(SAMPLE_THREADS), 0, s, logits, temperatures, seeds,
                     counters, values, indices, bad, vocab, chunks);
  hipLaunchKernelGGL(sample_pick_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, s, values, indices, bad, tokens, finite,
                     chunks);
  QIL_RETURN_LAUNCH_STATUS();
}

int qil_sample(const float* logits, const float* temperatures, const int* seeds, const int* counters, int* tokens,
               int* finite, void* workspace, int rows, int vocab, hipStream_t s) {
  if (rows == 0) return 0;
  if (rows > 65535) return -1;
  return launch_sample(logits, temperatures, seeds, counters, tokens, finite, workspace, rows, vocab, s);
}

}  // extern "C"

// ---------------------------------------------------------------------------------- the variant that allocates nothing
// Scratch memory of qil_sample_static.  In host code this name is only a handle for hipGetSymbolAddress, never a
// device address: the kernels get the looked-up address of the current device's copy.
static __device__ __align__(256) unsigned char scratch[(size_t)QIL_SAMPLE_STATIC_CELLS * 12];

#define QIL_MAX_DEVICES 64
static void* scratch_address[QIL_MAX_DEVICES];     // per device: where its copy of `scratch` lies (null: not looked up)
static std::mutex scratch_lock;

// The current device's copy of `scratch` (looked up once per device, with that device current); 0 or a HIP error.
static int scratch_of_current_device(void** address) {
  int device = -1;
  hipError_t status = hipGetDevice(&device);
  if (status != hipSuccess) return (int)status;
  if (device < 0 || device >= QIL_MAX_DEVICES) return (int)hipErrorInvalidDevice;
  std::lock_guard<std::mutex> guard(scratch_lock);
  if (scratch_address[device] == nullptr) {
    void* found = nullptr;
    status = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
    if (status != hipSuccess) return (int)status;
    if (found == nullptr) return (int)hipErrorInvalidSymbol;
    scratch_address[device] = found;
  }
  *address = scratch_address[device];
  return 0;
}

extern "C" {

int qil_sample_static_prepare(void) {
  void* address = nullptr;
  return scratch_of_current_device(&address);
}

int qil_sample_static(const float* logits, const float* temperatures, const int* seeds, const int* counters,
                      int* tokens, int* finite, int rows, int vocab, hipStream_t s) {
  if (rows == 0) return 0;
  if (rows < 0 || vocab < 1 || rows > 65535) return -1;
  const long long chunks = ((long long)vocab + SAMPLE_CHUNK - 1) / SAMPLE_CHUNK;
  if ((long long)rows * chunks > QIL_SAMPLE_STATIC_CELLS) return -2;
  void* address = nullptr;
  const int status = scratch_of_current_device(&address);
  if (status) return status;
  return launch_sample(logits, temperatures, seeds, counters, tokens, finite, address, rows, vocab, s);
}

}  // extern "C"
