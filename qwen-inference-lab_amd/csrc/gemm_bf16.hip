// bfloat16 matrix product on the matrix cores for few rows (decode, selected logit rows):
//   C[M, N] = A[M, K] W[N, K]^T (+ bias[N]),  float32 accumulation.
// Both operands have K contiguous (qil/model.py:32-40).  The product is bound by streaming W once
// from HBM; A is small and would be re-read from L2 by every block, so the work is cut into wide,
// short pieces: a block owns 128 * NT rows of W (8 waves, each 16 * NT rows) and ONE of `splits`
// ranges of K.  It stages its slice of A in LDS once, then every wave streams its rows of W from
// global memory straight into v_mfma_f32_16x16x32_bf16 operands, loading UNROLL k steps ahead of
// the first product that uses them.  A's traffic is M / (128 NT) of W's.
//
// With splits > 1 a block writes a float32 partial result C[split, M, N], and the kernel that
// consumes the product (norm, rotary/store, SiLU gate) adds the partials in split order, so
// every sum is made in a fixed order.  With splits == 1 the result may be rounded to bfloat16
// here and take the bias.
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

#define GEMM_WAVES 8
#define GEMM_LDS_PAD 8          // bf16 elements between rows of the staged A slice

// chunk: k columns of A staged at a time (a multiple of 32); the block's range is walked in chunks.
template <int MT, int NT, int UNROLL, bool ALIGNED, typename OUT>
__global__ void __launch_bounds__(GEMM_WAVES * QIL_WAVE)
gemm_bf16_stream_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, const float* __restrict__ bias,
                        OUT* __restrict__ C, int M, int N, int K, int steps_per_split, int chunk) {
  extern __shared__ __align__(16) bf16_t a_lds[];          // [16 MT][chunk + pad]
  const int lane = threadIdx.x & (QIL_WAVE - 1), wave = threadIdx.x / QIL_WAVE;
  const int r = lane & 15, kb = lane >> 4;
  const int n0 = (blockIdx.x * GEMM_WAVES + wave) * 16 * NT, m0 = blockIdx.y * 16 * MT, split = blockIdx.z;
  const int row_width = chunk + GEMM_LDS_PAD;

  f32x4 acc[MT][NT];
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int j = 0; j < NT; ++j) acc[t][j] = (f32x4){0.f, 0.f, 0.f, 0.f};

  const int k_begin = split * steps_per_split * 32, k_end = min(K, k_begin + steps_per_split * 32);
  // W fragments of the next UNROLL k steps are always in flight: the first group is requested before A
  // is even staged, and each later group before the products of the group in hand.  Two register
  // buffers take turns; the loop is written out in pairs so that each is indexed statically.
  uint4 b0[UNROLL][NT], b1[UNROLL][NT];
  auto request = [&](uint4 (&b)[UNROLL][NT], int k0) {     // k steps starting at column k0
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int k = k0 + u * 32 + kb * 8;
#pragma unroll
      for (int j = 0; j < NT; ++j) b[u][j] = load_frag<ALIGNED>(W, n0 + j * 16 + r, N, k < k_end ? k : K, K);
    }
  };
  auto multiply = [&](const uint4 (&b)[UNROLL][NT], int step, int steps) {
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      if (step + u < steps) {
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          const uint4 a = *reinterpret_cast<const uint4*>(a_lds + (t * 16 + r) * row_width + (step + u) * 32 + kb * 8);
#pragma unroll
          for (int j = 0; j < NT; ++j)
            acc[t][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                                __builtin_bit_cast(bf16x8, b[u][j]), acc[t][j], 0, 0, 0);
        }
      }
    }
  };
  request(b0, k_begin);
  for (int kc = k_begin; kc < k_end; kc += chunk) {          // chunk is a multiple of 64 * UNROLL columns
    const int width = min(chunk, k_end - kc);               // columns of this chunk (last one may be short)
    __syncthreads();                                        // the previous chunk is consumed
    for (int idx = threadIdx.x; idx < 16 * MT * (chunk / 8); idx += GEMM_WAVES * QIL_WAVE) {
      const int m = idx / (chunk / 8), c = (idx - m * (chunk / 8)) * 8;
      const uint4 v = c < width ? load_frag<ALIGNED>(A, m0 + m, M, kc + c, K) : make_uint4(0, 0, 0, 0);
      *reinterpret_cast<uint4*>(a_lds + m * row_width + c) = v;
    }
    __syncthreads();
    const int steps = (width + 31) / 32;
    for (int step = 0; step < steps; step += 2 * UNROLL) {
      request(b1, kc + (step + UNROLL) * 32);               // past k_end a request loads nothing
      multiply(b0, step, steps);
      request(b0, kc + (step + 2 * UNROLL) * 32);           // may be the first group of the next chunk
      multiply(b1, step + UNROLL, steps);
    }
  }
  // lane holds D[m = 4 kb + i][n = r] of each tile
  OUT* out = C + (size_t)split * M * N;
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int m = m0 + t * 16 + 4 * kb + i, n = n0 + j * 16 + r;
        if (m < M && n < N) store_out(out + (size_t)m * N + n, acc[t][j][i] + (bias ? bias[n] : 0.f));
      }
}

template <int MT, int NT, int UNROLL, typename OUT>
static int launch_stream(const bf16_t* A, const bf16_t* W, const float* bias, OUT* C, int M, int N, int K, int splits,
                         int chunk, hipStream_t s) {
  const int steps = (K + 31) / 32;
  const int steps_per_split = (steps + splits - 1) / splits;
  const int grain = 64 * UNROLL;                                         // the k loop runs in pairs of UNROLL steps
  if (chunk <= 0 || chunk > steps_per_split * 32) chunk = steps_per_split * 32;
  chunk = (chunk + grain - 1) / grain * grain;
  const size_t cap = 64 * 1024 / (16 * MT * sizeof(bf16_t));             // elements per row that fit 64 KB
  if ((size_t)chunk + GEMM_LDS_PAD > cap) chunk = (int)((cap - GEMM_LDS_PAD) / grain * grain);
  if (chunk < grain) return -1;
  const size_t lds = (size_t)16 * MT * (chunk + GEMM_LDS_PAD) * sizeof(bf16_t);
  dim3 grid((N + 128 * NT - 1) / (128 * NT), (M + 16 * MT - 1) / (16 * MT), splits);
  const bool aligned = (K % 8 == 0) && (((uintptr_t)A | (uintptr_t)W) % 16 == 0);
  if (aligned)
    hipLaunchKernelGGL((gemm_bf16_stream_kernel<MT, NT, UNROLL, true, OUT>), grid, dim3(GEMM_WAVES * QIL_WAVE), lds, s,
                       A, W, bias, C, M, N, K, steps_per_split, chunk);
  else
    hipLaunchKernelGGL((gemm_bf16_stream_kernel<MT, NT, UNROLL, false, OUT>), grid, dim3(GEMM_WAVES * QIL_WAVE), lds, s,
                       A, W, bias, C, M, N, K, steps_per_split, chunk);
  return 0;
}

// Shapes of the kernel that exist: code = MT * 100 + NT * 10 + UNROLL.
#define QIL_GEMM_SHAPES(X) \
  X(1, 1, 4) X(1, 1, 8) X(1, 2, 4) X(1, 2, 8) X(1, 4, 4) X(2, 1, 4) X(2, 1, 8) X(2, 2, 4) X(4, 1, 4) X(4, 1, 8) \
  X(4, 2, 4) X(4, 2, 2)

template <typename OUT>
static int launch_shape(int code, const bf16_t* A, const bf16_t* W, const float* bias, OUT* C, int M, int N, int K,
                        int splits, int chunk, hipStream_t s) {
#define X(MT, NT, UNROLL) \
  if (code == MT * 100 + NT * 10 + UNROLL) return launch_stream<MT, NT, UNROLL, OUT>(A, W, bias, C, M, N, K, splits, chunk, s);
  QIL_GEMM_SHAPES(X)
#undef X
  return -1;
}

// The plan for a product: kernel shape code and the number of K splits.
static void plan(int M, int N, int K, bool may_split, int* code, int* splits) {
  const int steps = (K + 31) / 32;
  const int mt = M <= 16 ? 1 : M <= 32 ? 2 : 4;
  const int column_blocks = (N + 127) / 128;
  int sp = 1;
  if (may_split) {
    // about three blocks per CU (256 CUs), at least 8 k steps per split, fewer splits for more rows
    const int most = 8;                                   // the consumer reads every partial
    sp = (768 + column_blocks - 1) / column_blocks;
    if (sp > most) sp = most;
    while (sp > 1 && steps / sp < 8) --sp;
    if (sp < 1) sp = 1;
  }
  *code = mt * 100 + 10 + 4;
  *splits = sp;
}

// How many ways the product will be split over K when partial sums are allowed.
extern "C" int qil_gemm_bf16_splits(int M, int N, int K) {
  int code, splits;
  plan(M, N, K, true, &code, &splits);
  return splits;
}

// out_dtype QIL_BF16: C bfloat16 [M, N], splits must be 1.  QIL_F32: C float32 [splits, M, N], the
// value being the sum over the first axis; bias (if any) requires splits == 1.
// shape: 0 = chosen here, else a code of QIL_GEMM_SHAPES; chunk: 0 = chosen here (tuning runs set both).
extern "C" int qil_gemm_bf16(const void* A, const void* W, const float* bias, void* C, int M, int N, int K,
                             int out_dtype, int splits, int shape, int chunk, hipStream_t s) {
  if (M == 0 || N == 0) return 0;
  if (K < 1 || splits < 1 || splits > 65535 || (splits > 1 && (out_dtype != QIL_F32 || bias))) return -1;
  int code = shape, planned;
  if (!code) plan(M, N, K, false, &code, &planned);
  int status;
  if (out_dtype == QIL_F32)
    status = launch_shape<float>(code, (const bf16_t*)A, (const bf16_t*)W, bias, (float*)C, M, N, K, splits, chunk, s);
  else
    status = launch_shape<bf16_t>(code, (const bf16_t*)A, (const bf16_t*)W, bias, (bf16_t*)C, M, N, K, splits, chunk, s);
  if (status) return status;
  QIL_RETURN_LAUNCH_STATUS();
}
