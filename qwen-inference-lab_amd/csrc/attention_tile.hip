// Attention of prompt portions (sequences with two or more rows in the step) over the paged cache,
// flash style on the matrix cores: no score matrix in memory, float32 online softmax.
//
// Block = 4 waves sharing one kv head and one range of keys; each wave owns a 16-row tile of one
// query head.  With g = heads / kv_heads query heads per kv head, a block covers GH = min(g, 4)
// heads (4 if g >= 3) and 4 / GH row tiles, so K and V tiles are staged in LDS once for the whole
// group (qil/model.py:59-61 expands them per query head instead).  Grid: (row tiles of the
// longest sequence, sequences, kv_heads * head chunks); blocks past a sequence's rows and
// sequences with a single row (the row kernel's) return at once.
//
// A row at absolute position p sees key j iff j <= p, and j > p - window with a window
// (qil/model.py:62-64).  Keys at or beyond the block's last position + 1 are never loaded: they
// are not written yet or belong to nobody; their LDS slots are zero so that 0 * garbage cannot
// make a NaN.
//
// Matrix-core formulation (wave64, 16x16 tiles).  Scores are computed transposed,
//   S^T[key, row] = sum_dim K[key, dim] Q[row, dim]        A = K tile (LDS), B = Q (registers)
// so that a lane ends up with the scores of ONE row (row = lane % 16) for keys 4 (lane / 16) + i:
// maxima, sums and rescaling are per-lane scalars, reduced over the 4 lane groups by two
// shuffles.  The same registers are then the B operand of
//   O^T[dim, row] = sum_key V^T[dim, key] P^T[key, row]    A = V tile transposed in LDS
// bfloat16 uses v_mfma_f32_16x16x32_bf16 (P rounded to bfloat16, float32 accumulation); float32
// uses v_mfma_f32_16x16x4_f32: float32 inputs and products, no reduced-precision mode.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define TILE_THREADS 256

template <typename T> struct TileTraits;
template <> struct TileTraits<bf16_t> {
  static constexpr int BK = 64;        // keys per LDS tile
  static constexpr int KSTEP = 32;     // dims per score MFMA
  static constexpr int PAD = 8;        // LDS row padding in elements
};
template <> struct TileTraits<float> {
  static constexpr int BK = 32;
  static constexpr int KSTEP = 4;
  static constexpr int PAD = 4;
};

__device__ __forceinline__ float softmax_exp(float x, bf16_t) { return __builtin_amdgcn_exp2f(x * 1.44269504088896f); }
__device__ __forceinline__ float softmax_exp(float x, float) { return expf(x); }

template <typename T, int DMAX>
__global__ void __launch_bounds__(TILE_THREADS)
attn_tile_kernel(const T* __restrict__ q, int q_stride, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                 const int* __restrict__ block_tables, int table_stride, const int* __restrict__ cu_seqlens,
                 const int* __restrict__ seq_starts, T* __restrict__ out, int heads, int kv_heads, int d,
                 int page_size, int window, float scale, int GH, int chunks) {
  using TT = TileTraits<T>;
  constexpr int BK = TT::BK, KSTEP = TT::KSTEP, PAD = TT::PAD;
  constexpr bool BF16 = sizeof(T) == 2;
  constexpr int QFRAGS = DMAX / KSTEP;          // score MFMA steps over the head dim
  constexpr int DTILES = DMAX / 16;             // output dim tiles
  constexpr int SUB = BK / 16;                  // 16-key sub-tiles per LDS tile
  extern __shared__ __align__(16) unsigned char lds_raw[];

  const int seq = blockIdx.y;
  const int q0 = cu_seqlens[seq], n = cu_seqlens[seq + 1] - q0;
  if (n < 2) return;
  const int RT = 4 / GH;
  const int tile_row0 = blockIdx.x * 16 * RT;
  if (tile_row0 >= n) return;
  const int kvh = blockIdx.z / chunks, chunk = blockIdx.z % chunks;
  const int g = heads / kv_heads;
  const int lane = threadIdx.x & (QIL_WAVE - 1), wave = threadIdx.x / QIL_WAVE;
  const int r = lane & 15, kb = lane >> 4;
  const int head_local = chunk * GH + wave % GH, row_tile = wave / GH;
  const bool wave_active = head_local < g && tile_row0 + row_tile * 16 < n;
  const int head = kvh * g + head_local;
  const int start = seq_starts[seq];

  const int rows_in_block = min(16 * RT, n - tile_row0);
  const int pos_first = start + tile_row0;
  const int key_end = pos_first + rows_in_block;                       // last position + 1
  const int key_begin = window > 0 ? max(0, pos_first - window + 1) : 0;

  const int dt = (d + 15) / 16;                        // dim tiles in use
  const int k_row = (BF16 ? (d + 31) / 32 * 32 : dt * 16) + PAD;       // elements per K row in LDS (staging
                                                                       // writes whole dim tiles)
  const int v_row = BK + PAD;                                          // elements per V^T row in LDS
  T* Ks = reinterpret_cast<T*>(lds_raw);                               // [BK][k_row]
  T* Vt = Ks + BK * k_row;                                             // [dt * 16][v_row]

  const int my_row = tile_row0 + row_tile * 16 + r;
  const bool row_valid = wave_active && my_row < n;
  const int my_pos = start + my_row;
  const int* table = block_tables + (size_t)seq * table_stride;

  // ---- Q fragments: B operand, Q[row r][dims of this lane's k slots]
  bf16x8 qb[BF16 ? QFRAGS : 1];
  float qf[BF16 ? 1 : QFRAGS];
  {
    const T* qrow = q + (size_t)(q0 + (row_valid ? my_row : 0)) * q_stride + (size_t)(wave_active ? head : 0) * d;
    if constexpr (BF16) {
#pragma unroll
      for (int ks = 0; ks < QFRAGS; ++ks) {
        const int dim = ks * 32 + kb * 8;
        uint4 raw = make_uint4(0, 0, 0, 0);
        if (row_valid && dim < d) raw = *reinterpret_cast<const uint4*>(qrow + dim);
        qb[ks] = __builtin_bit_cast(bf16x8, raw);
      }
    } else {
#pragma unroll
      for (int ks = 0; ks < QFRAGS; ++ks) {
        const int dim = ks * 4 + kb;
        qf[ks] = (row_valid && dim < d) ? qrow[dim] : 0.f;
      }
    }
  }

  float m = -INFINITY, l = 0.f;
  f32x4 o[DTILES];
#pragma unroll
  for (int t = 0; t < DTILES; ++t) o[t] = (f32x4){0.f, 0.f, 0.f, 0.f};

  const int vec_per_key = (dt * 16) / 8;               // 8-element vectors per key covering the dim tiles
  for (int k0 = key_begin / BK * BK; k0 < key_end; k0 += BK) {
    __syncthreads();                                   // the previous tile is consumed
    // ---- stage K (row major) and V (transposed) of keys [k0, k0 + BK)
    for (int idx = threadIdx.x; idx < BK * vec_per_key; idx += TILE_THREADS) {
      const int kl = idx / vec_per_key, dv = (idx - kl * vec_per_key) * 8;
      const int key = k0 + kl;
      const bool valid = key >= key_begin && key < key_end && dv < d;
      T* kdst = Ks + kl * k_row + dv;
      if constexpr (BF16) {
        uint4 kraw = make_uint4(0, 0, 0, 0), vraw = make_uint4(0, 0, 0, 0);
        if (valid) {
          const size_t page = table[key / page_size];
          const size_t base = ((page * kv_heads + kvh) * page_size + (key % page_size)) * (size_t)d + dv;
          kraw = *reinterpret_cast<const uint4*>(k_cache + base);
          const bf16_t* column = v_cache + ((page * kv_heads + kvh) * (size_t)d + dv) * page_size + (key % page_size);
          uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
          for (int e = 0; e < 8; ++e) w[e >> 1] |= (uint32_t)column[(size_t)e * page_size] << ((e & 1) * 16);
          vraw = make_uint4(w[0], w[1], w[2], w[3]);
        }
        *reinterpret_cast<uint4*>(kdst) = kraw;
        const uint32_t w[4] = {vraw.x, vraw.y, vraw.z, vraw.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) Vt[(dv + e) * v_row + kl] = (bf16_t)(w[e >> 1] >> ((e & 1) * 16));
      } else {
        float kv8[8], vv8[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) { kv8[e] = 0.f; vv8[e] = 0.f; }
        if (valid) {
          const size_t page = table[key / page_size];
          const size_t base = ((page * kv_heads + kvh) * page_size + (key % page_size)) * (size_t)d + dv;
          ld8(k_cache + base, kv8);
          const float* column = v_cache + ((page * kv_heads + kvh) * (size_t)d + dv) * page_size + (key % page_size);
#pragma unroll
          for (int e = 0; e < 8; ++e) vv8[e] = column[(size_t)e * page_size];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) { kdst[e] = kv8[e]; Vt[(dv + e) * v_row + kl] = vv8[e]; }
      }
    }
    if constexpr (BF16) {
      // K rows are read in steps of 32 dims: zero the tail between the dim tiles and the padded width
      const int tail0 = dt * 16, tail = (d + 31) / 32 * 32 - tail0;
      if (tail > 0)
        for (int idx = threadIdx.x; idx < BK * tail; idx += TILE_THREADS)
          Ks[(idx / tail) * k_row + tail0 + idx % tail] = 0;
    }
    __syncthreads();
    if (!wave_active) continue;

    // ---- S^T = K Q^T for the tile's 16-key sub-tiles
    f32x4 s[SUB];
#pragma unroll
    for (int jt = 0; jt < SUB; ++jt) {
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
      const T* krow = Ks + (jt * 16 + r) * k_row;
      if constexpr (BF16) {
#pragma unroll
        for (int ks = 0; ks < QFRAGS; ++ks) {
          if (ks * 32 < d) {
            const bf16x8 a = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(krow + ks * 32 + kb * 8));
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qb[ks], acc, 0, 0, 0);
          }
        }
      } else {
#pragma unroll
        for (int ks = 0; ks < QFRAGS; ++ks)
          if (ks * 4 < d) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(krow[ks * 4 + kb], qf[ks], acc, 0, 0, 0);
      }
      s[jt] = acc;
    }
    // ---- mask, scale, online softmax (per-lane row statistics)
    float mx = -INFINITY;
#pragma unroll
    for (int jt = 0; jt < SUB; ++jt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = k0 + jt * 16 + 4 * kb + i;
        const bool visible = row_valid && key <= my_pos && (window <= 0 || key > my_pos - window);
        const float v = visible ? s[jt][i] * scale : -INFINITY;
        s[jt][i] = v;
        mx = fmaxf(mx, v);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, QIL_WAVE));
    mx = fmaxf(mx, __shfl_xor(mx, 32, QIL_WAVE));
    const float m_new = fmaxf(m, mx);
    const float alpha = (m_new == -INFINITY) ? 1.f : softmax_exp(m - m_new, T());   // m = -inf gives 0
    float psum = 0.f;
#pragma unroll
    for (int jt = 0; jt < SUB; ++jt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = (s[jt][i] == -INFINITY) ? 0.f : softmax_exp(s[jt][i] - m_new, T());
        s[jt][i] = p;
        psum += p;
      }
    l = l * alpha + psum;
    m = m_new;
#pragma unroll
    for (int t = 0; t < DTILES; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) o[t][i] *= alpha;

    // ---- O^T += V^T P^T
    if constexpr (BF16) {
#pragma unroll
      for (int st = 0; st < SUB / 2; ++st) {
        uint32_t packed[4];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          packed[i] = (uint32_t)f32_to_bf16(s[2 * st][2 * i]) | ((uint32_t)f32_to_bf16(s[2 * st][2 * i + 1]) << 16);
          packed[2 + i] = (uint32_t)f32_to_bf16(s[2 * st + 1][2 * i]) |
                          ((uint32_t)f32_to_bf16(s[2 * st + 1][2 * i + 1]) << 16);
        }
        const bf16x8 b = __builtin_bit_cast(bf16x8, make_uint4(packed[0], packed[1], packed[2], packed[3]));
#pragma unroll
        for (int t = 0; t < DTILES; ++t) {
          if (t < dt) {
            const T* vrow = Vt + (t * 16 + r) * v_row + st * 32 + 4 * kb;
            const uint2 lo = *reinterpret_cast<const uint2*>(vrow);
            const uint2 hi = *reinterpret_cast<const uint2*>(vrow + 16);
            const bf16x8 a = __builtin_bit_cast(bf16x8, make_uint4(lo.x, lo.y, hi.x, hi.y));
            o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, o[t], 0, 0, 0);
          }
        }
      }
    } else {
#pragma unroll
      for (int jt = 0; jt < SUB; ++jt)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int t = 0; t < DTILES; ++t)
            if (t < dt)
              o[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(Vt[(t * 16 + r) * v_row + jt * 16 + 4 * kb + i], s[jt][i],
                                                          o[t], 0, 0, 0);
    }
  }

  if (!wave_active) return;
  l += __shfl_xor(l, 16, QIL_WAVE);
  l += __shfl_xor(l, 32, QIL_WAVE);
  if (!row_valid) return;
  const float inv = 1.f / l;
  T* orow = out + ((size_t)(q0 + my_row) * heads + head) * d;
#pragma unroll
  for (int t = 0; t < DTILES; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int dim = t * 16 + 4 * kb + i;
      if (dim < d) st(orow + dim, o[t][i] * inv);
    }
}

template <typename T, int DMAX>
static int launch_tile(const void* q, int q_stride, const void* k_cache, const void* v_cache, const int* block_tables,
                       int table_stride, const int* cu_seqlens, const int* seq_starts, void* out, int n_seqs,
                       int max_query, int heads, int kv_heads, int d, int page_size, int window, float scale,
                       hipStream_t s) {
  using TT = TileTraits<T>;
  const int g = heads / kv_heads;
  const int GH = g >= 3 ? 4 : g, chunks = (g + GH - 1) / GH, RT = 4 / GH;
  const bool bf16 = sizeof(T) == 2;
  const int k_row = (bf16 ? (d + 31) / 32 * 32 : (d + 15) / 16 * 16) + TT::PAD, v_row = TT::BK + TT::PAD;
  const size_t lds = ((size_t)TT::BK * k_row + (size_t)((d + 15) / 16 * 16) * v_row) * sizeof(T);
  auto kernel = attn_tile_kernel<T, DMAX>;
  static size_t granted = 0;                     // per instantiation
  if (lds > 64 * 1024 && lds > granted) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
    granted = lds;
  }
  dim3 grid((max_query + 16 * RT - 1) / (16 * RT), n_seqs, kv_heads * chunks);
  hipLaunchKernelGGL(kernel, grid, dim3(TILE_THREADS), lds, s, (const T*)q, q_stride, (const T*)k_cache,
                     (const T*)v_cache, block_tables, table_stride, cu_seqlens, seq_starts, (T*)out, heads, kv_heads, d,
                     page_size, window, scale, GH, chunks);
  return (int)hipGetLastError();
}

// Sequences with >= 2 rows.  q: rows of stride q_stride, head h at h * d; out [rows, heads * d].
// Requires d % 8 == 0, 8 <= d <= 256.  Returns -1 on a size it does not take.
extern "C" int qil_attn_tile(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                             const int* block_tables, int table_stride, const int* cu_seqlens, const int* seq_starts,
                             void* out, int n_seqs, int max_query, int heads, int kv_heads, int d, int page_size,
                             int window, float scale, int dtype, hipStream_t s) {
  if (n_seqs == 0 || max_query < 2) return 0;
  if (d % 8 || d < 8 || d > 256 || heads % kv_heads || n_seqs > 65535 || kv_heads * 2 > 65535) return -1;
#define QIL_TILE_CASE(T, DMAX)                                                                                      \
  return launch_tile<T, DMAX>(q, q_stride, k_cache, v_cache, block_tables, table_stride, cu_seqlens, seq_starts, out, \
                              n_seqs, max_query, heads, kv_heads, d, page_size, window, scale, s)
  if (dtype == QIL_F32) {
    if (d <= 64) QIL_TILE_CASE(float, 64);
    if (d <= 128) QIL_TILE_CASE(float, 128);
    QIL_TILE_CASE(float, 256);
  }
  if (d <= 64) QIL_TILE_CASE(bf16_t, 64);
  if (d <= 128) QIL_TILE_CASE(bf16_t, 128);
  QIL_TILE_CASE(bf16_t, 256);
#undef QIL_TILE_CASE
}
