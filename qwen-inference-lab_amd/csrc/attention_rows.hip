// Split-context attention of single query rows over the paged cache, and the merge of the splits.
//
// Every token of the step is a row with its own visible range of keys:
//   [lo, ctx) with ctx = position + 1, lo = window > 0 ? max(0, ctx - window) : 0
// (key j visible iff j <= position, qil/model.py:62-64).  A decoded token is one row; the tokens of a
// prompt portion are rows sharing a block table, whose keys were written before this kernel runs.
//
// Partial kernel: grid (rows, kv_heads, parts), 256 threads.  A block owns the keys
// [part * P, (part + 1) * P) of one row and one kv head and serves the whole group of query heads
// that read this kv head (h // g, qil/model.py:59-61), so K and V are read once per group rather
// than once per query head (the reference's kernel reads them per query head:
// qil/paged_attention.py:13-41).  Scores, maxima, exponentials, sums and weighted values are
// float32 (qil/paged_attention.py:27-41).  A block whose range is empty returns without writing,
// and the merge skips the same parts (qil/paged_attention.py:33-34 handles it with a safe maximum).
// With a single part the normalised result is written directly.
//
// Merge kernel: grid (rows, heads): out = sum_p acc_p exp(m_p - m) / sum_p l_p exp(m_p - m)
// (qil/paged_attention.py:44-58).
//
// Lanes: a token's d elements are spread over TG = next_pow2(ceil(d / 8)) lanes, eight elements a
// lane; a wave handles 64 / TG tokens at a time.
#include "common.h"

#define ATT_THREADS 256
#define ATT_WAVES (ATT_THREADS / QIL_WAVE)

// The sum of every 16 consecutive lanes, in their first lane (all lanes get a sum of the 16 values; the order of the
// additions is the first lane's in every group).  Four data-parallel moves: neighbours, pairs, fours mirrored in
// a half row, eights mirrored in the row.
__device__ __forceinline__ float row16_sum(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));
  return v;
}

// The sum of every aligned group of 2^log2 consecutive lanes (up to 32), in all of its lanes: the same moves, as
// many as the group needs, and one exchange between the two rows of 16 for groups of 32.
__device__ __forceinline__ float group_sum(float v, int log2) {
  if (log2 >= 1) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
  if (log2 >= 2) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
  if (log2 >= 3) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
  if (log2 >= 4) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));
  if (log2 >= 5) v += __shfl_xor(v, 16, QIL_WAVE);
  return v;
}

template <typename T, int GT>
__global__ void __launch_bounds__(ATT_THREADS)
attn_rows_partial_kernel(const T* __restrict__ q, int q_stride, const T* __restrict__ k_cache,
                         const T* __restrict__ v_cache, const int* __restrict__ block_tables, int table_stride,
                         const int* __restrict__ row_seq, const int* __restrict__ positions,
                         const int* __restrict__ row_index, float* __restrict__ part_acc,
                         float* __restrict__ part_m, float* __restrict__ part_l,
                         T* __restrict__ out, int heads, int kv_heads, int d, int page_size, int window,
                         float scale, int P, int parts, int tg_log2) {
  extern __shared__ float lds[];
  const int slot_row = blockIdx.x, kvh = blockIdx.y, part = blockIdx.z;   // slot_row indexes the workspace
  const int row = row_index ? row_index[slot_row] : slot_row;             // row of the step's batch
  const int g = heads / kv_heads;
  const int ctx = positions[row] + 1;
  const int lo = window > 0 ? max(0, ctx - window) : 0;
  const int begin = max(part * P, lo), end = min((part + 1) * P, ctx);
  if (begin >= end) return;
  const int count = end - begin;

  const int TG = 1 << tg_log2, TPW = QIL_WAVE >> tg_log2;
  const int lane = threadIdx.x & (QIL_WAVE - 1), wave = threadIdx.x / QIL_WAVE;
  const int sub = lane & (TG - 1), slot = lane >> tg_log2;   // slot: which token of the wave's group
  const int e0 = sub * 8;
  const bool live = e0 < d;                       // lanes past d (padding of TG to a power of two) idle
  const int* table = block_tables + (size_t)row_seq[row] * table_stride;

  float* scores = lds;                            // [GT][P]
  float* reduce = lds + GT * P;                   // [2][ATT_WAVES][GT] the waves' maxima and sums
  float* wave_acc = reduce + 64;                  // [ATT_WAVES][GT][d]

  for (int h0 = 0; h0 < g; h0 += GT) {
    // ---- scores of this head tile against the block's keys
    float qv[GT][8];
#pragma unroll
    for (int h = 0; h < GT; ++h) {
      const int head = kvh * g + h0 + h;
      if (live && h0 + h < g) ld8(q + (size_t)row * q_stride + (size_t)head * d + e0, qv[h]);
      else
#pragma unroll
        for (int e = 0; e < 8; ++e) qv[h][e] = 0.f;
    }
    // four of the wave's keys at a time, their loads first: a loop that waits for memory once a key costs a
    // round trip per key (a key past the end reads the last one again and stores nothing)
    const int stride = ATT_WAVES * TPW;
    for (int t0 = wave * TPW + slot; t0 < count; t0 += 4 * stride) {
      float kv[4][8];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = begin + min(t0 + u * stride, count - 1);
        const size_t page = table[j / page_size];
        const size_t base = ((page * kv_heads + kvh) * page_size + (j % page_size)) * (size_t)d + e0;
        if (live) ld8(k_cache + base, kv[u]);
        else
#pragma unroll
          for (int e = 0; e < 8; ++e) kv[u][e] = 0.f;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int t = t0 + u * stride;
#pragma unroll
        for (int h = 0; h < GT; ++h) {
          float dot = 0.f;
#pragma unroll
          for (int e = 0; e < 8; ++e) dot += qv[h][e] * kv[u][e];
          dot = group_sum(dot, tg_log2);
          if (sub == 0 && t < count) scores[h * P + t] = dot * scale;
        }
      }
    }
    __syncthreads();

    // ---- softmax statistics per head (block wide), probabilities back into LDS: the tile's heads together, the
    // waves' maxima and sums meeting in LDS in wave order (three barriers a tile of heads, not four a head)
    float m_h[GT], l_h[GT];
#pragma unroll
    for (int h = 0; h < GT; ++h) {
      float m = -INFINITY;
      for (int t = threadIdx.x; t < count; t += ATT_THREADS) m = fmaxf(m, scores[h * P + t]);
      m = wave_max(m);
      if (lane == 0) reduce[wave * GT + h] = m;
    }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < GT; ++h) {
      float m = reduce[h];
#pragma unroll
      for (int w = 1; w < ATT_WAVES; ++w) m = fmaxf(m, reduce[w * GT + h]);
      float l = 0.f;
      for (int t = threadIdx.x; t < count; t += ATT_THREADS) {
        const float p = expf(scores[h * P + t] - m);
        scores[h * P + t] = p;
        l += p;
      }
      l = wave_sum(l);
      if (lane == 0) reduce[(ATT_WAVES + wave) * GT + h] = l;
      m_h[h] = m;
    }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < GT; ++h) {
      float l = 0.f;
#pragma unroll
      for (int w = 0; w < ATT_WAVES; ++w) l += reduce[(ATT_WAVES + w) * GT + h];      // fixed order
      l_h[h] = l;
    }

    // ---- weighted values.  V is [pages, kv_heads, d, page_size]: a key's elements lie page_size apart and the keys
    // of a page side by side, so here a wave's lanes are 16 consecutive keys x 4 chunks of 8 elements (a load
    // instruction then reads whole 64-byte runs of 16 keys, not 16 bytes of 4 keys), and the head's elements are
    // taken 32 at a time.
    const int v_key = lane & 15, v_e0 = (lane >> 4) * 8;
    for (int c0 = 0; c0 < d; c0 += 32) {
      const int ve = c0 + v_e0;
      const bool v_live = ve < d;
      float acc[GT][8];
#pragma unroll
      for (int h = 0; h < GT; ++h)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[h][e] = 0.f;
      constexpr int V_STRIDE = ATT_WAVES * 16;
      for (int t0 = wave * 16 + v_key; t0 < count; t0 += 2 * V_STRIDE) {      // two keys at a time, their loads first
        float vv[2][8];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int j = begin + min(t0 + u * V_STRIDE, count - 1);
          const size_t page = table[j / page_size];
          const T* column = v_cache + ((page * kv_heads + kvh) * (size_t)d + ve) * page_size + (j % page_size);
#pragma unroll
          for (int e = 0; e < 8; ++e) vv[u][e] = v_live ? ld(column + (size_t)e * page_size) : 0.f;
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int t = t0 + u * V_STRIDE;
          if (t < count) {
#pragma unroll
            for (int h = 0; h < GT; ++h) {
              const float p = scores[h * P + t];
#pragma unroll
              for (int e = 0; e < 8; ++e) acc[h][e] += p * vv[u][e];
            }
          }
        }
      }
      // sum over the wave's 16 keys (fixed order), then over the waves below
#pragma unroll
      for (int h = 0; h < GT; ++h)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[h][e] = row16_sum(acc[h][e]);
      if (v_key == 0 && v_live) {
#pragma unroll
        for (int h = 0; h < GT; ++h)
#pragma unroll
          for (int e = 0; e < 8; ++e) wave_acc[(wave * GT + h) * d + ve + e] = acc[h][e];
      }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < GT * d; idx += ATT_THREADS) {
      const int h = idx / d, e = idx - h * d;
      if (h0 + h >= g) continue;
      float total = 0.f;
#pragma unroll
      for (int w = 0; w < ATT_WAVES; ++w) total += wave_acc[(w * GT + h) * d + e];
      const int head = kvh * g + h0 + h;
      // m_h / l_h live in registers indexed by a compile-time h; select without dynamic indexing
      float m = 0.f, l = 1.f;
#pragma unroll
      for (int hh = 0; hh < GT; ++hh)
        if (hh == h) { m = m_h[hh]; l = l_h[hh]; }
      if (parts == 1) {
        st(out + ((size_t)row * heads + head) * d + e, total / l);
      } else {
        const size_t cell = ((size_t)slot_row * heads + head) * parts + part;
        part_acc[cell * d + e] = total;
        if (e == 0) { part_m[cell] = m; part_l[cell] = l; }
      }
    }
    __syncthreads();
  }
}

// One wave a block; a head takes tg lanes (a power of two >= d / 4, four elements a lane), 64 / tg heads a wave.
// The parts are read eight at a time with all their loads first; the sums run over the parts in order.
template <typename T>
__global__ void __launch_bounds__(QIL_WAVE)
attn_rows_merge_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_m,
                       const float* __restrict__ part_l, const int* __restrict__ positions,
                       const int* __restrict__ row_index, T* __restrict__ out, int heads, int d,
                       int window, int P, int parts, int tg) {
  const int slot_row = blockIdx.x;
  const int head = blockIdx.y * (QIL_WAVE / tg) + threadIdx.x / tg, e = (threadIdx.x % tg) * 4;
  const bool head_there = head < heads;                    // the same for the tg lanes of a head; all of them take part in the maximum
  const int row = row_index ? row_index[slot_row] : slot_row;
  const int ctx = positions[row] + 1;
  const int lo = window > 0 ? max(0, ctx - window) : 0;
  const int first = lo / P, last = (ctx - 1) / P;
  const size_t cell0 = ((size_t)slot_row * heads + head) * parts;
  // the largest exponent: a head's lanes take a part each, then the largest among them (one round trip to memory for
  // up to tg parts, not one for every four)
  float m = -INFINITY;
  for (int p0 = first; p0 <= last; p0 += tg) {
    const int p = p0 + (int)(threadIdx.x % tg);
    if (head_there && p <= last) m = fmaxf(m, part_m[cell0 + p]);
  }
  for (int o = tg >> 1; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, QIL_WAVE));
  if (!head_there || e >= d) return;
  // the sums run over the parts in order, eight parts' loads at a time
  constexpr int AT_ONCE = 8;
  float denom = 0.f;
  float4 numer = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int p0 = first; p0 <= last; p0 += AT_ONCE) {
    float mv[AT_ONCE], lv[AT_ONCE];
    float4 acc[AT_ONCE];
#pragma unroll
    for (int j = 0; j < AT_ONCE; ++j) {
      const size_t cell = cell0 + min(p0 + j, last);
      mv[j] = part_m[cell];
      lv[j] = part_l[cell];
      acc[j] = *reinterpret_cast<const float4*>(part_acc + cell * d + e);
    }
#pragma unroll
    for (int j = 0; j < AT_ONCE; ++j) {
      if (p0 + j <= last) {
        const float f = expf(mv[j] - m);
        denom += lv[j] * f;
        numer.x += acc[j].x * f; numer.y += acc[j].y * f; numer.z += acc[j].z * f; numer.w += acc[j].w * f;
      }
    }
  }
  T* to = out + ((size_t)row * heads + head) * d + e;
  st(to, numer.x / denom); st(to + 1, numer.y / denom); st(to + 2, numer.z / denom); st(to + 3, numer.w / denom);
}

// Launch shape of the merge: lanes a head and the grid.
static void merge_shape(int rows, int heads, int d, int* tg, dim3* grid) {
  int lanes = 1;
  while (lanes * 4 < d) lanes *= 2;
  *tg = lanes;                                             // d <= 256: at most 64
  *grid = dim3(rows, (heads + QIL_WAVE / lanes - 1) / (QIL_WAVE / lanes));
}

static int next_pow2_log2(int v) {
  int l = 0;
  while ((1 << l) < v) ++l;
  return l;
}

// LDS floats the partial kernel needs.
static size_t rows_lds_floats(int gt, int P, int d) { return (size_t)gt * P + 64 + (size_t)ATT_WAVES * gt * d; }

template <typename T>
static int launch_rows(const void* q, int q_stride, const void* k_cache, const void* v_cache, const int* block_tables,
                       int table_stride, const int* row_seq, const int* positions, const int* row_index,
                       float* part_acc, float* part_m,
                       float* part_l, void* out, int rows, int heads, int kv_heads, int d, int page_size, int window,
                       float scale, int P, int parts, hipStream_t s, bool merge = true) {
  const int g = heads / kv_heads;
  const int gt = g >= 8 ? 8 : g > 2 ? 4 : g;            // head tile: 1, 2, 4 or 8
  const int tg_log2 = next_pow2_log2((d + 7) / 8);
  const size_t lds = rows_lds_floats(gt, P, d) * sizeof(float);
  dim3 grid(rows, kv_heads, parts);
#define QIL_ROWS_CASE(GT)                                                                                          \
  hipLaunchKernelGGL((attn_rows_partial_kernel<T, GT>), grid, dim3(ATT_THREADS), lds, s, (const T*)q, q_stride,    \
                     (const T*)k_cache, (const T*)v_cache, block_tables, table_stride, row_seq, positions,         \
                     row_index, part_acc, part_m, part_l, (T*)out, heads, kv_heads, d, page_size, window, scale, P, parts,    \
                     tg_log2)
  switch (gt) {
    case 1: QIL_ROWS_CASE(1); break;
    case 2: QIL_ROWS_CASE(2); break;
    case 4: QIL_ROWS_CASE(4); break;
    default: QIL_ROWS_CASE(8); break;
  }
#undef QIL_ROWS_CASE
  int status = (int)hipGetLastError();
  if (status || parts == 1 || !merge) return status;
  int tg;
  dim3 merge_grid;
  merge_shape(rows, heads, d, &tg, &merge_grid);
  hipLaunchKernelGGL(attn_rows_merge_kernel<T>, merge_grid, dim3(QIL_WAVE), 0, s, part_acc, part_m, part_l, positions,
                     row_index, (T*)out, heads, d, window, P, parts, tg);
  return (int)hipGetLastError();
}

extern "C" {

// Bytes of float32 workspace for `rows` rows split into `parts` parts (0 when parts == 1).
size_t qil_attn_rows_workspace(int rows, int heads, int d, int parts) {
  return parts <= 1 ? 0 : (size_t)rows * heads * parts * (d + 2) * sizeof(float);
}

// q: rows of stride q_stride elements, head h at offset h * d.  out: [all rows, heads * d].
// row_index: null (the kernel's rows are the batch's rows 0 .. rows-1) or the batch rows to serve.
// workspace: qil_attn_rows_workspace bytes.  P: keys per part, parts = ceil(max context / P).
// Requires d % 8 == 0, d <= 256, P <= 1024.  Returns -1 on a size it does not take.
int qil_attn_rows(const void* q, int q_stride, const void* k_cache, const void* v_cache, const int* block_tables,
                  int table_stride, const int* row_seq, const int* positions, const int* row_index, void* workspace,
                  void* out, int rows,
                  int heads, int kv_heads, int d, int page_size, int window, float scale, int P, int parts, int dtype,
                  hipStream_t s) {
  if (rows == 0) return 0;
  if (d % 8 || d > 256 || d < 8 || heads % kv_heads || P < 1 || P > 1024 || parts < 1 || parts > 65535 ||
      kv_heads > 65535) return -1;
  const int g = heads / kv_heads;
  const int gt = g >= 8 ? 8 : g > 2 ? 4 : g;
  if (rows_lds_floats(gt, P, d) * sizeof(float) > 64 * 1024) return -1;
  float* acc = (float*)workspace;
  float* m = acc ? acc + (size_t)rows * heads * parts * d : nullptr;
  float* l = m ? m + (size_t)rows * heads * parts : nullptr;
  if (dtype == QIL_F32)
    return launch_rows<float>(q, q_stride, k_cache, v_cache, block_tables, table_stride, row_seq, positions, row_index,
                              acc, m, l, out, rows, heads, kv_heads, d, page_size, window, scale, P, parts, s);
  return launch_rows<bf16_t>(q, q_stride, k_cache, v_cache, block_tables, table_stride, row_seq, positions, row_index,
                             acc, m, l, out, rows, heads, kv_heads, d, page_size, window, scale, P, parts, s);
}

// The same without the merge: the parts' results stay in the workspace for a consumer that merges them itself
// (parts > 1; `out` is not written).
int qil_attn_rows_unmerged(const void* q, int q_stride, const void* k_cache, const void* v_cache, const int* block_tables,
                           int table_stride, const int* row_seq, const int* positions, void* workspace, int rows,
                           int heads, int kv_heads, int d, int page_size, int window, float scale, int P, int parts,
                           int dtype, hipStream_t s) {
  if (rows == 0) return 0;
  if (d % 8 || d > 256 || d < 8 || heads % kv_heads || P < 1 || P > 1024 || parts < 2 || parts > 65535 ||
      kv_heads > 65535 || !workspace) return -1;
  const int g = heads / kv_heads;
  const int gt = g >= 8 ? 8 : g > 2 ? 4 : g;
  if (rows_lds_floats(gt, P, d) * sizeof(float) > 64 * 1024) return -1;
  float* acc = (float*)workspace;
  float* m = acc + (size_t)rows * heads * parts * d;
  float* l = m + (size_t)rows * heads * parts;
  if (dtype == QIL_F32)
    return launch_rows<float>(q, q_stride, k_cache, v_cache, block_tables, table_stride, row_seq, positions, nullptr,
                              acc, m, l, nullptr, rows, heads, kv_heads, d, page_size, window, scale, P, parts, s, false);
  return launch_rows<bf16_t>(q, q_stride, k_cache, v_cache, block_tables, table_stride, row_seq, positions, nullptr,
                             acc, m, l, nullptr, rows, heads, kv_heads, d, page_size, window, scale, P, parts, s, false);
}

// Merge of partial results written by a partial kernel (this file's or the matrix-core decode kernel's).
int qil_attn_merge(const void* workspace, const int* positions, const int* row_index, void* out, int rows, int heads,
                   int d, int window, int P, int parts, int dtype, hipStream_t s) {
  if (rows == 0 || parts <= 1) return 0;
  const float* acc = (const float*)workspace;
  const float* m = acc + (size_t)rows * heads * parts * d;
  const float* l = m + (size_t)rows * heads * parts;
  if (d % 4 || d > 256) return -1;
  int tg;
  dim3 grid;
  merge_shape(rows, heads, d, &tg, &grid);
  const dim3 block(QIL_WAVE);
  if (dtype == QIL_F32)
    hipLaunchKernelGGL(attn_rows_merge_kernel<float>, grid, block, 0, s, acc, m, l, positions, row_index, (float*)out,
                       heads, d, window, P, parts, tg);
  else
    hipLaunchKernelGGL(attn_rows_merge_kernel<bf16_t>, grid, block, 0, s, acc, m, l, positions, row_index, (bf16_t*)out,
                       heads, d, window, P, parts, tg);
  QIL_RETURN_LAUNCH_STATUS();
}

}  // extern "C"
