// The merge of split-context attention results, made by the product that consumes them.
#pragma once
#include "common.h"

// A given as the unmerged partial results of split-context attention (attention_rows.hip,
// attention_decode.hip): acc [M, heads, parts, d], m and l [M, heads, parts], float32.  Row m, column
// head * d + e of A is sum_p acc_p[e] exp(m_p - max m) / sum_p l_p exp(m_p - max m) over the parts that
// hold keys of the row: the merge of attn_rows_merge_kernel, made while A is staged.
struct UnmergedA {
  const float* acc;
  const float* m;
  const float* l;
  const int* positions;                                    // [M]: a row's context is its position + 1
  int heads, d, parts, P, window;
};

// E (4 or 8) merged values of row m starting at column k (all of one head: d % E == 0), float32.
// AT_ONCE: parts whose loads are in flight together (E * AT_ONCE registers).
template <int E, int AT_ONCE = 4>
__device__ __forceinline__ void merged_values(const UnmergedA& u, int m, int k, float (&out)[E]) {
  const int head = k / u.d, e = k - head * u.d;
  const int ctx = u.positions[m] + 1;
  const int lo = u.window > 0 ? max(0, ctx - u.window) : 0;
  const int first = lo / u.P, last = (ctx - 1) / u.P;
  const size_t cell0 = ((size_t)m * u.heads + head) * u.parts;
  auto load = [&](const float* p, float (&to)[E]) {
    if constexpr (E == 8) {
      ld8(p, to);
    } else {
      const float4 v = *reinterpret_cast<const float4*>(p);
      to[0] = v.x; to[1] = v.y; to[2] = v.z; to[3] = v.w;
    }
  };
  // AT_ONCE parts at a time, all their loads first: a loop that waits for memory once per part would cost more
  // than the merge kernel it replaces.  The first parts' sums and values are asked for together with their
  // maxima (they do not depend on the largest maximum, only their use does): one wait for up to AT_ONCE parts.
  float mv[AT_ONCE], lv[AT_ONCE], part[AT_ONCE][E];
#pragma unroll
  for (int j = 0; j < AT_ONCE; ++j) {
    const int p = min(first + j, last);
    mv[j] = u.m[cell0 + p];
    lv[j] = u.l[cell0 + p];
    load(u.acc + (cell0 + p) * u.d + e, part[j]);
  }
  float top = -INFINITY;
#pragma unroll
  for (int j = 0; j < AT_ONCE; ++j) top = fmaxf(top, mv[j]);
  for (int p0 = first + AT_ONCE; p0 <= last; p0 += 16) {    // the other parts' maxima, sixteen loads at a time
    float more[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) more[j] = u.m[cell0 + min(p0 + j, last)];
#pragma unroll
    for (int j = 0; j < 16; ++j) top = fmaxf(top, more[j]);
  }
  float denom = 0.f, numer[E];
#pragma unroll
  for (int i = 0; i < E; ++i) numer[i] = 0.f;
  for (int p0 = first; p0 <= last; p0 += AT_ONCE) {
    if (p0 != first) {
#pragma unroll
      for (int j = 0; j < AT_ONCE; ++j) {
        const int p = min(p0 + j, last);
        mv[j] = u.m[cell0 + p];
        lv[j] = u.l[cell0 + p];
        load(u.acc + (cell0 + p) * u.d + e, part[j]);
      }
    }
#pragma unroll
    for (int j = 0; j < AT_ONCE; ++j) {                     // the order and the arithmetic of the merge kernel
      if (p0 + j <= last) {
        const float f = expf(mv[j] - top);
        denom += lv[j] * f;
#pragma unroll
        for (int i = 0; i < E; ++i) numer[i] += part[j][i] * f;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < E; ++i) out[i] = numer[i] / denom;
}
