// The q/k/v epilogue shared by the matrix products: rows of W are q heads, then k heads,
// then v heads, with the two halves of a rotation pair as neighbours (2i, 2i + 1).  Four
// finished sums (weight rows n .. n+3 of batch row m; head sizes are multiples of 4, so
// they lie in one head) are rotated at the token's position if they belong to q or k
// (/root/reference/internal/llm/forward.go:96-101, 180-196), rounded once, and go to the
// q output or into the token's slot of the paged cache.
#pragma once
#include "common.h"

namespace hfee {

typedef uint32_t qkv_u32x2 __attribute__((ext_vector_type(2)));

struct QkvArgs {
  const int* positions;       // [M]
  const int* token_segment;   // [M]
  const int* block_tables;
  int bt_stride;
  const float* cos_table;     // [positions][half] or null
  const float* sin_table;
  int half;                   // rotated pairs per head
  void* cache;                // one cache layer, or null (keys and values are not written)
  CacheLayout lay;
  int num_heads;
  // (the tiled kernels hand this struct to every epilogue: the gated one finds its activation here)
  int gate_act;               // GATE_SILU ...
};


// Where four finished sums go and what they are rotated by: everything that has to be
// read for them, so that a kernel can ask for it before its sums are ready.
struct QkvPlace {
  float c[2], s[2];      // cosine and sine of the two pairs (rotate[p] says whether pair p is rotated)
  bool rotate[2];
  bf16_t* dst;           // null: nothing to store
  int step;              // elements between the four values at dst (1: one 8-byte store)
  bool cached;           // dst lies in the cache: only finite values go there
};

__device__ __forceinline__ QkvPlace qkv_place(const QkvArgs& q, void* C, int64_t ldc, int m, int n) {
  QkvPlace w;
  const int hd = q.lay.head_dim;
  const int head = n / hd, d = n - head * hd;
  const int pos = q.positions[m];
  const bool is_v = head >= q.num_heads + q.lay.kv_heads;
  const bool rotated = !is_v && q.cos_table != nullptr && d < 2 * q.half;
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    w.rotate[p] = rotated && d + 2 * p < 2 * q.half;
    w.c[p] = w.rotate[p] ? q.cos_table[(int64_t)pos * q.half + (d >> 1) + p] : 1.f;
    w.s[p] = w.rotate[p] ? q.sin_table[(int64_t)pos * q.half + (d >> 1) + p] : 0.f;
  }
  w.dst = nullptr;
  w.step = 1;
  w.cached = head >= q.num_heads;
  if (head < q.num_heads) {
    w.dst = (bf16_t*)C + (int64_t)m * ldc + n;
  } else if (q.cache != nullptr) {
    const int page = q.block_tables[(int64_t)q.token_segment[m] * q.bt_stride + (pos >> q.lay.page_shift)];
    const int slot = pos & (q.lay.page_size - 1);
    bf16_t* cache = (bf16_t*)q.cache;
    if (!is_v) {
      w.dst = cache + q.lay.key_offset(page, head - q.num_heads, slot, d);
    } else {
      w.dst = cache + q.lay.value_offset(page, head - q.num_heads - q.lay.kv_heads, slot, d);
      w.step = q.lay.page_size;          // a head's value columns lie page_size apart
    }
  }
  return w;
}

__device__ __forceinline__ void qkv_put(const QkvPlace& w, float* v) {
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    if (w.rotate[p]) {
      const float x0 = v[2 * p], x1 = v[2 * p + 1];
      v[2 * p] = x0 * w.c[p] - x1 * w.s[p];
      v[2 * p + 1] = x0 * w.s[p] + x1 * w.c[p];
    }
  }
  bf16_t o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) o[i] = float_to_bf16(w.cached ? finite_for_bf16(v[i]) : v[i]);
  if (w.dst == nullptr) return;
  if (w.step == 1) {
    *reinterpret_cast<qkv_u32x2*>(w.dst) = *reinterpret_cast<const qkv_u32x2*>(o);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) w.dst[(int64_t)i * w.step] = o[i];
  }
}

__device__ __forceinline__ void qkv_store(const QkvArgs& q, void* C, int64_t ldc, int m, int n, float* v) {
  qkv_put(qkv_place(q, C, ldc, m, n), v);
}

}  // namespace hfee
