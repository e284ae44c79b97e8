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
};


__device__ __forceinline__ void qkv_store(const QkvArgs& q, void* C, int64_t ldc, int m, int n, float* v) {
  const int hd = q.lay.head_dim;
  const int head = n / hd, d = n - head * hd;
  const int pos = q.positions[m];
  const bool is_v = head >= q.num_heads + q.lay.kv_heads;
  if (!is_v && q.cos_table != nullptr && d < 2 * q.half) {
    const float* cs = q.cos_table + (int64_t)pos * q.half + (d >> 1);
    const float* sn = q.sin_table + (int64_t)pos * q.half + (d >> 1);
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      if (d + 2 * p < 2 * q.half) {
        const float x0 = v[2 * p], x1 = v[2 * p + 1], c = cs[p], s = sn[p];
        v[2 * p] = x0 * c - x1 * s;
        v[2 * p + 1] = x0 * s + x1 * c;
      }
    }
  }
  bf16_t o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) o[i] = float_to_bf16(v[i]);
  if (head < q.num_heads) {
    *reinterpret_cast<qkv_u32x2*>((bf16_t*)C + (int64_t)m * ldc + n) = *reinterpret_cast<const qkv_u32x2*>(o);
  } else if (q.cache != nullptr) {
    const int page = q.block_tables[(int64_t)q.token_segment[m] * q.bt_stride + (pos >> q.lay.page_shift)];
    const int slot = pos & (q.lay.page_size - 1);
    bf16_t* cache = (bf16_t*)q.cache;
    if (!is_v) {
      *reinterpret_cast<qkv_u32x2*>(cache + q.lay.key_offset(page, head - q.num_heads, slot, d)) =
          *reinterpret_cast<const qkv_u32x2*>(o);
    } else {
      const int kvh = head - q.num_heads - q.lay.kv_heads;
#pragma unroll
      for (int i = 0; i < 4; ++i) cache[q.lay.value_offset(page, kvh, slot, d + i)] = o[i];
    }
  }
}

}  // namespace hfee
