// Plain paged attention: one wave per (token, head), any head size, any page size.
// It is the 32-bit path's attention and the slow twin of the matrix-core kernels.
//
// The reference's order (/root/reference/internal/llm/forward.go:144-178,
// /root/reference/internal/ggml/ops.go:136-150): score_j = dot(q, k_j) * scale for
// the keys 0..pos of the token's own sequence (the range is the causal mask),
// subtract the maximum, exponentiate, sum, and accumulate the values in ascending
// j.  Here lane (j mod 64) owns key j, so which lane adds which term depends only
// on the key's absolute position: the result for a token does not change with the
// way the work was cut into steps, with the batch around it or with page numbers.
#include "common.h"

using namespace hfee;

namespace {

template <typename T>
__global__ __launch_bounds__(64) void attention_ref_kernel(
    T* __restrict__ out, int64_t ld_out, const T* __restrict__ q, int64_t ldq,
    const T* __restrict__ cache, CacheLayout lay, const int* __restrict__ positions,
    const int* __restrict__ token_segment, const int* __restrict__ block_tables, int bt_stride,
    int num_heads, float scale, int window) {
  extern __shared__ float lds[];
  const int hd = lay.head_dim;
  float* qs = lds;            // [hd]
  float* es = lds + hd;       // [64]
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int kvh = h / (num_heads / lay.kv_heads);
  const int pos = positions[t];
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int* bt = block_tables + (int64_t)token_segment[t] * bt_stride;

  for (int d = lane; d < hd; d += 64) qs[d] = to_float<T>(q[(int64_t)t * ldq + h * hd + d]);
  __syncthreads();

  const int first_block = lo & ~63;
  // pass 1: the maximum score
  float m = -INFINITY;
  for (int base = first_block; base <= pos; base += 64) {
    const int j = base + lane;
    if (j >= lo && j <= pos) {
      const T* kr = cache + lay.key_offset(bt[j >> lay.page_shift], kvh, j & (lay.page_size - 1), 0);
      const int kc = lay.key_chunk();
      const int64_t chunk_stride = lay.key_chunk_stride();
      float s = 0.f;
      for (int d = 0; d < hd; ++d) s = fmaf(qs[d], to_float<T>(kr[(d / kc) * chunk_stride + d % kc]), s);
      m = fmaxf(m, s * scale);
    }
  }
  m = wave_max(m);

  // pass 2: exponentials, their sum, and the weighted values
  float lsum = 0.f;
  float o[4] = {0.f, 0.f, 0.f, 0.f};   // dims lane, lane+64, lane+128, lane+192
  for (int base = first_block; base <= pos; base += 64) {
    const int j = base + lane;
    float e = 0.f;
    if (j >= lo && j <= pos) {
      const T* kr = cache + lay.key_offset(bt[j >> lay.page_shift], kvh, j & (lay.page_size - 1), 0);
      const int kc = lay.key_chunk();
      const int64_t chunk_stride = lay.key_chunk_stride();
      float s = 0.f;
      for (int d = 0; d < hd; ++d) s = fmaf(qs[d], to_float<T>(kr[(d / kc) * chunk_stride + d % kc]), s);
      e = expf(s * scale - m);
      lsum += e;
    }
    __syncthreads();
    es[lane] = e;
    __syncthreads();
    const int jb = max(base, lo), je = min(base + 63, pos);
    for (int jj = jb; jj <= je; ++jj) {
      const float w = es[jj - base];
      const int page = bt[jj >> lay.page_shift], slot = jj & (lay.page_size - 1);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int d = lane + 64 * r;
        if (d < hd) o[r] = fmaf(w, to_float<T>(cache[lay.value_offset(page, kvh, slot, d)]), o[r]);
      }
    }
  }
  lsum = wave_sum(lsum);
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int d = lane + 64 * r;
    if (d < hd) out[(int64_t)t * ld_out + h * hd + d] = from_float<T>(o[r] / lsum);
  }
}

}  // namespace

HFEE_API int hfee_attention_ref(void* out, int64_t ld_out, const void* q, int64_t ldq, const void* cache,
                                int dtype, const int* positions, const int* token_segment,
                                const int* block_tables, int bt_stride, int num_heads, int kv_heads,
                                int head_dim, int page_size, float scale, int window, int n,
                                hipStream_t stream) {
  HFEE_REQUIRE(n >= 0, "attention_ref: bad token count");
  if (n == 0) return 0;
  HFEE_REQUIRE(num_heads > 0 && kv_heads > 0 && num_heads % kv_heads == 0,
               "attention_ref: %d heads are not a multiple of %d kv heads", num_heads, kv_heads);
  HFEE_REQUIRE(head_dim >= 1 && head_dim <= 256, "attention_ref: head_dim %d is outside 1..256", head_dim);
  HFEE_REQUIRE(num_heads <= 65535, "attention_ref: too many heads");
  HFEE_REQUIRE(window >= 0, "attention_ref: negative window");
  HFEE_REQUIRE(ldq >= (int64_t)num_heads * head_dim && ld_out >= (int64_t)num_heads * head_dim,
               "attention_ref: q/out row too short");
  CacheLayout lay;
  if (make_cache_layout(&lay, kv_heads, head_dim, page_size)) return 1;
  dim3 grid(n, num_heads);
  const size_t lds = (head_dim + 64) * sizeof(float);
  if (dtype == 0)
    attention_ref_kernel<float><<<grid, 64, lds, stream>>>((float*)out, ld_out, (const float*)q, ldq,
        (const float*)cache, lay, positions, token_segment, block_tables, bt_stride, num_heads, scale, window);
  else if (dtype == 1)
    attention_ref_kernel<bf16_t><<<grid, 64, lds, stream>>>((bf16_t*)out, ld_out, (const bf16_t*)q, ldq,
        (const bf16_t*)cache, lay, positions, token_segment, block_tables, bt_stride, num_heads, scale, window);
  else
    return fail("attention_ref: unknown dtype %d", dtype);
  HFEE_CHECK_LAUNCH("attention_ref");
  return 0;
}
