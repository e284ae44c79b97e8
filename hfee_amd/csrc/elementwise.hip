// Embedding gather, RMSNorm, rotary encoding with the write into the paged
// cache, SiLU gating and the residual add.  All of them are bound by memory
// traffic; sums, angles and the residual stream are float32.
//
// Formulas (file:line in /root/reference):
//   embedding   internal/llm/forward.go:75-77
//   RMSNorm     internal/ggml/ops.go:124-134  (x * scale * weight, eps inside the root)
//   rotation    internal/llm/forward.go:180-196, cache write forward.go:99-101
//   SiLU gate   internal/ggml/ops.go:159-165  (g / (1 + exp(-g)) * up)
//   residual    internal/ggml/ops.go:152-157
#include <type_traits>

#include "common.h"
#include "gemm_entry.h"

using namespace hfee;

HFEE_DEFINE_LAST_ERROR

// ------------------------------------------------------------------ embedding
template <typename T>
__global__ void embed_kernel(float* __restrict__ out, const T* __restrict__ table,
                             const int* __restrict__ ids, int d) {
  const int row = blockIdx.x;
  const int64_t src = (int64_t)ids[row] * d;
  for (int j = threadIdx.x; j < d; j += blockDim.x) out[(int64_t)row * d + j] = to_float<T>(table[src + j]);
}

// bfloat16 rows of a width that is a multiple of 8, 16-byte aligned: eight elements a
// thread, a row over several workgroups (a decode step's few rows then take one round of
// loads, not sixteen one after the other)
__global__ __launch_bounds__(256) void embed_bf16_wide_kernel(float* __restrict__ out, const bf16_t* __restrict__ table,
                                                              const int* __restrict__ ids, int d) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  const int row = blockIdx.x, j = 8 * (blockIdx.y * 256 + threadIdx.x);
  if (j >= d) return;
  const u32x4 v = *reinterpret_cast<const u32x4*>(table + (int64_t)ids[row] * d + j);
  float* o = out + (int64_t)row * d + j;
  f32x4 lo, hi;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    lo[2 * i] = __uint_as_float(v[i] << 16);
    lo[2 * i + 1] = __uint_as_float(v[i] & 0xffff0000u);
    hi[2 * i] = __uint_as_float(v[2 + i] << 16);
    hi[2 * i + 1] = __uint_as_float(v[2 + i] & 0xffff0000u);
  }
  *reinterpret_cast<f32x4*>(o) = lo;
  *reinterpret_cast<f32x4*>(o + 4) = hi;
}

// The same for at most 64 rows, with the first half of the norm that follows: also
// bfloat16(x * weight) into emit_out and, for the row's columns that this workgroup takes,
// their sum of squares into emit_ss[blockIdx.y * 64 + row] (the form in which the products
// of at most 64 rows take a norm in two halves: hfee_gemm_skinny's scale_ss).
template <typename TW>
__global__ __launch_bounds__(256) void embed_bf16_emit_kernel(float* __restrict__ out, const bf16_t* __restrict__ table,
                                                              const int* __restrict__ ids, int d,
                                                              const TW* __restrict__ weight, bf16_t* __restrict__ emit_out,
                                                              int64_t ld_emit, float* __restrict__ emit_ss) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  __shared__ float parts[4];
  const int row = blockIdx.x, j = 8 * (blockIdx.y * 256 + threadIdx.x);
  float ss = 0.f;
  if (j < d) {
    const u32x4 v = *reinterpret_cast<const u32x4*>(table + (int64_t)ids[row] * d + j);
    float x[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[2 * i] = __uint_as_float(v[i] << 16);
      x[2 * i + 1] = __uint_as_float(v[i] & 0xffff0000u);
    }
    float* o = out + (int64_t)row * d + j;
    *reinterpret_cast<f32x4*>(o) = f32x4{x[0], x[1], x[2], x[3]};
    *reinterpret_cast<f32x4*>(o + 4) = f32x4{x[4], x[5], x[6], x[7]};
    u32x4 e;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ss = fmaf(x[2 * i], x[2 * i], ss);
      ss = fmaf(x[2 * i + 1], x[2 * i + 1], ss);
      e[i] = (uint32_t)float_to_bf16(x[2 * i] * to_float<TW>(weight[j + 2 * i])) |
             (uint32_t)float_to_bf16(x[2 * i + 1] * to_float<TW>(weight[j + 2 * i + 1])) << 16;
    }
    *reinterpret_cast<u32x4*>(emit_out + (int64_t)row * ld_emit + j) = e;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
  if ((threadIdx.x & 63) == 0) parts[threadIdx.x >> 6] = ss;
  __syncthreads();
  if (threadIdx.x == 0) emit_ss[blockIdx.y * 64 + row] = (parts[0] + parts[1]) + (parts[2] + parts[3]);
}

// hfee_embed of a bfloat16 table for at most 64 rows, which also writes bfloat16(out * emit_weight)
// to emit_out [n, d] (rows ld_emit apart, 16-byte aligned) and the rows' sums of squares to
// emit_ss, in ceil(d / 2,048) shares of 64 floats (a workgroup takes 2,048 columns of a row).
HFEE_API int hfee_embed_emit(float* out, const void* table, const int* ids, int n, int d, const void* emit_weight,
                             int emit_weight_dtype, void* emit_out, int64_t ld_emit, float* emit_ss,
                             int64_t emit_ss_floats, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && n <= 64 && d > 0 && d % 8 == 0, "embed_emit: at most 64 rows of a width that is a multiple of 8 (n=%d d=%d)", n, d);
  HFEE_REQUIRE((uintptr_t)table % 16 == 0 && (uintptr_t)out % 16 == 0 && (uintptr_t)emit_out % 16 == 0 && ld_emit % 8 == 0 &&
               ld_emit >= d && emit_weight && emit_ss, "embed_emit: 16-byte aligned rows expected");
  const dim3 grid(n > 0 ? n : 1, (d + 2047) / 2048);
  HFEE_REQUIRE(emit_ss_floats >= (int64_t)grid.y * 64, "embed_emit: %d shares of 64 floats expected", (int)grid.y);
  if (n == 0) return 0;
  if (emit_weight_dtype == DT_F32)
    embed_bf16_emit_kernel<float><<<grid, 256, 0, stream>>>(out, (const bf16_t*)table, ids, d, (const float*)emit_weight,
                                                            (bf16_t*)emit_out, ld_emit, emit_ss);
  else if (emit_weight_dtype == DT_BF16)
    embed_bf16_emit_kernel<bf16_t><<<grid, 256, 0, stream>>>(out, (const bf16_t*)table, ids, d, (const bf16_t*)emit_weight,
                                                             (bf16_t*)emit_out, ld_emit, emit_ss);
  else
    return fail("embed_emit: unknown dtype %d", emit_weight_dtype);
  HFEE_CHECK_LAUNCH("embed_emit");
  return 0;
}

HFEE_API int hfee_embed(float* out, const void* table, int table_dtype, const int* ids,
                        int n, int d, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && d > 0, "embed: bad sizes n=%d d=%d", n, d);
  if (n == 0) return 0;
  if (table_dtype == DT_BF16 && d % 8 == 0 && (uintptr_t)table % 16 == 0 && (uintptr_t)out % 16 == 0 && n <= 65535) {
    embed_bf16_wide_kernel<<<dim3(n, (d + 2047) / 2048), 256, 0, stream>>>(out, (const bf16_t*)table, ids, d);
    HFEE_CHECK_LAUNCH("embed");
    return 0;
  }
  if (table_dtype == DT_F32)
    embed_kernel<float><<<n, 256, 0, stream>>>(out, (const float*)table, ids, d);
  else if (table_dtype == DT_BF16)
    embed_kernel<bf16_t><<<n, 256, 0, stream>>>(out, (const bf16_t*)table, ids, d);
  else
    return fail("embed: unknown dtype %d", table_dtype);
  HFEE_CHECK_LAUNCH("embed");
  return 0;
}

// ------------------------------------------------------------- rows as they are
// out[r] = x[rows[r] or r], rounded to the output's type: what stands where a norm would,
// in a model that has none there.  One block per output row.
template <typename TOut>
__global__ void cast_rows_kernel(TOut* __restrict__ out, const float* __restrict__ x, const int* __restrict__ rows, int d) {
  const int r = blockIdx.x;
  const float* xr = x + (int64_t)(rows ? rows[r] : r) * d;
  TOut* o = out + (int64_t)r * d;
  for (int j = threadIdx.x; j < d; j += blockDim.x) o[j] = from_float<TOut>(xr[j]);
}

HFEE_API int hfee_cast_rows(void* out, int out_dtype, const float* x, const int* rows, int n, int d, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && d > 0, "cast_rows: bad sizes n=%d d=%d", n, d);
  if (n == 0) return 0;
  if (out_dtype == DT_F32) cast_rows_kernel<float><<<n, 256, 0, stream>>>((float*)out, x, rows, d);
  else if (out_dtype == DT_BF16) cast_rows_kernel<bf16_t><<<n, 256, 0, stream>>>((bf16_t*)out, x, rows, d);
  else return fail("cast_rows: unknown dtype %d", out_dtype);
  HFEE_CHECK_LAUNCH("cast_rows");
  return 0;
}

// -------------------------------------------------------------------- RMSNorm
// One block per output row.  rows == nullptr: row r of x; else row rows[r] of x.
template <typename TOut, typename TW>
__global__ void rmsnorm_kernel(TOut* __restrict__ out, const float* __restrict__ x,
                               const TW* __restrict__ w, const int* __restrict__ rows,
                               float eps, int d) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const float* xr = x + (int64_t)(rows ? rows[r] : r) * d;
  float ss = 0.f;
  for (int j = threadIdx.x; j < d; j += blockDim.x) {
    const float v = xr[j];
    ss = fmaf(v, v, ss);
  }
  ss = block_sum(ss, scratch);
  const float scale = 1.0f / sqrtf(ss / (float)d + eps);
  TOut* o = out + (int64_t)r * d;
  for (int j = threadIdx.x; j < d; j += blockDim.x)
    o[j] = from_float<TOut>(xr[j] * scale * to_float<TW>(w[j]));
}

// The same with 16-byte loads and the row kept in registers between the sum and the
// scaling (d <= 4 * NV * blockDim.x, a multiple of 4; rows 16-byte aligned).
template <typename TOut, typename TW, int NV>
__global__ void rmsnorm_rows_kernel(TOut* __restrict__ out, const float* __restrict__ x,
                                    const TW* __restrict__ w, const int* __restrict__ rows,
                                    float eps, int d) {
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const float* xr = x + (int64_t)(rows ? rows[r] : r) * d;
  f32x4 v[NV];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int j = 4 * (threadIdx.x + i * blockDim.x);
    v[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (j < d) v[i] = *reinterpret_cast<const f32x4*>(xr + j);
#pragma unroll
    for (int c = 0; c < 4; ++c) ss = fmaf(v[i][c], v[i][c], ss);
  }
  ss = block_sum(ss, scratch);
  const float scale = 1.0f / sqrtf(ss / (float)d + eps);
  TOut* o = out + (int64_t)r * d;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int j = 4 * (threadIdx.x + i * blockDim.x);
    if (j < d) {
      TOut y[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) y[c] = from_float<TOut>(v[i][c] * scale * to_float<TW>(w[j + c]));
      if constexpr (sizeof(TOut) == 2) *reinterpret_cast<uint2*>(o + j) = *reinterpret_cast<const uint2*>(y);
      else *reinterpret_cast<f32x4*>(o + j) = *reinterpret_cast<const f32x4*>(y);
    }
  }
}

HFEE_API int hfee_rmsnorm(void* out, int out_dtype, const float* x, const void* w, int w_dtype,
                          const int* rows, float eps, int n, int d, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && d > 0, "rmsnorm: bad sizes n=%d d=%d", n, d);
  HFEE_REQUIRE(eps >= 0.f, "rmsnorm: eps must not be negative");
  if (n == 0) return 0;
  const int threads = d >= 2048 ? 512 : 256;
  // rows that start 16-byte aligned (8 for a bfloat16 result) and fit in registers
  const bool rows_fit = d % 4 == 0 && d <= 16 * threads && (uintptr_t)x % 16 == 0 &&
                        (uintptr_t)out % (out_dtype == DT_F32 ? 16 : 8) == 0;
  const int nv = (d + 4 * threads - 1) / (4 * threads);          // 1 .. 4
#define LAUNCH(TO, TW)                                                                                              \
  do {                                                                                                              \
    if (rows_fit && nv <= 1) rmsnorm_rows_kernel<TO, TW, 1><<<n, threads, 0, stream>>>((TO*)out, x, (const TW*)w, rows, eps, d);      \
    else if (rows_fit && nv == 2) rmsnorm_rows_kernel<TO, TW, 2><<<n, threads, 0, stream>>>((TO*)out, x, (const TW*)w, rows, eps, d); \
    else if (rows_fit) rmsnorm_rows_kernel<TO, TW, 4><<<n, threads, 0, stream>>>((TO*)out, x, (const TW*)w, rows, eps, d);            \
    else rmsnorm_kernel<TO, TW><<<n, threads, 0, stream>>>((TO*)out, x, (const TW*)w, rows, eps, d);                \
  } while (0)
  if (out_dtype == DT_F32 && w_dtype == DT_F32) LAUNCH(float, float);
  else if (out_dtype == DT_F32 && w_dtype == DT_BF16) LAUNCH(float, bf16_t);
  else if (out_dtype == DT_BF16 && w_dtype == DT_F32) LAUNCH(bf16_t, float);
  else if (out_dtype == DT_BF16 && w_dtype == DT_BF16) LAUNCH(bf16_t, bf16_t);
  else return fail("rmsnorm: unknown dtypes out=%d w=%d", out_dtype, w_dtype);
#undef LAUNCH
  HFEE_CHECK_LAUNCH("rmsnorm");
  return 0;
}

// ------------------------------------------------------------------ SiLU gate
template <typename T>
__global__ void swiglu_kernel(T* __restrict__ out, int64_t ld_out, const T* __restrict__ gate,
                              const T* __restrict__ up, int64_t ld_in, int col_stride, int width, int act) {
  const int row = blockIdx.y;
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= width) return;
  const float g = to_float<T>(gate[(int64_t)row * ld_in + (int64_t)j * col_stride]);
  const float u = to_float<T>(up[(int64_t)row * ld_in + (int64_t)j * col_stride]);
  out[(int64_t)row * ld_out + j] = from_float<T>((act == GATE_SILU ? g / (1.0f + expf(-g)) : gate_other_exact(g, act)) * u);
}

// col_stride: distance between consecutive gate (and up) columns: 1 for two separate
// blocks, 2 when gate and up alternate.  act: the gate's activation (GATE_SILU ...).
HFEE_API int hfee_swiglu(void* out, int64_t ld_out, const void* gate, const void* up, int64_t ld_in,
                         int col_stride, int dtype, int n, int width, int act, hipStream_t stream) {
  HFEE_REQUIRE(act >= 0 && act < GATE_KINDS, "swiglu: unknown activation %d", act);
  HFEE_REQUIRE(n >= 0 && width > 0 && ld_out >= width && col_stride >= 1 &&
               ld_in >= (int64_t)(width - 1) * col_stride + 1, "swiglu: bad sizes");
  HFEE_REQUIRE(n <= 65535 * 16, "swiglu: too many rows (%d)", n);
  if (n == 0) return 0;
  // grid.y is limited to 65535: fold rows beyond that into several launches
  for (int row0 = 0; row0 < n; row0 += 65535) {
    const int rows = n - row0 < 65535 ? n - row0 : 65535;
    dim3 grid((width + 255) / 256, rows);
    if (dtype == DT_F32)
      swiglu_kernel<float><<<grid, 256, 0, stream>>>((float*)out + row0 * ld_out, ld_out,
                                                     (const float*)gate + row0 * ld_in,
                                                     (const float*)up + row0 * ld_in, ld_in, col_stride, width, act);
    else if (dtype == DT_BF16)
      swiglu_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)out + row0 * ld_out, ld_out,
                                                      (const bf16_t*)gate + row0 * ld_in,
                                                      (const bf16_t*)up + row0 * ld_in, ld_in, col_stride, width, act);
    else
      return fail("swiglu: unknown dtype %d", dtype);
  }
  HFEE_CHECK_LAUNCH("swiglu");
  return 0;
}

// --------------------------------------------------------------- residual add
template <typename T>
__global__ void add_kernel(float* __restrict__ x, const T* __restrict__ y, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < total) x[i] += to_float<T>(y[i]);
}

HFEE_API int hfee_residual_add(float* x, const void* y, int y_dtype, int64_t total, hipStream_t stream) {
  HFEE_REQUIRE(total >= 0, "residual_add: bad size");
  if (total == 0) return 0;
  const int64_t blocks = (total + 255) / 256;
  HFEE_REQUIRE(blocks < (1ll << 31), "residual_add: too many elements");
  if (y_dtype == DT_F32) add_kernel<float><<<(unsigned)blocks, 256, 0, stream>>>(x, (const float*)y, total);
  else if (y_dtype == DT_BF16) add_kernel<bf16_t><<<(unsigned)blocks, 256, 0, stream>>>(x, (const bf16_t*)y, total);
  else return fail("residual_add: unknown dtype %d", y_dtype);
  HFEE_CHECK_LAUNCH("residual_add");
  return 0;
}

// ------------------------------------------------- rotation + write to the cache
// One block per token.  q is rotated in place; k is rotated and written to the
// token's slot of its page, v is written transposed.  cos/sin: [positions][half]
// float32, made on the host in float64 from the exact angle position * inv_freq.
// pairing 0: (i, i + half); pairing 1: (2i, 2i + 1).  Dimensions at and beyond
// 2 * half are not rotated.  Any of q, k/v may be null (nothing to do for it).
template <typename T>
__global__ void rope_cache_kernel(T* __restrict__ q, int64_t ldq, const T* __restrict__ k, int64_t ldk,
                                  const T* __restrict__ v, int64_t ldv,
                                  const int* __restrict__ positions, const int* __restrict__ token_segment,
                                  const int* __restrict__ block_tables, int bt_stride,
                                  const float* __restrict__ cos_table, const float* __restrict__ sin_table,
                                  int half, int pairing, T* __restrict__ cache, CacheLayout lay,
                                  int num_heads) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int hd = lay.head_dim;
  const float* cs = cos_table ? cos_table + (int64_t)pos * half : nullptr;
  const float* sn = sin_table ? sin_table + (int64_t)pos * half : nullptr;

  if (q != nullptr && cs != nullptr) {
    T* qt = q + (int64_t)t * ldq;
    for (int w = threadIdx.x; w < num_heads * half; w += blockDim.x) {
      const int h = w / half, i = w - h * half;
      const int a = pairing == 0 ? i : 2 * i;
      const int b = pairing == 0 ? i + half : 2 * i + 1;
      const float x0 = to_float<T>(qt[h * hd + a]), x1 = to_float<T>(qt[h * hd + b]);
      const float c = cs[i], s = sn[i];
      qt[h * hd + a] = from_float<T>(x0 * c - x1 * s);
      qt[h * hd + b] = from_float<T>(x0 * s + x1 * c);
    }
  }
  if (k == nullptr || cache == nullptr) return;

  const int page = block_tables[(int64_t)token_segment[t] * bt_stride + (pos >> lay.page_shift)];
  const int slot = pos & (lay.page_size - 1);
  const T* kt = k + (int64_t)t * ldk;
  const T* vt = v + (int64_t)t * ldv;
  const int rot = cs != nullptr ? 2 * half : 0;
  for (int w = threadIdx.x; w < lay.kv_heads * hd; w += blockDim.x) {
    const int h = w / hd, dd = w - h * hd;
    float val;
    if (dd < rot) {
      int i, partner;
      bool first;
      if (pairing == 0) { first = dd < half; i = first ? dd : dd - half; partner = first ? dd + half : dd - half; }
      else { first = (dd & 1) == 0; i = dd >> 1; partner = first ? dd + 1 : dd - 1; }
      const float me = to_float<T>(kt[h * hd + dd]), other = to_float<T>(kt[h * hd + partner]);
      const float c = cs[i], s = sn[i];
      val = first ? (me * c - other * s) : (other * s + me * c);
    } else {
      val = to_float<T>(kt[h * hd + dd]);
    }
    cache[lay.key_offset(page, h, slot, dd)] = finite_for_cache<T>(from_float<T>(val));
    cache[lay.value_offset(page, h, slot, dd)] = finite_for_cache<T>(vt[h * hd + dd]);
  }
}

// Where q, k and v come from when the product that makes them was cut along K over
// workgroups and its partial products have not been added up: `count` matrices of float32
// [rows, ld], `stride` floats apart, whose columns are q, then k (from k_col), then v (from
// v_col).  at null: q, k and v are read as bfloat16 rows.
struct QkvCuts {
  const float* at;
  int count;
  int64_t stride, ld;
  int k_col, v_col;
};

// The same for bfloat16 with adjacent pairs (2i, 2i + 1), eight elements (16 bytes, four
// pairs) per thread and step: head_dim and 2 * half multiples of 8, rows 16-byte aligned.
// With `cuts`, the partial products are added up here, in their order, and rounded to
// bfloat16 as the kernel that would have added them does: q is only written, k and v only
// say that the cache is written.
// Into how many workgroups the KV heads of 16 tokens' values are dealt (0: a head alone does not
// fit), and the LDS of each: at most 48 KB, 32 bytes a column.
struct GroupShares {
  int parts;
  size_t bytes;
};
inline GroupShares group_shares(int kv_heads, int head_dim, int n) {
  const int most = (int)(48 * 1024 / ((size_t)32 * head_dim));       // heads a workgroup
  if (most < 1) return GroupShares{0, 0};
  int parts = (kv_heads + most - 1) / most;
  // (few tokens: the groups' workgroups, which run longest, over more of the chip, 128 of them if the
  // heads allow: a layer of a 256-token prefill at the 8B shape 209 -> 205 us, nothing from 2,048 tokens on)
  const int groups = (n + 15) / 16;
  while (parts < kv_heads && groups * parts < 128) ++parts;
  const int heads_a_part = (kv_heads + parts - 1) / parts;
  parts = (kv_heads + heads_a_part - 1) / heads_a_part;              // (no workgroup without a head)
  return GroupShares{parts, (size_t)32 * heads_a_part * head_dim};
}

// (CUTS is a compile-time choice: as a check at run time in front of every load it cost the
// plain kernel 3.6 us of 14 at 2,048 tokens)
template <bool CUTS>
__global__ void rope_cache_pairs_kernel(bf16_t* __restrict__ q, int64_t ldq, const bf16_t* __restrict__ k, int64_t ldk,
                                        const bf16_t* __restrict__ v, int64_t ldv, QkvCuts cuts,
                                        const int* __restrict__ positions, const int* __restrict__ token_segment,
                                        const int* __restrict__ block_tables, int bt_stride,
                                        const float* __restrict__ cos_table, const float* __restrict__ sin_table,
                                        int half, bf16_t* __restrict__ cache, CacheLayout lay, int num_heads,
                                        int n, int values_by_groups) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  union Eight {
    u32x4 u;
    bf16_t e[8];
  };
  // elements col .. col + 7 of row t: from the bfloat16 row, or the sum of the cuts
  auto eight = [&](const bf16_t* row, int t, int col) {
    Eight x;
    if constexpr (!CUTS) {
      x.u = *reinterpret_cast<const u32x4*>(row);
      return x;
    }
    // (all cuts asked for together, up to 2, 4 or 8 of them; past the last one: a repeat that is not
    // added.  Always eight, two cuts of a 512-token portion cost the kernel twice the plain one's time.)
    auto sum_of = [&](auto most) {
      constexpr int MOST = decltype(most)::value;
      const float* p = cuts.at + (int64_t)t * cuts.ld + col;
      f32x4 lo[MOST], hi[MOST];
#pragma unroll
      for (int z = 0; z < MOST; ++z) {
        const float* pz = p + (int64_t)min(z, cuts.count - 1) * cuts.stride;
        lo[z] = *reinterpret_cast<const f32x4*>(pz);
        hi[z] = *reinterpret_cast<const f32x4*>(pz + 4);
      }
      f32x4 a = lo[0], b = hi[0];
#pragma unroll
      for (int z = 1; z < MOST; ++z)
        if (z < cuts.count) {
          a += lo[z];
          b += hi[z];
        }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        x.e[i] = float_to_bf16(a[i]);
        x.e[4 + i] = float_to_bf16(b[i]);
      }
    };
    if (cuts.count <= 2) sum_of(std::integral_constant<int, 2>{});
    else if (cuts.count <= 4) sum_of(std::integral_constant<int, 4>{});
    else sum_of(std::integral_constant<int, 8>{});
    return x;
  };
  // Some workgroups take the values of 16 consecutive tokens each.  The cache keeps values
  // transposed (a column of a head holds the page's slots side by side), so a token alone
  // writes two bytes here and two bytes there; 16 tokens that fill 16 slots in a row of one
  // page (a prompt's portion that starts on a page's edge) write 32 bytes a column at once.
  // (the groups' workgroups, which run longer than a token's, come first: none is left over at the end)
  // (values_by_groups: into how many workgroups the KV heads of such a group are dealt, so that a
  // workgroup's share of the 16 tokens' values fits its LDS: 40 heads of 128 are four of ten)
  const int groups = values_by_groups ? ((n + 15) / 16) * values_by_groups : 0;
  if ((int)blockIdx.x < groups) {
    extern __shared__ __attribute__((aligned(16))) bf16_t group_values[];      // [16][heads of this workgroup * head_dim]
    __shared__ int g_pos[16], g_page[16];
    const int part = (int)blockIdx.x % values_by_groups, heads_a_part = (lay.kv_heads + values_by_groups - 1) / values_by_groups;
    const int h_first = part * heads_a_part, c_first = h_first * lay.head_dim;
    const int t0 = 16 * ((int)blockIdx.x / values_by_groups), count = min(16, n - t0);
    const int width = max(0, min(lay.kv_heads - h_first, heads_a_part)) * lay.head_dim, chunks = width / 8;
    const int pieces = count * chunks;
    for (int first = threadIdx.x; first < pieces; first += 8 * blockDim.x) {      // eight loads in flight
      u32x4 piece[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int idx = min(first + u * (int)blockDim.x, pieces - 1), j = idx / chunks, c = idx - j * chunks;
        piece[u] = eight(v + (int64_t)(t0 + j) * ldv + c_first + 8 * c, t0 + j, cuts.v_col + c_first + 8 * c).u;
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int idx = first + u * (int)blockDim.x, j = idx / chunks, c = idx - j * chunks;
        if (idx < pieces) *reinterpret_cast<u32x4*>(group_values + j * width + 8 * c) = piece[u];
      }
    }
    if (threadIdx.x < count) {
      const int p = positions[t0 + threadIdx.x];
      g_pos[threadIdx.x] = p;
      g_page[threadIdx.x] = block_tables[(int64_t)token_segment[t0 + threadIdx.x] * bt_stride + (p >> lay.page_shift)];
    }
    __syncthreads();
    bool in_a_row = count == 16 && (g_pos[0] & 15) == 0;
    for (int j = 1; j < count; ++j) in_a_row = in_a_row && g_pos[j] == g_pos[0] + j && g_page[j] == g_page[0];
    for (int col = threadIdx.x; col < width; col += blockDim.x) {
      const int h = h_first + col / lay.head_dim, d = col % lay.head_dim;
      if (in_a_row) {
        union { u32x4 u[2]; bf16_t e[16]; } row;
#pragma unroll
        for (int j = 0; j < 16; ++j) row.e[CacheLayout::value_slot(j)] = finite_bf16(group_values[j * width + col]);
        u32x4* dst = reinterpret_cast<u32x4*>(cache + lay.value_column(g_page[0], h, d) + (g_pos[0] & (lay.page_size - 1)));
        dst[0] = row.u[0];
        dst[1] = row.u[1];
      } else {
        for (int j = 0; j < count; ++j)
          cache[lay.value_offset(g_page[j], h, g_pos[j] & (lay.page_size - 1), d)] = finite_bf16(group_values[j * width + col]);
      }
    }
    return;
  }
  const int t = (int)blockIdx.x - groups;
  const int pos = positions[t];
  const int hd = lay.head_dim, per_head = hd / 8;
  const float* cs = cos_table ? cos_table + (int64_t)pos * half : nullptr;
  const float* sn = sin_table ? sin_table + (int64_t)pos * half : nullptr;
  const int rot = cs != nullptr ? 2 * half : 0;
  // elements d .. d + 7 of a head: pairs d/2 .. d/2 + 3 (rot is a multiple of 8: all or none are rotated)
  auto rotate = [&](Eight& x, int d) {
    if (d >= rot) return;
    const f32x4 c = *reinterpret_cast<const f32x4*>(cs + (d >> 1)), s = *reinterpret_cast<const f32x4*>(sn + (d >> 1));
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const float x0 = bf16_to_float(x.e[2 * p]), x1 = bf16_to_float(x.e[2 * p + 1]);
      x.e[2 * p] = float_to_bf16(x0 * c[p] - x1 * s[p]);
      x.e[2 * p + 1] = float_to_bf16(x0 * s[p] + x1 * c[p]);
    }
  };
  // One walk over the token's pieces of eight elements, q's first and then k's (with v's): what
  // a thread needs of the tables is asked for before the first piece, so that the workgroups of
  // few tokens (a decode step) wait once for memory and not once for q and once again for k.
  const bool with_q = q != nullptr && (cs != nullptr || cuts.at != nullptr);
  const bool with_kv = k != nullptr && cache != nullptr;
  const int q_pieces = with_q ? num_heads * per_head : 0, kv_pieces = with_kv ? lay.kv_heads * per_head : 0;
  int page = 0;
  if (with_kv) page = block_tables[(int64_t)token_segment[t] * bt_stride + (pos >> lay.page_shift)];
  const int slot = pos & (lay.page_size - 1);
  bf16_t* qt = q + (int64_t)t * ldq;
  const bf16_t* kt = k + (int64_t)t * ldk;
  const bf16_t* vt = v + (int64_t)t * ldv;
  for (int u = threadIdx.x; u < q_pieces + kv_pieces; u += blockDim.x) {
    if (u < q_pieces) {
      const int d = (u % per_head) * 8;
      Eight x = eight(qt + u * 8, t, u * 8);
      rotate(x, d);
      *reinterpret_cast<u32x4*>(qt + u * 8) = x.u;
      continue;
    }
    const int w = u - q_pieces;
    const int h = w / per_head, d = (w - h * per_head) * 8;
    Eight x = eight(kt + w * 8, t, cuts.k_col + w * 8), y;
    if (!values_by_groups) y = eight(vt + w * 8, t, cuts.v_col + w * 8);
    rotate(x, d);
#pragma unroll
    for (int c = 0; c < 4; ++c) x.u[c] = finite_bf16x2(x.u[c]);       // only finite values go into the cache
    *reinterpret_cast<u32x4*>(cache + lay.key_offset(page, h, slot, d)) = x.u;
    if (values_by_groups) continue;                                    // (other workgroups write the values)
    bf16_t* vc = cache + lay.value_offset(page, h, slot, d);          // column d of the head; the next is page_size on
#pragma unroll
    for (int c = 0; c < 8; ++c) vc[(int64_t)c * lay.page_size] = finite_bf16(y.e[c]);
  }
}

HFEE_API int hfee_rope_cache_write(void* q, int64_t ldq, const void* k, int64_t ldk, const void* v, int64_t ldv,
                                   int dtype, const int* positions, const int* token_segment,
                                   const int* block_tables, int bt_stride,
                                   const float* cos_table, const float* sin_table, int half, int pairing,
                                   int table_positions, int max_position,
                                   void* cache, int num_heads, int kv_heads, int head_dim, int page_size,
                                   int n, int portions, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0, "rope_cache_write: bad token count");
  if (n == 0) return 0;
  HFEE_REQUIRE(pairing == 0 || pairing == 1, "rope_cache_write: pairing must be 0 (half) or 1 (interleaved)");
  HFEE_REQUIRE(half >= 0 && 2 * half <= head_dim, "rope_cache_write: rotary width %d exceeds head_dim %d",
               2 * half, head_dim);
  HFEE_REQUIRE(cos_table == nullptr || max_position < table_positions,
               "rope_cache_write: position %d is beyond the rotation table (%d positions)",
               max_position, table_positions);
  HFEE_REQUIRE((k == nullptr) == (v == nullptr), "rope_cache_write: k and v come together");
  CacheLayout lay;
  if (make_cache_layout(&lay, kv_heads, head_dim, page_size)) return 1;
  HFEE_REQUIRE(q == nullptr || ldq >= (int64_t)num_heads * head_dim, "rope_cache_write: q row too short");
  HFEE_REQUIRE(k == nullptr || (ldk >= (int64_t)kv_heads * head_dim && ldv >= (int64_t)kv_heads * head_dim),
               "rope_cache_write: k/v row too short");
  if (dtype == DT_F32)
    rope_cache_kernel<float><<<n, 256, 0, stream>>>((float*)q, ldq, (const float*)k, ldk, (const float*)v, ldv,
        positions, token_segment, block_tables, bt_stride, cos_table, sin_table, half, pairing,
        (float*)cache, lay, num_heads);
  else if (dtype == DT_BF16 && pairing == 1 && head_dim % 8 == 0 && half % 4 == 0 &&
           (q == nullptr || (ldq % 8 == 0 && (uintptr_t)q % 16 == 0)) &&
           (k == nullptr || (ldk % 8 == 0 && ldv % 8 == 0 && (uintptr_t)k % 16 == 0 && (uintptr_t)v % 16 == 0)) &&
           (uintptr_t)cos_table % 16 == 0 && (uintptr_t)sin_table % 16 == 0 && (uintptr_t)cache % 16 == 0)
  {
    // (the values of 16 tokens through LDS, if a workgroup's share of it fits and there is more than one group)
    const GroupShares shares = group_shares(kv_heads, head_dim, n);
    // (`portions`: the tokens hold runs of consecutive positions of a sequence.  Without them, single
    // tokens of many sequences, a group's workgroup would write 16 tokens' values two bytes at a time
    // on its own, eight workgroups for 128 tokens where every token's own workgroup can do it: 13 us
    // against 5 at 128 rows)
    const int by_groups = portions != 0 && k != nullptr && cache != nullptr && n >= 32 ? shares.parts : 0;
    rope_cache_pairs_kernel<false><<<n + by_groups * ((n + 15) / 16), 256, by_groups ? shares.bytes : 0, stream>>>(
        (bf16_t*)q, ldq, (const bf16_t*)k, ldk, (const bf16_t*)v, ldv, QkvCuts{nullptr, 0, 0, 0, 0, 0}, positions,
        token_segment, block_tables, bt_stride, cos_table, sin_table, half, (bf16_t*)cache, lay, num_heads, n, by_groups);
  }
  else if (dtype == DT_BF16)
    rope_cache_kernel<bf16_t><<<n, 256, 0, stream>>>((bf16_t*)q, ldq, (const bf16_t*)k, ldk, (const bf16_t*)v, ldv,
        positions, token_segment, block_tables, bt_stride, cos_table, sin_table, half, pairing,
        (bf16_t*)cache, lay, num_heads);
  else
    return fail("rope_cache_write: unknown dtype %d", dtype);
  HFEE_CHECK_LAUNCH("rope_cache_write");
  return 0;
}

// The same for q, k and v that lie as the partial products of a q/k/v product cut along K
// (hfee_gemm_bf16_cuts): `cuts` matrices of float32 [n, width], width = (num_heads + 2 *
// kv_heads) * head_dim, one after the other.  The partial products are added up in their
// order and rounded to bfloat16, then rotated (adjacent pairs); q goes to `q` (bfloat16, rows
// ldq apart), k and v into the cache: the numbers of the adding kernel followed by
// hfee_rope_cache_write, in one launch.  bfloat16 cache, adjacent pairs, head_dim and the
// rotary width multiples of 8.
HFEE_API int hfee_rope_cache_write_cuts(void* q, int64_t ldq, const float* partial, int cuts,
                                        const int* positions, const int* token_segment, const int* block_tables,
                                        int bt_stride, const float* cos_table, const float* sin_table, int half,
                                        int table_positions, int max_position, void* cache, int num_heads,
                                        int kv_heads, int head_dim, int page_size, int n, int portions,
                                        hipStream_t stream) {
  HFEE_REQUIRE(n >= 0, "rope_cache_write_cuts: bad token count");
  if (n == 0) return 0;
  HFEE_REQUIRE(q != nullptr && partial != nullptr && cache != nullptr && positions != nullptr &&
                   token_segment != nullptr && block_tables != nullptr,
               "rope_cache_write_cuts: q, the partial products, the cache and its tables are needed");
  HFEE_REQUIRE(cuts >= 1 && cuts <= 8, "rope_cache_write_cuts: 1 to 8 cuts, got %d", cuts);
  HFEE_REQUIRE(half >= 0 && 2 * half <= head_dim, "rope_cache_write_cuts: rotary width %d exceeds head_dim %d",
               2 * half, head_dim);
  HFEE_REQUIRE(cos_table == nullptr || max_position < table_positions,
               "rope_cache_write_cuts: position %d is beyond the rotation table (%d positions)", max_position,
               table_positions);
  CacheLayout lay;
  if (make_cache_layout(&lay, kv_heads, head_dim, page_size)) return 1;
  const int64_t width = (int64_t)(num_heads + 2 * kv_heads) * head_dim;
  HFEE_REQUIRE(head_dim % 8 == 0 && half % 4 == 0 && ldq % 8 == 0 && ldq >= (int64_t)num_heads * head_dim &&
                   (uintptr_t)q % 16 == 0 && (uintptr_t)partial % 16 == 0 && (uintptr_t)cos_table % 16 == 0 &&
                   (uintptr_t)sin_table % 16 == 0 && (uintptr_t)cache % 16 == 0,
               "rope_cache_write_cuts: head_dim and the rotary width must be multiples of 8 and the operands 16-byte aligned");
  const QkvCuts c{partial, cuts, (int64_t)n * width, width, num_heads * head_dim, (num_heads + kv_heads) * head_dim};
  const GroupShares shares = group_shares(kv_heads, head_dim, n);
  const int by_groups = portions != 0 && n >= 32 ? shares.parts : 0;
  // (k and v: any pointers that are not null; with cuts they are never read.  More threads than
  // the plain kernel has, a piece each where that is at most 768: a thread's eight elements
  // are up to sixteen loads, and few tokens leave CUs without a workgroup)
  const int pieces = (num_heads + kv_heads) * (head_dim / 8);
  const int threads = pieces >= 768 ? 768 : pieces > 512 ? (pieces + 63) / 64 * 64 : 512;
  rope_cache_pairs_kernel<true><<<n + by_groups * ((n + 15) / 16), threads, by_groups ? shares.bytes : 0, stream>>>(
      (bf16_t*)q, ldq, (const bf16_t*)q, 0, (const bf16_t*)q, 0, c, positions, token_segment, block_tables, bt_stride,
      cos_table, sin_table, half, (bf16_t*)cache, lay, num_heads, n, by_groups);
  HFEE_CHECK_LAUNCH("rope_cache_write_cuts");
  return 0;
}
