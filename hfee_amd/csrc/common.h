// Shared device helpers and the host-side error channel of the kernel library.
// Target: gfx950 (CDNA4), wave64.  Every entry point is extern "C", takes raw
// device pointers, sizes and a stream, checks its arguments on the host and
// returns 0, or a nonzero code after recording a message that
// hfee_last_error() returns.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#define HFEE_API extern "C" __attribute__((visibility("default")))

typedef uint16_t bf16_t;   // storage type of bfloat16 values

namespace hfee {

constexpr int kWave = 64;

// ---- host-side error channel -------------------------------------------------
inline char* error_buffer() {
  static thread_local char buffer[512];
  return buffer;
}

inline int fail(const char* fmt, ...) {   // records the message, returns 1
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return 1;
}

// Exactly one translation unit of each shared library expands this.
#define HFEE_DEFINE_LAST_ERROR \
  HFEE_API const char* hfee_last_error() { return hfee::error_buffer(); }

#define HFEE_REQUIRE(cond, ...)                     \
  do {                                              \
    if (!(cond)) return hfee::fail(__VA_ARGS__);    \
  } while (0)

#define HFEE_CHECK_LAUNCH(name)                                              \
  do {                                                                       \
    hipError_t e_ = hipGetLastError();                                       \
    if (e_ != hipSuccess) return hfee::fail("%s: launch failed: %s", name,   \
                                            hipGetErrorString(e_));          \
  } while (0)

// ---- bfloat16 <-> float --------------------------------------------------------
__device__ __forceinline__ float bf16_to_float(bf16_t v) {
  return __uint_as_float(((uint32_t)v) << 16);
}

__device__ __forceinline__ bf16_t float_to_bf16(float f) {
  // round to nearest even; gfx950 has the conversion in hardware (v_cvt_pk_bf16_f32)
  return __builtin_bit_cast(bf16_t, (__bf16)f);
}

// ---- loads of what is read once ---------------------------------------------------
// Weights and the cache are streamed: every byte is read once a step and not again before
// everything else has passed through the caches.  The non-temporal hint tells the caches so;
// a read-only stream over device memory measures 7.1 TB/s with it and 6.3 TB/s without.
template <typename V>
__device__ __forceinline__ V load_streamed(const V* p) {
#ifdef HFEE_PLAIN_LOADS
  return *p;
#else
  return __builtin_nontemporal_load(p);
#endif
}

// ---- what goes into the cache is finite ------------------------------------------
// The matrix-core attention multiplies keys and values that a query must not see by a
// weight of zero instead of skipping them, and such keys may lie in a page that belonged
// to another request before.  Zero times infinity is NaN, so an infinity or NaN that one
// request's numbers overflowed to must never reach the cache, or it would turn up in the
// output of whoever gets the page next: every write to the cache goes through these (an
// infinity becomes the largest finite number of its sign, a NaN a finite number).
constexpr float kBf16Max = 3.3895313892515355e38f;      // 0x7F7F: the largest finite bfloat16
constexpr float kF32Max = 3.4028234663852886e38f;

__device__ __forceinline__ float finite_for_bf16(float v) { return fminf(fmaxf(v, -kBf16Max), kBf16Max); }

__device__ __forceinline__ bf16_t finite_bf16(bf16_t b) {
  return (b & 0x7F80) == 0x7F80 ? (bf16_t)((b & 0x8000) | 0x7F7F) : b;
}

__device__ __forceinline__ uint32_t finite_bf16x2(uint32_t w) {
  return (uint32_t)finite_bf16((bf16_t)(w & 0xffff)) | ((uint32_t)finite_bf16((bf16_t)(w >> 16)) << 16);
}

template <typename T> __device__ __forceinline__ T finite_for_cache(T v);
template <> __device__ __forceinline__ float finite_for_cache<float>(float v) { return fminf(fmaxf(v, -kF32Max), kF32Max); }
template <> __device__ __forceinline__ bf16_t finite_for_cache<bf16_t>(bf16_t v) { return finite_bf16(v); }

template <typename T> __device__ __forceinline__ float to_float(T v);
template <> __device__ __forceinline__ float to_float<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_float<bf16_t>(bf16_t v) { return bf16_to_float(v); }

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float v) { return float_to_bf16(v); }

// The activation of a gated feed-forward's gate, as the entry points name it.  The SiLU
// (/root/reference/internal/ggml/ops.go:159-165) is written out where it is used, in the
// form that each kernel has been measured with; the others are here, in forms that cost
// one exponential, as the SiLU does, so that an epilogue which carries them beside it stays
// small: g/2 (1 + tanh y) = g / (1 + exp(-2y)), and the error function by its rational
// approximation with exp(-x^2) (Abramowitz and Stegun 7.1.26, absolute error below 1.5e-7;
// the kernels that use these round the result to bfloat16).
enum { GATE_SILU = 0, GATE_GELU_TANH = 1, GATE_GELU = 2, GATE_RELU = 3, GATE_KINDS = 4 };

template <int ACT>
__device__ __forceinline__ float gate_other_as(float g) {
  if constexpr (ACT == GATE_GELU_TANH) {
    const float y = 0.7978845608028654f * (g + 0.044715f * g * g * g);
    return g * __frcp_rn(1.0f + __expf(-2.0f * y));
  } else if constexpr (ACT == GATE_GELU) {
    const float x = fabsf(g) * 0.7071067811865476f, t = __frcp_rn(1.0f + 0.3275911f * x);
    const float poly = t * (0.254829592f + t * (-0.284496736f + t * (1.421413741f + t * (-1.453152027f + t * 1.061405429f))));
    const float erf_abs = 1.0f - poly * __expf(-x * x);
    return 0.5f * g * (1.0f + (g < 0.f ? -erf_abs : erf_abs));
  } else {
    return fmaxf(g, 0.0f);
  }
}

__device__ __forceinline__ float gate_other(float g, int act) {
  return act == GATE_GELU_TANH ? gate_other_as<GATE_GELU_TANH>(g)
         : act == GATE_GELU    ? gate_other_as<GATE_GELU>(g)
                               : gate_other_as<GATE_RELU>(g);
}

// The same to the last bit of the library's functions, for the 32-bit path.
__device__ __forceinline__ float gate_other_exact(float g, int act) {
  if (act == GATE_GELU_TANH) return 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
  if (act == GATE_GELU) return 0.5f * g * (1.0f + erff(g * 0.7071067811865476f));
  return fmaxf(g, 0.0f);
}

// ---- reductions with a fixed order -------------------------------------------
// Every lane ends with the same value; the tree's shape does not depend on data.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// Sum over a block of up to 1024 threads; `scratch` holds 16 floats of LDS.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nwaves = (blockDim.x + 63) >> 6;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < nwaves; ++w) total += scratch[w];
  return total;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nwaves = (blockDim.x + 63) >> 6;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = scratch[0];
  for (int w = 1; w < nwaves; ++w) total = fmaxf(total, scratch[w]);
  return total;
}

// ---- weights in tiles, for the products of up to 64 rows ------------------------------
// [N, K] as rows of tiles of 16 rows x 32 columns, K and N filled up with zeros to whole
// tiles.  A tile is 512 elements (a kilobyte of bfloat16) in the order [column group of
// 8][row][8 columns]: lane l of a wave that holds the tile as the row operand of
// v_mfma_f32_16x16x32_bf16 (row l % 16, columns 8 (l / 16) .. + 7) finds its 16 bytes at
// 16 l, so the wave's load is the kilobyte from front to back.  The tiles of 16 rows follow
// one another along K.
struct WeightTiles {
  static constexpr int ROWS = 16, COLUMNS = 32, TILE = ROWS * COLUMNS;
  static constexpr int PER_COLUMN = TILE / COLUMNS;      // a lane's place moves by this per column (in steps of 32 columns)
  __host__ __device__ static __forceinline__ int64_t row_stride(int K) {
    return (int64_t)((K + COLUMNS - 1) / COLUMNS) * TILE;
  }
  // where the lane with row `row` (any row of the matrix) and column group g (0..3) finds its
  // eight elements of columns 0..31; columns 32 c .. 32 c + 31 are c * TILE further on
  __device__ static __forceinline__ const bf16_t* lane_place(const bf16_t* w, int64_t stride, int row, int g) {
    return w + (int64_t)(row >> 4) * stride + (g * ROWS + (row & 15)) * 8;
  }
};

// ---- the paged cache's layout -------------------------------------------------
// One cache layer is [num_pages][2][kv_heads][page_size * head_dim] elements:
// keys of a (page, head) as [slot][head_dim], values transposed as [head_dim][slot'],
// where slot' is the slot with bits 2 and 3 exchanged: within every 16 slots the order
// is 0-3, 8-11, 4-7, 12-15.  The matrix-core attention holds, per lane, the keys
// 4G..4G+3 and 8+4G..8+4G+3 of a 16-key step; stored this way they are 16 contiguous
// bytes of one value column in bfloat16.
struct CacheLayout {
  int64_t page_stride;   // elements between pages: 2 * kv_heads * page_size * head_dim
  int kv_heads;
  int head_dim;
  int page_size;
  int page_shift;        // log2(page_size)

  // Keys lie in chunks of key_chunk dims: [head_dim / key_chunk][slot][key_chunk].  With chunks
  // of 16 (head sizes that are multiples of 16) the sixteen bytes that a lane of the attention
  // kernels loads as a matrix operand (eight dims of one key) stand beside those of the
  // page's other keys, so that a load instruction of a wave covers whole 128-byte lines: that
  // is what lets the decode kernel read keys as a stream (non-temporal loads refetch a line
  // that an instruction takes only a part of), 5.5 -> 6.3 TB/s.  Other head sizes (the 32-bit
  // path takes any): one chunk, a key's dims in a row.
  __host__ __device__ __forceinline__ int key_chunk() const { return head_dim % 16 == 0 ? 16 : head_dim; }
  __host__ __device__ __forceinline__ int64_t key_chunk_stride() const { return (int64_t)page_size * key_chunk(); }
  __host__ __device__ __forceinline__ int64_t key_offset(int page, int kvh, int slot, int d) const {
    const int kc = key_chunk();
    return (int64_t)page * page_stride + (int64_t)kvh * page_size * head_dim + (int64_t)(d / kc) * page_size * kc +
           (int64_t)slot * kc + d % kc;
  }
  __host__ __device__ static __forceinline__ int value_slot(int slot) {
    return (slot & ~12) | ((slot & 4) << 1) | ((slot & 8) >> 1);
  }
  // first element of value column d of a (page, head): page_size slots follow
  __host__ __device__ __forceinline__ int64_t value_column(int page, int kvh, int d) const {
    return (int64_t)page * page_stride + (int64_t)(kv_heads + kvh) * page_size * head_dim + (int64_t)d * page_size;
  }
  __host__ __device__ __forceinline__ int64_t value_offset(int page, int kvh, int slot, int d) const {
    return value_column(page, kvh, d) + value_slot(slot);
  }
};

inline int make_cache_layout(CacheLayout* out, int kv_heads, int head_dim, int page_size) {
  if (page_size < 16 || (page_size & (page_size - 1)) != 0)
    return fail("page_size must be a power of two >= 16, got %d", page_size);
  if (kv_heads < 1 || head_dim < 1) return fail("bad cache shape: kv_heads %d head_dim %d", kv_heads, head_dim);
  out->kv_heads = kv_heads;
  out->head_dim = head_dim;
  out->page_size = page_size;
  out->page_stride = (int64_t)2 * kv_heads * page_size * head_dim;
  int s = 0;
  while ((1 << s) < page_size) ++s;
  out->page_shift = s;
  return 0;
}

}  // namespace hfee
