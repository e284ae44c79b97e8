// bfloat16 matrix products on the matrix cores: C[M,N] = A[M,K] * W[N,K]^T with
// float32 accumulation.  The role of /root/reference/internal/ggml/ops.go:54-91
// (every weight row is read once for all rows of the batch).
//
// Two kernels:
//  * tiled   (M > 64, prefill): 128x128x32 tiles staged through LDS, four waves,
//            each wave a 64x64 block of v_mfma_f32_32x32x16_bf16 tiles.  Bound by
//            the matrix cores.
//  * skinny  (M <= 64, decode): bound by reading W once from HBM.  A workgroup owns
//            16 weight rows; its eight waves split K and stream their slices of W
//            straight from global memory into v_mfma_f32_16x16x32_bf16 operands
//            (no LDS on the way); the batch rows are the other operand.  Partial
//            sums meet in LDS in a fixed order.
// Output modes: bfloat16 store, float32 store, float32 accumulate (the residual
// add of /root/reference/internal/llm/forward.go:106-107 fused into the epilogue).
#include "common.h"
#include "qkv_epilogue.h"
#include "gemm_entry.h"


using namespace hfee;

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

enum { OUT_BF16 = 0, OUT_F32 = 1, OUT_ADD_F32 = 2, OUT_SWIGLU = 3, OUT_QKV = 4 };

union Chunk {           // eight bfloat16 values = 16 bytes
  u32x4 u;
  bf16x8 v;
  bf16_t e[8];
};

// Eight consecutive elements of a row starting at column k (zeros beyond K or when
// the row is out of range).  VEC: the row start is 16-byte aligned and K % 8 == 0.
template <bool VEC>
__device__ __forceinline__ Chunk load_chunk(const bf16_t* __restrict__ row, bool row_ok, int k, int K) {
  Chunk c;
  c.u = u32x4{0u, 0u, 0u, 0u};
  if (!row_ok) return c;
  if (VEC) {
    if (k < K) c.u = *reinterpret_cast<const u32x4*>(row + k);
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (k + j < K) c.e[j] = row[k + j];
  }
  return c;
}

template <int MODE>
__device__ __forceinline__ void store_out(void* C, int64_t ldc, int m, int n, float v) {
  if (MODE == OUT_BF16) ((bf16_t*)C)[(int64_t)m * ldc + n] = float_to_bf16(v);
  else if (MODE == OUT_F32) ((float*)C)[(int64_t)m * ldc + n] = v;
  else ((float*)C)[(int64_t)m * ldc + n] += v;
}

// ------------------------------------------------------------------- tiled ---
constexpr int TBM = 128, TBN = 128, TBK = 32, TPITCH = 40;   // LDS row pitch in elements (80 bytes)

template <int MODE, bool VEC>
__global__ __launch_bounds__(256) void gemm_bf16_tiled_kernel(void* __restrict__ C, int64_t ldc,
                                                              const bf16_t* __restrict__ A, int64_t lda,
                                                              const bf16_t* __restrict__ W, int64_t ldw,
                                                              int M, int N, int K) {
  __shared__ __attribute__((aligned(16))) bf16_t As[2][TBM * TPITCH];
  __shared__ __attribute__((aligned(16))) bf16_t Ws[2][TBN * TPITCH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.y * TBM, n0 = blockIdx.x * TBN;

  // staging: thread -> (row, 16-byte chunk) of the 128 x 32 tile, two rows apart by 64
  const int srow = tid >> 2, schunk = (tid & 3) * 8;
  const bf16_t* a_row[2];
  const bf16_t* w_row[2];
  bool a_ok[2], w_ok[2];
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const int am = m0 + srow + 64 * p, wn_ = n0 + srow + 64 * p;
    a_ok[p] = am < M;
    w_ok[p] = wn_ < N;
    a_row[p] = A + (int64_t)(a_ok[p] ? am : 0) * lda;
    w_row[p] = W + (int64_t)(w_ok[p] ? wn_ : 0) * ldw;
  }

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  Chunk ra[2], rw[2];
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    ra[p] = load_chunk<VEC>(a_row[p], a_ok[p], schunk, K);
    rw[p] = load_chunk<VEC>(w_row[p], w_ok[p], schunk, K);
  }
  const int ktiles = (K + TBK - 1) / TBK;
  int buf = 0;
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    *reinterpret_cast<u32x4*>(&As[0][(srow + 64 * p) * TPITCH + schunk]) = ra[p].u;
    *reinterpret_cast<u32x4*>(&Ws[0][(srow + 64 * p) * TPITCH + schunk]) = rw[p].u;
  }
  __syncthreads();

  const int lrow = lane & 31, lk = (lane >> 5) * 8;
  for (int kt = 0; kt < ktiles; ++kt) {
    if (kt + 1 < ktiles) {
      const int k = (kt + 1) * TBK + schunk;
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        ra[p] = load_chunk<VEC>(a_row[p], a_ok[p], k, K);
        rw[p] = load_chunk<VEC>(w_row[p], w_ok[p], k, K);
      }
    }
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      bf16x8 a[2], b[2];
#pragma unroll
      for (int i = 0; i < 2; ++i)
        a[i] = *reinterpret_cast<const bf16x8*>(&As[buf][(wm * 64 + i * 32 + lrow) * TPITCH + ks * 16 + lk]);
#pragma unroll
      for (int j = 0; j < 2; ++j)
        b[j] = *reinterpret_cast<const bf16x8*>(&Ws[buf][(wn * 64 + j * 32 + lrow) * TPITCH + ks * 16 + lk]);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < ktiles) {
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        *reinterpret_cast<u32x4*>(&As[buf ^ 1][(srow + 64 * p) * TPITCH + schunk]) = ra[p].u;
        *reinterpret_cast<u32x4*>(&Ws[buf ^ 1][(srow + 64 * p) * TPITCH + schunk]) = rw[p].u;
      }
    }
    __syncthreads();
    buf ^= 1;
  }

  // D layout of the 32x32 tile: register r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column l%32
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = n0 + wn * 64 + j * 32 + lrow;
      if (n >= N) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (m < M) store_out<MODE>(C, ldc, m, n, acc[i][j][r]);
      }
    }
}


// The gate's activation of a finished sum.  ACT is known when the epilogue is compiled: an
// epilogue is unrolled over a wave's 128 gates, and with a choice between the activations at each
// of them it was 45,000 instructions where the reference's alone has 8,000 (a layer of a
// 2,048-token prefill took 969 us instead of 885).
template <int ACT>
__device__ __forceinline__ float gated(float g) {
  if constexpr (ACT == GATE_SILU) return g * __frcp_rn(1.0f + __expf(-g));
  else return gate_other_as<ACT>(g);
}

// Calls f(std::integral_constant<int, ACT>) for the activation of a gating product (MODE says whether it is one).
template <int MODE, typename F>
__device__ __forceinline__ void with_gate_activation(int act, F&& f) {
  if (MODE != OUT_SWIGLU || act == GATE_SILU) f(std::integral_constant<int, GATE_SILU>{});
  else if (act == GATE_GELU_TANH) f(std::integral_constant<int, GATE_GELU_TANH>{});
  else if (act == GATE_GELU) f(std::integral_constant<int, GATE_GELU>{});
  else f(std::integral_constant<int, GATE_RELU>{});
}

// How a wave holds a tile of a product that was formed transposed (weights as the row
// operand).  ACC is what the matrix instruction leaves: f32x16 for 32 x 32 x 16 (register r of
// lane l holds C[m_base + l % 32][n_base + 8 (r / 4) + 4 (l / 32) + r % 4]), f32x4 for
// 16 x 16 x 32 (C[m_base + l % 16][n_base + 4 (l / 16) + r]).  Either way four registers are four
// consecutive columns of one row of C: a tile of R x R is Q such groups a lane, group q at
// columns STEP q + 4 (l / R).
template <typename ACC>
struct TileOf {
  static constexpr int R = sizeof(ACC) == 64 ? 32 : 16;      // rows and columns of a tile
  static constexpr int STEP = 4 * (64 / R);                  // columns from one of a lane's groups to its next
  static constexpr int Q = R / STEP;                         // groups a lane and tile
  static_assert(sizeof(ACC) == 64 || sizeof(ACC) == 16, "f32x16 or f32x4");
};

// Stores a tile that was formed transposed.  `vec`: rows of C start 16-byte aligned (8 for
// bfloat16).  m: this lane's row of C (m_base + l % R).
template <int MODE, int ACT = GATE_SILU, typename ACC>
__device__ __forceinline__ void store_tile_t(void* C, int64_t ldc, int M, int N, int m, int n_base, int lane,
                                             const ACC& t, bool vec) {
  using T = TileOf<ACC>;
  if (m >= M) return;
#pragma unroll
  for (int q = 0; q < T::Q; ++q) {
    const int n = n_base + T::STEP * q + 4 * (lane / T::R);
    if (n >= N) continue;
    float v[4] = {t[4 * q], t[4 * q + 1], t[4 * q + 2], t[4 * q + 3]};
    if (MODE == OUT_SWIGLU) {          // columns n, n+1 are gate, up of output column n / 2
      bf16_t* c = (bf16_t*)C + (int64_t)m * ldc + (n >> 1);
      const bf16_t o0 = float_to_bf16(gated<ACT>(v[0]) * v[1]);
      const bf16_t o1 = float_to_bf16(gated<ACT>(v[2]) * v[3]);
      if (vec && n + 3 < N) {
        *reinterpret_cast<uint32_t*>(c) = (uint32_t)o0 | ((uint32_t)o1 << 16);
      } else {
        c[0] = o0;
        if (n + 3 < N) c[1] = o1;
      }
    } else if (MODE == OUT_BF16) {
      bf16_t* c = (bf16_t*)C + (int64_t)m * ldc + n;
      if (vec && n + 3 < N) {
        u32x2 o;
        o[0] = (uint32_t)float_to_bf16(v[0]) | ((uint32_t)float_to_bf16(v[1]) << 16);
        o[1] = (uint32_t)float_to_bf16(v[2]) | ((uint32_t)float_to_bf16(v[3]) << 16);
        *reinterpret_cast<u32x2*>(c) = o;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < N) c[i] = float_to_bf16(v[i]);
      }
    } else {
      float* c = (float*)C + (int64_t)m * ldc + n;
      if (vec && n + 3 < N) {
        f32x4 o = {v[0], v[1], v[2], v[3]};
        if (MODE == OUT_ADD_F32) o += *reinterpret_cast<const f32x4*>(c);
        *reinterpret_cast<f32x4*>(c) = o;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < N) c[i] = MODE == OUT_ADD_F32 ? c[i] + v[i] : v[i];
      }
    }
  }
}

// The same for a wave's whole TM x TN tiles, through the LDS: a lane holds four
// consecutive columns of one row, so a store instruction of the plain way writes 16 or
// 32 bytes each to 32 different rows of C; here a strip of 32 rows is laid down in the
// wave's own piece of LDS (rows 16 bytes askew) and read back so that 16 bytes a lane
// make whole rows of C, 256 bytes and more at a time.  For tiles that lie inside C, with
// rows of C that start 16-byte aligned; the caller has made sure that nobody reads the
// LDS any more.  lds: the wave's own STAGE_BYTES.
// (TN tiles of R columns a strip row; R rows a strip)
template <int MODE, int TN, int R = 32>
struct Stage {
  static constexpr int ES = (MODE == OUT_BF16 || MODE == OUT_SWIGLU) ? 2 : 4;     // bytes of an element of C
  static constexpr int OC = MODE == OUT_SWIGLU ? R / 2 * TN : R * TN;            // columns of C in a strip row
  static constexpr int PITCH = OC * ES + 16;
  static constexpr int CHUNKS = OC * ES / 16;
  static constexpr int BYTES = (R * PITCH + 1023) / 1024 * 1024;
};

template <int MODE, int TM, int TN, int ACT = GATE_SILU, typename ACC>
__device__ __forceinline__ void store_wave_staged(char* lds, void* C, int64_t ldc, int M, int m_first, int n_first,
                                                  int lane, const ACC (&acc)[TM][TN]) {
  using T = TileOf<ACC>;
  constexpr int R = T::R;
  using S = Stage<MODE, TN, R>;
  constexpr int TOTAL = R * S::CHUNKS, PIECES = (TOTAL + 63) / 64;      // 16-byte pieces of a strip, and per lane
  const int lrow = lane % R, h = lane / R;
  char* crow = (char*)C + ((int64_t)m_first * ldc + (MODE == OUT_SWIGLU ? n_first / 2 : n_first)) * S::ES;
  // where piece `it` of this lane in strip i goes (null: nowhere)
  auto place = [&](int i, int it) -> f32x4* {
    const int idx = lane + 64 * it, row = idx / S::CHUNKS, c = idx - row * S::CHUNKS;
    return idx < TOTAL && m_first + i * R + row < M
               ? reinterpret_cast<f32x4*>(crow + (int64_t)(i * R + row) * ldc * S::ES + c * 16) : nullptr;
  };
  // What is added to is asked for a strip ahead: with the strips one after the other each would
  // wait for its own values from memory (eight strips of 16 rows: 78 us against 74.6 for four of 32,
  // output product of the 8B shape).
  f32x4 old[2][PIECES];
  auto ask_old = [&](int i, f32x4* into) {
    if constexpr (MODE == OUT_ADD_F32) {
#pragma unroll
      for (int it = 0; it < PIECES; ++it) {
        const f32x4* p = place(i, it);
        if (p) into[it] = *p;
      }
    }
  };
  ask_old(0, old[0]);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    if (i + 1 < TM) ask_old(i + 1, old[(i + 1) & 1]);
    char* mine = lds + lrow * S::PITCH;
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int q = 0; q < T::Q; ++q) {
        const ACC& t = acc[i][j];
        const float v[4] = {t[4 * q], t[4 * q + 1], t[4 * q + 2], t[4 * q + 3]};
        const int col = j * R + T::STEP * q + 4 * h;          // this group's first column within the strip
        if constexpr (MODE == OUT_SWIGLU) {
          const bf16_t o0 = float_to_bf16(gated<ACT>(v[0]) * v[1]);
          const bf16_t o1 = float_to_bf16(gated<ACT>(v[2]) * v[3]);
          *reinterpret_cast<uint32_t*>(mine + (col / 2) * 2) = (uint32_t)o0 | ((uint32_t)o1 << 16);
        } else if constexpr (MODE == OUT_BF16) {
          u32x2 o;
          o[0] = (uint32_t)float_to_bf16(v[0]) | ((uint32_t)float_to_bf16(v[1]) << 16);
          o[1] = (uint32_t)float_to_bf16(v[2]) | ((uint32_t)float_to_bf16(v[3]) << 16);
          *reinterpret_cast<u32x2*>(mine + col * 2) = o;
        } else {
          *reinterpret_cast<f32x4*>(mine + col * 4) = f32x4{v[0], v[1], v[2], v[3]};
        }
      }
    // (the same wave wrote what it reads: its LDS instructions keep their order)
#pragma unroll
    for (int it = 0; it < PIECES; ++it) {
      const int idx = lane + 64 * it, row = idx / S::CHUNKS, c = idx - row * S::CHUNKS;
      f32x4* dst = place(i, it);
      if (dst) {
        const f32x4 piece = *reinterpret_cast<const f32x4*>(lds + row * S::PITCH + c * 16);
        *dst = MODE == OUT_ADD_F32 ? old[i & 1][it] + piece : piece;
      }
    }
  }
}

// The q/k/v epilogue for a wave's TM x TN tiles of transposed products: what
// belongs to a row (position, page, slot) is fetched once per row, what belongs to four
// columns (head, place in the head, q or k or v) once per four columns.
template <int TM, int TN, typename ACC>
__device__ __forceinline__ void store_wave_qkv(void* C, int64_t ldc, int M, int N, int m_first, int n_first, int lane,
                                               const ACC (&acc)[TM][TN], const QkvArgs& qkv) {
  using T = TileOf<ACC>;
  constexpr int R = T::R;
  const int lrow = lane % R, hd = qkv.lay.head_dim;
  int pos[TM], slot[TM];
  int64_t page_base[TM];
  bool row_ok[TM];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m_first + i * R + lrow;
    row_ok[i] = m < M;
    const int mm = row_ok[i] ? m : M - 1;
    pos[i] = qkv.positions[mm];
    slot[i] = pos[i] & (qkv.lay.page_size - 1);
    page_base[i] = 0;
    if (qkv.cache != nullptr)
      page_base[i] = (int64_t)qkv.block_tables[(int64_t)qkv.token_segment[mm] * qkv.bt_stride + (pos[i] >> qkv.lay.page_shift)] *
                     qkv.lay.page_stride;
  }
  bf16_t* cache = (bf16_t*)qkv.cache;
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int q = 0; q < T::Q; ++q) {
      const int n = n_first + j * R + T::STEP * q + 4 * (lane / R);
      if (n >= N) continue;
      const int head = n / hd, d = n - head * hd;
      const bool is_q = head < qkv.num_heads, is_v = head >= qkv.num_heads + qkv.lay.kv_heads;
      const bool rotate = !is_v && qkv.cos_table != nullptr && d < 2 * qkv.half;
      const bool second = d + 2 < 2 * qkv.half;              // the second pair is inside the rotated part too
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        if (!row_ok[i]) continue;
        float v[4] = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
        if (rotate) {
          const float* cs = qkv.cos_table + (int64_t)pos[i] * qkv.half + (d >> 1);
          const float* sn = qkv.sin_table + (int64_t)pos[i] * qkv.half + (d >> 1);
          const float x0 = v[0], x1 = v[1], c0 = cs[0], s0 = sn[0];
          v[0] = x0 * c0 - x1 * s0;
          v[1] = x0 * s0 + x1 * c0;
          if (second) {
            const float x2 = v[2], x3 = v[3], c1 = cs[1], s1 = sn[1];
            v[2] = x2 * c1 - x3 * s1;
            v[3] = x2 * s1 + x3 * c1;
          }
        }
        if (!is_q) {                                           // only finite values go into the cache
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = finite_for_bf16(v[e]);
        }
        u32x2 o;
        o[0] = (uint32_t)float_to_bf16(v[0]) | ((uint32_t)float_to_bf16(v[1]) << 16);
        o[1] = (uint32_t)float_to_bf16(v[2]) | ((uint32_t)float_to_bf16(v[3]) << 16);
        const int m = m_first + i * R + lrow;
        if (is_q) {
          *reinterpret_cast<u32x2*>((bf16_t*)C + (int64_t)m * ldc + n) = o;
        } else if (cache != nullptr) {
          if (!is_v) {
            *reinterpret_cast<u32x2*>(cache + page_base[i] + qkv.lay.key_offset(0, head - qkv.num_heads, slot[i], d)) = o;
          } else {
            bf16_t* col = cache + page_base[i] + qkv.lay.value_offset(0, head - qkv.num_heads - qkv.lay.kv_heads, slot[i], d);
            col[0] = (bf16_t)(o[0] & 0xffff);
            col[qkv.lay.page_size] = (bf16_t)(o[0] >> 16);
            col[2 * qkv.lay.page_size] = (bf16_t)(o[1] & 0xffff);
            col[3 * qkv.lay.page_size] = (bf16_t)(o[1] >> 16);
          }
        }
      }
    }
}

// ---------------------------------------------------------- tiled, pipelined ---
// The prefill product for aligned operands.  Four waves in a 2x2 grid, each with
// TM x TN tiles of 32x32 (a workgroup tile of 64 TM x 64 TN), K in steps of 64.
// Global loads run STAGES K steps ahead of the matrix instructions (a ring of
// register stages), the LDS holds two steps.  Epilogues: bfloat16 store, float32
// store, float32 accumulate, and the SiLU gate for weights whose rows alternate
// gate/up (C[m, j] = silu(row 2j) * row 2j+1).
constexpr int PBK = 64, PPITCH = 72;   // pitch 144 bytes: no bank conflicts
constexpr int XCDS = 8;                // accelerator dies of an MI355X

template <int TM, int TN>
struct PStage {
  u32x4 a[2 * TM], w[2 * TN];      // this thread's 16-byte chunks of the A tile and of the W tile
};

template <int MODE, int TM, int TN, int STAGES>
__global__ __launch_bounds__(256) void gemm_bf16_pipelined_kernel(void* __restrict__ C, int64_t ldc,
                                                                  const bf16_t* __restrict__ A, int64_t lda,
                                                                  const bf16_t* __restrict__ W, int64_t ldw,
                                                                  int M, int N, int K, QkvArgs qkv,
                                                                  int k_split, int64_t c_split) {
  constexpr int BM = 64 * TM, BN = 64 * TN;
  extern __shared__ __attribute__((aligned(16))) bf16_t lds_tiles[];
  // K cut over workgroups (k_split > 0): workgroup row blockIdx.y takes columns
  // y * k_split .. of A and W and leaves its product in a matrix of its own, c_split elements
  // after the one before; a second kernel adds them up.
  if (k_split > 0) {
    const int z = blockIdx.y;
    A += (int64_t)z * k_split;
    W += (int64_t)z * k_split;
    K = min(k_split, K - z * k_split);
    C = (void*)((float*)C + (int64_t)z * c_split);
  }
  auto a_tile = [&](int buf) { return lds_tiles + buf * (BM * PPITCH); };
  auto w_tile = [&](int buf) { return lds_tiles + 2 * BM * PPITCH + buf * (BN * PPITCH); };
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  // Workgroups go to the eight XCDs in turn, and each XCD has an L2 of its own.  Give
  // every XCD a contiguous run of tiles, rows of the batch varying fastest: the
  // workgroups that run together on an XCD then share a few W tiles, and W comes from
  // HBM once.
  int m0, n0;
  {
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const int total = tiles_m * tiles_n, per_xcd = (total + XCDS - 1) / XCDS;
    const int t = (int)(blockIdx.x % XCDS) * per_xcd + (int)(blockIdx.x / XCDS);
    if (t >= total) return;
    m0 = (t % tiles_m) * BM;
    n0 = (t / tiles_m) * BN;
  }

  // staging: a tile row is 8 chunks; thread -> row tid/8 + 32p, chunk tid%8
  const int srow = tid >> 3, schunk = (tid & 7) * 8;
  const bf16_t* a_ptr[2 * TM];
  const bf16_t* w_ptr[2 * TN];
#pragma unroll
  for (int p = 0; p < 2 * TM; ++p)   // rows beyond M or N read the last valid row; their results are not stored
    a_ptr[p] = A + (int64_t)min(m0 + srow + 32 * p, M - 1) * lda + schunk;
#pragma unroll
  for (int p = 0; p < 2 * TN; ++p)
    w_ptr[p] = W + (int64_t)min(n0 + srow + 32 * p, N - 1) * ldw + schunk;
  const int ktiles = (K + PBK - 1) / PBK;
  // The main loop has no branch around its loads and nothing that reads a loaded value
  // before it goes to the LDS: the compiler can then count the loads and wait only for
  // the stage it needs.  A chunk beyond K (K is a multiple of 8: it is inside or outside
  // as a whole) is read from the row's last chunk; only the last steps, which run after
  // the main loop, can hold such a chunk, and they replace it by zeros on its way to the LDS.
  auto inside = [&](int kt) { return kt * PBK + schunk < K; };
  auto load_stage = [&](PStage<TM, TN>& st, int kt) {
    const int ks = inside(kt) ? kt * PBK : K - 8 - schunk;
#pragma unroll
    for (int p = 0; p < 2 * TM; ++p) st.a[p] = *reinterpret_cast<const u32x4*>(a_ptr[p] + ks);
#pragma unroll
    for (int p = 0; p < 2 * TN; ++p) st.w[p] = *reinterpret_cast<const u32x4*>(w_ptr[p] + ks);
  };
  auto store_stage = [&](const PStage<TM, TN>& st, int buf, bool in) {
    const u32x4 zero{0u, 0u, 0u, 0u};
#pragma unroll
    for (int p = 0; p < 2 * TM; ++p)
      *reinterpret_cast<u32x4*>(a_tile(buf) + (srow + 32 * p) * PPITCH + schunk) = in ? st.a[p] : zero;
#pragma unroll
    for (int p = 0; p < 2 * TN; ++p)
      *reinterpret_cast<u32x4*>(w_tile(buf) + (srow + 32 * p) * PPITCH + schunk) = in ? st.w[p] : zero;
  };

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  PStage<TM, TN> ring[STAGES];
#pragma unroll
  for (int s = 0; s < STAGES; ++s) load_stage(ring[s], s);
  store_stage(ring[0], 0, inside(0));
  __syncthreads();

  const int lrow = lane & 31, lk = (lane >> 5) * 8;
  auto step = [&](auto slot_c, auto last_c, int kt) {
    constexpr int SLOT = decltype(slot_c)::value;
    constexpr bool LAST = decltype(last_c)::value;
    const int buf = kt & 1;
    load_stage(ring[SLOT], kt + STAGES);     // ring[SLOT] went to LDS one step ago
    // operands of the next 16 columns are read from the LDS while this 16's products run
    bf16x8 a[2][TM], b[2][TN];
    auto read_operands = [&](int ks, bf16x8* af, bf16x8* bf) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
        af[i] = *reinterpret_cast<const bf16x8*>(a_tile(buf) + (wm * 32 * TM + i * 32 + lrow) * PPITCH + ks * 16 + lk);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        bf[j] = *reinterpret_cast<const bf16x8*>(w_tile(buf) + (wn * 32 * TN + j * 32 + lrow) * PPITCH + ks * 16 + lk);
    };
    read_operands(0, a[0], b[0]);
#pragma unroll
    for (int ks = 0; ks < PBK / 16; ++ks) {
      if (ks + 1 < PBK / 16) read_operands(ks + 1, a[(ks + 1) & 1], b[(ks + 1) & 1]);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[ks & 1][j], a[ks & 1][i], acc[i][j], 0, 0, 0);   // transposed
    }
    store_stage(ring[(SLOT + 1) % STAGES], buf ^ 1, LAST ? inside(kt + 1) : true);
    __syncthreads();
  };
  static_assert(STAGES == 3, "the loop is written out for three stages");
  using std::integral_constant;
  int kt = 0;
  for (; kt + 4 < ktiles; kt += STAGES) {      // these steps store K steps before the last one: whole chunks only
    step(integral_constant<int, 0>{}, std::false_type{}, kt);
    step(integral_constant<int, 1>{}, std::false_type{}, kt + 1);
    step(integral_constant<int, 2>{}, std::false_type{}, kt + 2);
  }
  if (kt < ktiles) step(integral_constant<int, 0>{}, std::true_type{}, kt);        // one to four steps are left
  if (kt + 1 < ktiles) step(integral_constant<int, 1>{}, std::true_type{}, kt + 1);
  if (kt + 2 < ktiles) step(integral_constant<int, 2>{}, std::true_type{}, kt + 2);
  if (kt + 3 < ktiles) step(integral_constant<int, 0>{}, std::true_type{}, kt + 3);

  // the products were formed transposed: a lane holds four consecutive columns of a row
  const bool vec = MODE == OUT_SWIGLU ? (ldc % 2 == 0 && (uintptr_t)C % 4 == 0)
                 : MODE == OUT_BF16 ? (ldc % 4 == 0 && (uintptr_t)C % 8 == 0)
                                    : (ldc % 4 == 0 && (uintptr_t)C % 16 == 0);
  if constexpr (MODE == OUT_QKV) {
    store_wave_qkv<TM, TN>(C, ldc, M, N, m0 + wm * 32 * TM, n0 + wn * 32 * TN, lane, acc, qkv);
  } else {
    // (a gating product has a copy of the stores for each activation)
    with_gate_activation<MODE>(qkv.gate_act, [&](auto act) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          store_tile_t<MODE, decltype(act)::value>(C, ldc, M, N, m0 + wm * 32 * TM + i * 32 + lrow, n0 + wn * 32 * TN + j * 32,
                                                   lane, acc[i][j], vec);
    });
  }
}

// Scratch that a caller may bring for products with few tiles (see launch_pipelined).
struct Partial {
  float* at = nullptr;
  int64_t floats = 0;
};

// The second kernel of a product whose K was cut over workgroups: adds the `splits`
// partial products (each M x N float32, one after the other) in their order and stores
// the sum the way MODE says.  Four columns a thread; N is a multiple of 4 and the rows of C
// are aligned for it.
// Four columns of the cuts added up in their order: all cuts asked for together, as many as two, four
// or eight (past the last one: a repeat that is not added; with always eight a layer of a prefill of
// 128 to 512 tokens took 1 to 2 % longer).
template <int MOST>
__device__ __forceinline__ f32x4 cuts_added_of(const float* first, int64_t stride, int splits) {
  f32x4 part[MOST];
#pragma unroll
  for (int z = 0; z < MOST; ++z) part[z] = *reinterpret_cast<const f32x4*>(first + (int64_t)min(z, splits - 1) * stride);
  f32x4 sum = part[0];
#pragma unroll
  for (int z = 1; z < MOST; ++z)
    if (z < splits) sum += part[z];
  return sum;
}
__device__ __forceinline__ f32x4 cuts_added(const float* first, int64_t stride, int splits) {
  if (splits <= 2) return cuts_added_of<2>(first, stride, splits);
  if (splits <= 4) return cuts_added_of<4>(first, stride, splits);
  return cuts_added_of<8>(first, stride, splits);
}

template <int MODE>
__global__ __launch_bounds__(256) void gemm_split_finish_kernel(void* __restrict__ C, int64_t ldc,
                                                                const float* __restrict__ partial, int splits,
                                                                int M, int N) {
  const int quads = N >> 2;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)M * quads) return;
  const int m = (int)(idx / quads), n = 4 * (int)(idx - (int64_t)m * quads);
  f32x4 sum = cuts_added(partial + (int64_t)m * N + n, (int64_t)M * N, splits);
  if constexpr (MODE == OUT_BF16) {
    u32x2 o;
    o[0] = (uint32_t)float_to_bf16(sum[0]) | ((uint32_t)float_to_bf16(sum[1]) << 16);
    o[1] = (uint32_t)float_to_bf16(sum[2]) | ((uint32_t)float_to_bf16(sum[3]) << 16);
    *reinterpret_cast<u32x2*>((bf16_t*)C + (int64_t)m * ldc + n) = o;
  } else {
    f32x4* c = reinterpret_cast<f32x4*>((float*)C + (int64_t)m * ldc + n);
    if constexpr (MODE == OUT_ADD_F32) sum += *c;
    *c = sum;
  }
}

// What comes after a product that adds into the residual stream: the norm of the new rows.
// normed null: no norm.
struct NormAfter {
  bf16_t* normed = nullptr;     // [M, N] bfloat16, rows ldn apart
  int64_t ldn = 0;
  const void* weight = nullptr; // [N]
  bool weight_is_f32 = false;
  float eps = 0.f;
};

// The second kernel of a cut product that adds into the residual stream, together with the
// norm that reads the new rows next: one workgroup a row, which stays in registers between
// the sum of its squares and the scaling.  The same sums in the same order as
// gemm_split_finish_kernel followed by the norm's own kernel.  N a multiple of 4 and at
// most 16 * blockDim.x; rows of C, of the partial products and of normed aligned for
// 16-byte (normed: 8-byte) accesses.
template <typename TW, int NV>
__global__ void gemm_split_finish_norm_kernel(float* __restrict__ C, int64_t ldc, const float* __restrict__ partial,
                                              int splits, int M, int N, bf16_t* __restrict__ normed, int64_t ldn,
                                              const TW* __restrict__ w, float eps) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  f32x4 v[NV];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int n = 4 * (threadIdx.x + i * blockDim.x);
    v[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (n < N) {
      f32x4* c = reinterpret_cast<f32x4*>(C + (int64_t)m * ldc + n);
      const f32x4 old = *c;
      f32x4 sum = cuts_added(partial + (int64_t)m * N + n, (int64_t)M * N, splits);
      sum += old;
      *c = sum;
      v[i] = sum;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) ss = fmaf(v[i][e], v[i][e], ss);
  }
  ss = block_sum(ss, scratch);
  const float scale = 1.0f / sqrtf(ss / (float)N + eps);
  bf16_t* o = normed + (int64_t)m * ldn;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int n = 4 * (threadIdx.x + i * blockDim.x);
    if (n < N) {
      u32x2 y;
      y[0] = (uint32_t)float_to_bf16(v[i][0] * scale * to_float<TW>(w[n])) |
             ((uint32_t)float_to_bf16(v[i][1] * scale * to_float<TW>(w[n + 1])) << 16);
      y[1] = (uint32_t)float_to_bf16(v[i][2] * scale * to_float<TW>(w[n + 2])) |
             ((uint32_t)float_to_bf16(v[i][3] * scale * to_float<TW>(w[n + 3])) << 16);
      *reinterpret_cast<u32x2*>(o + n) = y;
    }
  }
}

// Launches it; false if the sizes do not fit it (nothing has been launched then).
inline bool launch_finish_norm(float* C, int64_t ldc, const float* partial, int splits, int M, int N,
                               const NormAfter& norm, hipStream_t stream) {
  const int threads = N >= 2048 ? 512 : 256;
  if (N % 4 != 0 || N > 16 * threads || norm.ldn % 4 != 0 || (uintptr_t)norm.normed % 8 != 0) return false;
  const int nv = (N + 4 * threads - 1) / (4 * threads);          // 1 .. 4
#define GO(TW)                                                                                                   \
  do {                                                                                                           \
    if (nv <= 1) gemm_split_finish_norm_kernel<TW, 1><<<M, threads, 0, stream>>>(C, ldc, partial, splits, M, N, norm.normed, norm.ldn, (const TW*)norm.weight, norm.eps);      \
    else if (nv == 2) gemm_split_finish_norm_kernel<TW, 2><<<M, threads, 0, stream>>>(C, ldc, partial, splits, M, N, norm.normed, norm.ldn, (const TW*)norm.weight, norm.eps); \
    else gemm_split_finish_norm_kernel<TW, 4><<<M, threads, 0, stream>>>(C, ldc, partial, splits, M, N, norm.normed, norm.ldn, (const TW*)norm.weight, norm.eps);              \
  } while (0)
  if (norm.weight_is_f32) GO(float);
  else GO(bf16_t);
#undef GO
  return true;
}

template <int MODE>
int raise_pipelined_lds(size_t lds) {
  static bool raised = false;
  if (!raised) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_bf16_pipelined_kernel<MODE, 2, 2, 3>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return fail("gemm_bf16: cannot raise the LDS limit: %s", hipGetErrorString(e));
    raised = true;
  }
  return 0;
}

// How many cuts the kernel of 256 x 128 tiles makes of such a product (0: it is not one of its
// cases): its loop runs at 1.2 PFLOP/s where the 128 x 128 kernel's, two workgroups a CU, reaches
// 0.7 (the down product of the 1B shape at 2,048 rows, N 2,048, K 8,192 in two cuts: 95 us
// against 70).  Its tiles are half as many: with up to eight cuts they must fill most of the chip
// and not more than the chip, a cut must be 1,024 columns at least (two cuts: K of 4,096 at
// least), and the rows may be padded to whole tiles of 256 by a third over their tiles of 128
// (measured with a tenth, a fifth and a third, and with five, six and eight cuts at most, on the
// narrow products of the 8B, 13B, 1B and 3B shapes at 160 to 1,280 rows, us with the kernel that adds
// the cuts: N 4,096, K 14,336 at 160 to 256 rows 57 to 59 -> 47 to 51, at 384 rows 78 -> 69, at 640
// 110 -> 101, at 896 148 -> 115; N 5,120, K 13,824 at 640 rows 140 -> 106; N 6,144, K 4,096 at 160 to 256
// rows 38 to 39 -> 33 to 34; one case lost, N 2,048, K 8,192 at 384 rows 38.7 -> 41.4).
inline int large_tile_cuts(int M, int N, int K) {
  if (M <= 16 || K % 64 != 0 || N % 4 != 0) return 0;
  const int64_t rows256 = (int64_t)((M + 255) / 256) * 256, rows128 = (int64_t)((M + 127) / 128) * 128;
  if (rows256 * 3 > rows128 * 4) return 0;
  const int64_t tiles = (int64_t)((N + 127) / 128) * (rows256 / 256);
  if (tiles > 128) return 0;
  int cuts = (int)(256 / tiles);
  if (cuts > 8) cuts = 8;
  while (cuts >= 2 && K / cuts < 1024) --cuts;
  if (cuts < 2 || tiles * cuts < 192 || (cuts == 2 && K < 4096)) return 0;
  const int k_split = ((K + cuts - 1) / cuts + 63) / 64 * 64;
  return (K + k_split - 1) / k_split;
}

inline bool cuts_by_large_tiles(int M, int N, int K, int splits) { return splits > 1 && large_tile_cuts(M, N, K) == splits; }

// One round of at most 256 tiles of 128 x 128 by the kernel that loads straight into LDS is faster
// whole than in cuts once the tiles are many for the length of K: the cuts' partial products and the kernel
// that adds them cost more than the idle CUs (us, whole against cut, the cut ones with the norm that their
// adding kernel does: N 3,072, K 2,048 at 256 / 512 / 1,024 rows 22.5 / 23.2 / 25.0 against 24.6 / 30.6 / 34.0;
// N 2,048, K 2,048 at 768 / 1,024 rows 30.4 / 31.0 against 33.8 / 40.9; N 6,144, K 4,096 at 384 / 512 rows 35.6 /
// 36.0 against 42.4 / 43.0; N 4,096, K 4,096 at 768 / 1,024 rows 46.2 / 49.9 against 49.3 / 55.3, but at 512 rows
// 42.6 against 40.7; N 5,120, K 5,120 at 768 rows 55.9 against 58.4, at 512 rows 50.3 against 48.5; from
// K = 8,192 on the cuts win at every number of rows).  Inside a prefill only the short K keeps the gain: a
// layer of the 1B shape at 1,024 / 2,048 rows 226 / 354 -> 214 / 346 us, of the 3B shape at 1,024 rows 299 -> 293,
// but of the 8B shape at 512 rows 287 -> 290 and of the 13B shape at 768 rows 534 -> 540 (there the kernel
// that adds the cuts is the rotation or the norm, which run anyway): whole below K = 4,096 only.
inline bool whole_in_one_round(int M, int N, int K, int64_t tiles) {
  return M > 64 && K % 64 == 0 && K < 4096 && tiles <= 256 && tiles * 4096 >= (int64_t)144 * K &&
         (int64_t)M * K < (1ll << 30) && (int64_t)N * K < (1ll << 30);
}

// How many ways K is cut for M x N x K (1: not at all): the large tiles' cuts where they apply;
// else through 128 x 128 tiles: with fewer than 256 of them (384 where K is long) a part of the
// chip stands idle while a few workgroups walk the whole of K (the output and down products of a
// prompt of 128 tokens: 32 tiles); the cut makes up to 512 workgroups of them, each with at least
// 512 columns.
inline int pipelined_splits(int M, int N, int K) {
  const int64_t tiles = (int64_t)((N + 127) / 128) * ((M + 127) / 128);
  if (whole_in_one_round(M, N, K, tiles)) return 1;
  if (const int cuts = large_tile_cuts(M, N, K); cuts > 1 && K >= 2048) return cuts;
  const bool long_k = K >= 8192;
  if (M <= 16 || tiles >= (long_k ? 384 : 256) || K < 2048 || N % 4 != 0) return 1;
  // (a short K in three or four cuts is a few steps between a prologue and an epilogue: with more than 96
  // tiles the whole product is faster, N 3,072, K 2,048 at 768 rows 31.7 us against 35.9, N 2,048 at 1,024 rows
  // 35.9 against 38.5; at K = 3,072 the cuts still win, 37.5 against 47)
  if (K < 3072 && tiles > 96) return 1;
  // (two workgroups of this kernel fit a CU; measured, a prompt of 128 tokens is faster with one a CU
  // and fewer partial products, one of 512 tokens with two; two cuts only pay where K is long)
  // (measured at 128 to 512 rows on the three narrow products of the 8B shape, µs for the pair of
  // kernels: 48 tiles in 5 cuts 24, in 8 cuts 31; 64 tiles in 4 cuts 25, in 6 cuts 30; 96 tiles whole
  // 46, in 3 cuts 38 to 41, in 5 cuts 32 to 36; 144 tiles in 2 cuts 50, in 3 cuts 42, in 4 cuts 51)
  int splits = tiles < 86 ? (int)(256 / tiles) : tiles < 256 ? (int)(512 / tiles) : 2;
  if (splits > 8) splits = 8;
  if (splits > K / 512) splits = K / 512;
  if (splits < 2 || (splits == 2 && !long_k)) return 1;
  const int k_split = ((K + splits - 1) / splits + 63) / 64 * 64;
  return (K + k_split - 1) / k_split;
}

template <int MODE, int TM, int TN, int NBUF>
int launch_direct64(void* C, int64_t ldc, const bf16_t* A, int64_t lda, const bf16_t* W, int64_t ldw,
                    int M, int N, int K, const QkvArgs& qkv, hipStream_t stream, int k_split = 0, int splits = 1,
                    int64_t split_stride = 0);
inline bool large_fits(int64_t lda, int64_t ldw, int M, int N, int K);

template <int MODE>
int launch_pipelined(void* C, int64_t ldc, const bf16_t* A, int64_t lda, const bf16_t* W, int64_t ldw,
                     int M, int N, int K, const QkvArgs& qkv, hipStream_t stream,
                     const Partial& partial = Partial{}, const NormAfter& norm = NormAfter{}, bool* normed = nullptr,
                     bool this_kernel_only = false) {
  // 128 x 128 tiles, two workgroups per CU.  (128 x 256 tiles halve the LDS reads per
  // matrix instruction but leave one wave per SIMD, and measured 20 % slower; 128 x 64
  // tiles, which put two workgroups on a CU where 128 x 128 leave one, 15 % slower at 65
  // to 256 rows; the kernel below that loads straight into LDS, with 128 x 128 tiles, level at
  // 128 rows and 3 to 7 % slower at 65 and at 256.)
  constexpr int TM = 2, TN = 2, STAGES = 3;
  const size_t lds = (size_t)2 * (64 * TM + 64 * TN) * PPITCH * sizeof(bf16_t);
  if (raise_pipelined_lds<MODE>(lds)) return 1;
  const int64_t tiles = (int64_t)((N + 64 * TN - 1) / (64 * TN)) * ((M + 64 * TM - 1) / (64 * TM));
  if (tiles > (1 << 30)) return fail("gemm_bf16: too many tiles");
  dim3 grid((unsigned)((tiles + XCDS - 1) / XCDS * XCDS));
  if constexpr (MODE == OUT_BF16 || MODE == OUT_F32 || MODE == OUT_ADD_F32) {
    const int splits = pipelined_splits(M, N, K);
    const bool rows_fit = MODE == OUT_BF16 ? (ldc % 4 == 0 && (uintptr_t)C % 8 == 0) : (ldc % 4 == 0 && (uintptr_t)C % 16 == 0);
    if (splits > 1 && rows_fit && partial.at != nullptr && (uintptr_t)partial.at % 16 == 0 &&
        partial.floats >= (int64_t)splits * M * N) {
      if (raise_pipelined_lds<OUT_F32>(lds)) return 1;
      const int k_split = ((K + splits - 1) / splits + 63) / 64 * 64;
      if (cuts_by_large_tiles(M, N, K, splits) && large_fits(lda, ldw, M, N, K)) {
        if (launch_direct64<OUT_F32, 4, 2, 3>(partial.at, N, A, lda, W, ldw, M, N, K, qkv, stream, k_split, splits,
                                              (int64_t)M * N))
          return 1;
      } else if (large_fits(lda, ldw, M, N, K)) {
        // (the kernel that loads straight into LDS, with 128 x 128 tiles: 2 to 4 us less than the one below
        // for every cut product of 65 to 512 rows of the 8B, 13B, 3B and 1B shapes, 20 to 50 us each)
        if (launch_direct64<OUT_F32, 2, 2, 3>(partial.at, N, A, lda, W, ldw, M, N, K, qkv, stream, k_split, splits,
                                              (int64_t)M * N))
          return 1;
      } else {
        grid.y = splits;
        gemm_bf16_pipelined_kernel<OUT_F32, TM, TN, STAGES><<<grid, 256, lds, stream>>>(
            partial.at, N, A, lda, W, ldw, M, N, K, qkv, k_split, (int64_t)M * N);
      }
      if constexpr (MODE == OUT_ADD_F32) {
        if (norm.normed != nullptr && launch_finish_norm((float*)C, ldc, partial.at, splits, M, N, norm, stream)) {
          *normed = true;
          return 0;
        }
      }
      const int64_t threads = (int64_t)M * (N / 4);
      gemm_split_finish_kernel<MODE><<<(unsigned)((threads + 255) / 256), 256, 0, stream>>>(C, ldc, partial.at, splits, M, N);
      return 0;
    }
  }
  // (one round of tiles, a workgroup a CU: the kernel that loads straight into LDS, a quarter faster
  // than two workgroups a CU of the one below: N 3,072, K 2,048 at 1,024 rows 25.2 us against 34.5, N 2,048,
  // K 2,048 at 2,048 rows 31.9 against 41.5, N 4,096, K 4,096 at 1,024 rows 44.1 against 59.8; with more
  // tiles than CUs it is the slower one, 39.0 against 34.1 and 49.8 against 42.1)
  if (!this_kernel_only && tiles <= 256 && large_fits(lda, ldw, M, N, K))
    return launch_direct64<MODE, 2, 2, 3>(C, ldc, A, lda, W, ldw, M, N, K, qkv, stream);
  gemm_bf16_pipelined_kernel<MODE, TM, TN, STAGES><<<grid, 256, lds, stream>>>(C, ldc, A, lda, W, ldw, M, N, K, qkv, 0, 0);
  return 0;
}

// acc += w x for the 16 x 16 x 32 matrix instruction, written as the instruction itself with
// the accumulator tied to one place in the accumulation registers: given the intrinsic for 48 or
// 64 accumulators of four registers in a loop of two alternating operand sets, the compiler
// moved them from place to place (three hundred register moves a K step, and spills).  What
// the compiler then no longer knows, and the hardware does not check: the result may be read
// by another kind of instruction only some cycles after the last matrix instruction
// (accumulators_settle, once behind the loop); between matrix instructions on one accumulator
// there are 47 others here, and the operands' waits the compiler still counts itself.
__device__ __forceinline__ void multiply_16x16x32(f32x4& acc, const bf16x8& w, const bf16x8& x) {
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(w), "v"(x));
}

__device__ __forceinline__ void accumulators_settle() {
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);       // (no read of an accumulator is moved up in front of the wait)
}

// ------------------------------------ tiled, one wave a SIMD, loads into the LDS ---
// Products with enough tiles of 256 rows to fill the chip.  A 128 x 128 tile at the
// full matrix rate asks the L1 for 64 bytes a clock, which is all a CU has, and the LDS
// for one 16-byte read per lane and matrix instruction; a wave tile of 128 x 128
// (TM = TN = 4: 256 accumulator registers, so one wave a SIMD) halves both.
//
// With one wave a SIMD nothing hides latency but distance and the order of issue:
//  * A K step (32 columns) goes from global memory straight into the LDS
//    (buffer_load_dwordx4 ... lds: lane l of a wave writes bytes 16 l .. 16 l + 15 of a
//    1 KB block), so no register stage and no LDS write instruction stands between the
//    matrix instructions.  Four LDS buffers of one K step each: a step is asked from
//    memory four steps before it is multiplied, and read into registers one step before.
//  * A 1 KB block is 16 tile rows of 64 bytes, unpadded; the four 16-byte chunks of row
//    r are stored in the order c ^ f(r), f(r) = bit 3 of r | bit 2 of r << 1: of the
//    functions whose bits are parities of row bits, the hardware's conflict counter
//    showed none for this one on a wave's 16-byte operand reads of 32 rows (rows lane % 32,
//    chunks 2 ks + lane / 32, the operand of the 32 x 32 x 16 instruction), and two-way
//    conflicts for e.g. ((r >> 1) ^ (r >> 3)) & 3; an operand of the 16 x 16 x 32 instruction
//    is one such block whole (row lane % 16, chunk lane / 16), every bank once whatever f.
//  * The one barrier of a step stands where the wave has nothing outstanding in the LDS,
//    and carries no fence (a fence would wait for every load in flight); what must have
//    landed is waited for by count.
//  * The order of issue is written out and pinned, every matrix instruction and what follows
//    it between two scheduling barriers: what does not stand between two matrix
//    instructions is not overlapped with them, and a burst of requests from four waves in
//    step queues at the CU's one address unit while the matrix pipes run dry.
//  * The kernel is bound by power, not by its schedule.  With the 32 x 32 x 16 instruction, by
//    the cycle counter and the constant-rate counter read around the loop (K = 8,192, all CUs
//    busy): a loop of the matrix instructions alone took 32.7 cycles an instruction at 1.82
//    GHz; with the LDS reads and the barrier 36.7 at 1.68; with the requests too, all to one
//    address, 37.3 at 1.47; the whole loop 36.0 at 1.39 (38.9 at 1.42 while the requests of a
//    step stood together under a quarter of its matrix instructions); after an idle gap the
//    same loop ran at 1.94 GHz and 54.6 cycles an instruction, the same 0.85 us a step; three,
//    four or five LDS buffers made no difference.  Hence the 16 x 16 x 32 instruction (see the
//    kernel): the same loop 18.4 cycles an instruction of half the size at 1.55 GHz, 195 us
//    where it took 212.
//  * The products are formed transposed (weights as the row operand): a lane then holds
//    four consecutive columns of one row of C and stores them with one instruction.
// K must be a multiple of 32 and every row's byte offset must fit 31 bits.
constexpr int DBK = 32, DROW = DBK * 2;      // bytes of a tile row in a buffer

// A workgroup barrier without a fence.  The barrier instruction does not count as a
// memory access for the compiler, so the empty statements on both sides keep the LDS
// reads and the loads into the LDS where they were written, relative to it.
__device__ __forceinline__ void barrier_no_fence() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

__device__ __forceinline__ uint32_t swizzle(uint32_t row) { return ((row >> 3) & 1u) | ((row >> 1) & 2u); }

template <int MODE, int TM, int TN>
__global__ __launch_bounds__(256) void gemm_bf16_direct_kernel(void* __restrict__ C, int64_t ldc,
                                                               const bf16_t* __restrict__ A, int64_t lda,
                                                               const bf16_t* __restrict__ W, int64_t ldw,
                                                               int M, int N, int K, QkvArgs qkv) {
#if defined(__HIP_DEVICE_COMPILE__)   // the host pass has no buffer resources; it only needs the stub
  constexpr int BM = 64 * TM, BN = 64 * TN, CA = BM / 64, CW = BN / 64;
  constexpr int BUF = (BM + BN) * DROW;            // bytes of one LDS buffer (A tile, then W tile)
  extern __shared__ __attribute__((aligned(1024))) char lds_bytes[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  int m0, n0;
  {
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const int total = tiles_m * tiles_n, per_xcd = (total + XCDS - 1) / XCDS;
    const int t = (int)(blockIdx.x % XCDS) * per_xcd + (int)(blockIdx.x / XCDS);
    if (t >= total) return;
    m0 = (t % tiles_m) * BM;
    n0 = (t / tiles_m) * BN;
  }
  // A wave's load p fills tile rows 64 p + 16 wave .. + 15: lane -> row lane / 4, LDS chunk lane % 4,
  // which holds the row's chunk (lane % 4) ^ f(row).  Rows beyond the edge read the last row.
  const int lr = 64 * 0 + 16 * wave + (lane >> 2);             // row within the first 64 rows
  uint32_t a_off[CA], w_off[CW];
#pragma unroll
  for (int p = 0; p < CA; ++p) {
    const uint32_t row = (uint32_t)(lr + 64 * p), chunk = (uint32_t)(lane & 3) ^ swizzle(row);
    a_off[p] = (uint32_t)(((int64_t)min(m0 + (int)row, M - 1) * lda + chunk * 8) * 2);
  }
#pragma unroll
  for (int p = 0; p < CW; ++p) {
    const uint32_t row = (uint32_t)(lr + 64 * p), chunk = (uint32_t)(lane & 3) ^ swizzle(row);
    w_off[p] = (uint32_t)(((int64_t)min(n0 + (int)row, N - 1) * ldw + chunk * 8) * 2);
  }
  const int ktiles = K / DBK;
  // Buffer loads: the row offset is a 32-bit register that never changes, the K step a
  // scalar; nothing is computed per load.  (0x00020000: a raw buffer of 32-bit data.)
  typedef __attribute__((address_space(3))) void* lds_ptr;
  const __amdgpu_buffer_rsrc_t a_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)A, 0, (int)(((int64_t)(M - 1) * lda + K) * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t w_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)W, 0, (int)(((int64_t)(N - 1) * ldw + K) * 2), 0x00020000);
  auto load_one = [&](int kt, int p) {            // request p of K step kt: CA of A, then CW of W
    const int koff = min(kt, ktiles - 1) * DROW;          // past the end: a repeat that nobody uses
    char* dst = lds_bytes + (kt & 3) * BUF + wave * 1024;
    if (p < CA) __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (lds_ptr)(dst + p * 4096), 16, a_off[p], koff, 0, 0);
    else __builtin_amdgcn_raw_ptr_buffer_load_lds(w_rsrc, (lds_ptr)(dst + BM * DROW + (p - CA) * 4096), 16, w_off[p - CA], koff, 0, 0);
  };
  auto load_step = [&](int kt) {
#pragma unroll
    for (int p = 0; p < CA + CW; ++p) load_one(kt, p);
  };

  // The matrix instruction is the 16 x 16 x 32 one: with operands as real ones are, the GPU
  // sustains 2.1 PFLOP/s of it where it sustains 1.76 of the 32 x 32 x 16 one (both 2.5 on zeros):
  // it passes an accumulator through the matrix pipe half as often for the same products, and the
  // products of a layer are bound by power.  A wave's tile is TM16 x TN16 tiles of 16 x 16.
  constexpr int TM16 = 2 * TM, TN16 = 2 * TN;
  f32x4 acc[TM16][TN16];
#pragma unroll
  for (int i = 0; i < TM16; ++i)
#pragma unroll
    for (int j = 0; j < TN16; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // An operand of the instruction is 16 tile rows x 32 columns, a whole K step of a 1 KB block:
  // lane l reads row l % 16, columns 8 (l / 16) .. + 7, which lie at chunk (l / 16) ^ f(row)
  // (f depends on bits 2 and 3 of the row, which are the lane's own: blocks start at multiples of 16)
  const int lrow = lane & 15;
  const uint32_t rd = (uint32_t)(lrow * DROW) + ((((uint32_t)lane >> 4) ^ swizzle((uint32_t)lrow)) << 4);
  const uint32_t a_rd = (uint32_t)(wm * 32 * TM * DROW), w_rd = (uint32_t)(BM * DROW + wn * 32 * TN * DROW);
  constexpr int RD = TM16 + TN16, MF = TM16 * TN16, LD = CA + CW;
  bf16x8 a[2][TM16], b[2][TN16];           // two sets: one is multiplied while the next step's is read
  auto read_one = [&](int buf, bf16x8* af, bf16x8* bf, int r) {      // in the order in which the products need them
    const char* tile = lds_bytes + buf * BUF + rd;
    const int j = r - 1, i = r - TN16;
    if (r == 0) af[0] = *reinterpret_cast<const bf16x8*>(tile + a_rd);
    else if (r <= TN16) bf[j] = *reinterpret_cast<const bf16x8*>(tile + w_rd + j * 16 * DROW);
    else af[i] = *reinterpret_cast<const bf16x8*>(tile + a_rd + i * 16 * DROW);
  };

#pragma unroll
  for (int s0 = 0; s0 < 4; ++s0) load_step(s0);
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * LD) : "memory");     // K step 0 has landed
  barrier_no_fence();
#pragma unroll
  for (int r = 0; r < RD; ++r) read_one(0, a[0], b[0], r);

  // One K step: the barrier, then MF matrix instructions on the operands that the step before
  // read, with the reads of the next step's operands under the first half of them and the
  // requests for K step kt + 4 spread over all of them (a request of a kilobyte keeps the CU's
  // one address unit busy for 16 cycles, and the four waves ask at the same time).  The order is
  // written out and pinned: every matrix instruction with what follows it stands between two
  // scheduling barriers.  In front of the barrier this wave's part of K step kt + 1 has landed
  // (it was asked for three steps ago: at most the loads of two steps are outstanding) and its
  // reads of K step kt are done; behind it everybody's, so that step kt + 1 can be read and the
  // buffer of step kt be asked into.  No fence: it would wait for every load in flight.
  constexpr int READ_SPAN = MF / 2;
  auto step = [&](int kt, const bf16x8* af, const bf16x8* bf, bf16x8* raf, bf16x8* rbf) {
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(2 * LD) : "memory");
    barrier_no_fence();
#pragma unroll
    for (int g = 0; g < MF; ++g) {
      const int i = g / TN16, j = g % TN16;
      multiply_16x16x32(acc[i][j], bf[j], af[i]);   // transposed
      if (g < READ_SPAN) {
#pragma unroll
        for (int r = (RD * g) / READ_SPAN; r < (RD * (g + 1)) / READ_SPAN; ++r) read_one((kt + 1) & 3, raf, rbf, r);
      }
#pragma unroll
      for (int l = (LD * g) / MF; l < (LD * (g + 1)) / MF; ++l) load_one(kt + 4, l);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  int kt = 0;
  for (; kt + 1 < ktiles; kt += 2) {
    step(kt, a[0], b[0], a[1], b[1]);
    step(kt + 1, a[1], b[1], a[0], b[0]);
  }
  if (kt < ktiles) step(kt, a[0], b[0], a[1], b[1]);
  accumulators_settle();
  // the repeats asked for past the end still write into this workgroup's LDS: let them
  // land before the wave can end and the LDS go to another workgroup
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  const bool vec = MODE == OUT_SWIGLU ? (ldc % 2 == 0 && (uintptr_t)C % 4 == 0)
                 : MODE == OUT_BF16 ? (ldc % 4 == 0 && (uintptr_t)C % 8 == 0)
                                    : (ldc % 4 == 0 && (uintptr_t)C % 16 == 0);
  if constexpr (MODE == OUT_QKV) {
    store_wave_qkv<TM16, TN16>(C, ldc, M, N, m0 + wm * 32 * TM, n0 + wn * 32 * TN, lane, acc, qkv);
  } else {
    using S = Stage<MODE, TN16, 16>;
    static_assert(4 * S::BYTES <= 4 * BUF, "the waves' strips fit in the LDS of the buffers");
    __syncthreads();      // nobody reads operands from the LDS any more
    const bool whole_rows = (ldc * S::ES) % 16 == 0 && (uintptr_t)C % 16 == 0 && n0 + wn * 32 * TN + 32 * TN <= N;
    // (a gating product has a copy of the stores for each activation)
    with_gate_activation<MODE>(qkv.gate_act, [&](auto act) {
      constexpr int ACT = decltype(act)::value;
      if (whole_rows) {
        store_wave_staged<MODE, TM16, TN16, ACT>(lds_bytes + wave * S::BYTES, C, ldc, M, m0 + wm * 32 * TM, n0 + wn * 32 * TN, lane, acc);
      } else {
#pragma unroll
        for (int i = 0; i < TM16; ++i)
#pragma unroll
          for (int j = 0; j < TN16; ++j)
            store_tile_t<MODE, ACT>(C, ldc, M, N, m0 + wm * 32 * TM + i * 16 + lrow, n0 + wn * 32 * TN + j * 16, lane, acc[i][j], vec);
      }
    });
  }
#endif
}

template <int MODE, int TM, int TN>
int launch_direct(void* C, int64_t ldc, const bf16_t* A, int64_t lda, const bf16_t* W, int64_t ldw,
                  int M, int N, int K, const QkvArgs& qkv, hipStream_t stream) {
  const size_t lds = (size_t)4 * (64 * TM + 64 * TN) * DROW;
  static bool raised = false;
  if (!raised) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_bf16_direct_kernel<MODE, TM, TN>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return fail("gemm_bf16: cannot raise the LDS limit: %s", hipGetErrorString(e));
    raised = true;
  }
  const int64_t tiles = (int64_t)((N + 64 * TN - 1) / (64 * TN)) * ((M + 64 * TM - 1) / (64 * TM));
  dim3 grid((unsigned)((tiles + XCDS - 1) / XCDS * XCDS));
  gemm_bf16_direct_kernel<MODE, TM, TN><<<grid, 256, lds, stream>>>(C, ldc, A, lda, W, ldw, M, N, K, qkv);
  return 0;
}

// The same, with K steps of 64 columns: a tile row is a whole 128-byte line, so the L2
// sees half as many requests, and there is one barrier per 64 columns.  It pays with
// three buffers, which the LDS holds for 256 x 128 tiles (with the two that fit for
// 256 x 256 tiles it measured slower than four buffers of 32 columns).
constexpr int EROW = 128;                    // bytes of a tile row in a buffer
// depends on the low five bits of the row only: a lane's operand rows are 32 apart
__device__ __forceinline__ uint32_t swizzle8(uint32_t row) { return (row ^ ((row >> 3) & 3u)) & 7u; }

// (CUT is a compile-time choice: the kernel of whole products holds no trace of it)
template <int MODE, int TM, int TN, int NBUF, bool CUT = false>
__global__ __launch_bounds__(256) void gemm_bf16_direct64_kernel(void* __restrict__ C, int64_t ldc,
                                                                 const bf16_t* __restrict__ A, int64_t lda,
                                                                 const bf16_t* __restrict__ W, int64_t ldw,
                                                                 int M, int N, int K, QkvArgs qkv, int k_split,
                                                                 int64_t split_stride) {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int BM = 64 * TM, BN = 64 * TN, CA = BM / 32, CW = BN / 32;
  constexpr int BUF = (BM + BN) * EROW;
  if constexpr (CUT) {
    // K cut over workgroups: blockIdx.y takes columns blockIdx.y * k_split .. of A and W (a multiple
    // of 64) and leaves its partial product, float32, split_stride words after the one before
    const int k_first = (int)blockIdx.y * k_split;
    A += k_first;
    W += k_first;
    K = min(K - k_first, k_split);
    C = (void*)((float*)C + (int64_t)blockIdx.y * split_stride);
  }
  extern __shared__ __attribute__((aligned(1024))) char lds_bytes[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  int m0, n0;
  {
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const int total = tiles_m * tiles_n, per_xcd = (total + XCDS - 1) / XCDS;
    const int t = (int)(blockIdx.x % XCDS) * per_xcd + (int)(blockIdx.x / XCDS);
    if (t >= total) return;
    m0 = (t % tiles_m) * BM;
    n0 = (t / tiles_m) * BN;
  }
  // A wave's load p fills tile rows 32 p + 8 wave .. + 7: lane -> row lane / 8, LDS chunk lane % 8,
  // which holds the row's chunk (lane % 8) ^ f(row).
  const int lr = 8 * wave + (lane >> 3);
  uint32_t a_off[CA], w_off[CW];
#pragma unroll
  for (int p = 0; p < CA; ++p) {
    const uint32_t row = (uint32_t)(lr + 32 * p), chunk = (uint32_t)(lane & 7) ^ swizzle8(row);
    a_off[p] = (uint32_t)(((int64_t)min(m0 + (int)row, M - 1) * lda + chunk * 8) * 2);
  }
#pragma unroll
  for (int p = 0; p < CW; ++p) {
    const uint32_t row = (uint32_t)(lr + 32 * p), chunk = (uint32_t)(lane & 7) ^ swizzle8(row);
    w_off[p] = (uint32_t)(((int64_t)min(n0 + (int)row, N - 1) * ldw + chunk * 8) * 2);
  }
  const int ktiles = K / 64;
  typedef __attribute__((address_space(3))) void* lds_ptr;
  const __amdgpu_buffer_rsrc_t a_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)A, 0, (int)(((int64_t)(M - 1) * lda + K) * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t w_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)W, 0, (int)(((int64_t)(N - 1) * ldw + K) * 2), 0x00020000);
  auto load_one = [&](int kt, int buf, int p) {     // request p of K step kt: CA of A, then CW of W
    const int koff = min(kt, ktiles - 1) * EROW;         // past the end: a repeat that nobody uses
    char* dst = lds_bytes + buf * BUF + wave * 1024;
    if (p < CA) __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (lds_ptr)(dst + p * 4096), 16, a_off[p], koff, 0, 0);
    else __builtin_amdgcn_raw_ptr_buffer_load_lds(w_rsrc, (lds_ptr)(dst + BM * EROW + (p - CA) * 4096), 16, w_off[p - CA], koff, 0, 0);
  };
  auto load_step = [&](int kt, int buf) {
#pragma unroll
    for (int p = 0; p < CA + CW; ++p) load_one(kt, buf, p);
  };

  // (the 16 x 16 x 32 matrix instruction, as in the kernel above: TM16 x TN16 tiles of 16 x 16 a wave)
  constexpr int TM16 = 2 * TM, TN16 = 2 * TN;
  f32x4 acc[TM16][TN16];
#pragma unroll
  for (int i = 0; i < TM16; ++i)
#pragma unroll
    for (int j = 0; j < TN16; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // An operand is 16 tile rows x 32 columns, half of the 64 columns of a step: lane l reads row
  // l % 16, columns 32 kc + 8 (l / 16) .. + 7, which lie at chunk (4 kc + l / 16) ^ f(row); f takes
  // bit 4 of the row too, which is the parity of the block of 16 rows.
  const int lrow = lane & 15;
  uint32_t rd[2][2];       // [half of the step][parity of the block of 16 rows]
#pragma unroll
  for (int kc = 0; kc < 2; ++kc)
#pragma unroll
    for (int odd = 0; odd < 2; ++odd)
      rd[kc][odd] = (uint32_t)(lrow * EROW) + (((uint32_t)(kc * 4 + (lane >> 4)) ^ swizzle8((uint32_t)(lrow + 16 * odd))) << 4);
  const uint32_t a_rd = (uint32_t)(wm * 32 * TM * EROW), w_rd = (uint32_t)(BM * EROW + wn * 32 * TN * EROW);
  constexpr int RD = TM16 + TN16, MF = TM16 * TN16, LD = CA + CW;
  static_assert(LD % 2 == 0, "a step's requests go out in two halves");
  bf16x8 a[2][TM16], b[2][TN16];           // one set a half step: one is multiplied while the next is read
  auto read_one = [&](int buf, int kc, bf16x8* af, bf16x8* bf, int r) {      // in the order in which the products need them
    const char* tile = lds_bytes + buf * BUF;
    const int j = r - 1, i = r - TN16;
    if (r == 0) af[0] = *reinterpret_cast<const bf16x8*>(tile + a_rd + rd[kc][0]);
    else if (r <= TN16) bf[j] = *reinterpret_cast<const bf16x8*>(tile + w_rd + j * 16 * EROW + rd[kc][j & 1]);
    else af[i] = *reinterpret_cast<const bf16x8*>(tile + a_rd + i * 16 * EROW + rd[kc][i & 1]);
  };

  // steps 0 and 1 and the first half of step 2 (the rule below: the second half of step kt + 2 goes
  // out under the first half of step kt)
#pragma unroll
  for (int s0 = 0; s0 < 2; ++s0) load_step(s0, s0);
#pragma unroll
  for (int p = 0; p < LD / 2; ++p) load_one(2, 2, p);
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LD + LD / 2) : "memory");     // K step 0 has landed
  barrier_no_fence();
#pragma unroll
  for (int r = 0; r < RD; ++r) read_one(0, 0, a[0], b[0], r);

  // One step of 64 columns in two halves of MF matrix instructions with the barrier between
  // them; the order is written out and pinned (every matrix instruction with what follows it
  // stands between two scheduling barriers).  Under a half's first matrix instructions go the
  // reads of the next half's operands.  Requests, one for every fifth matrix instruction or so (a
  // request of a kilobyte keeps the CU's one address unit busy for 16 cycles, and the four waves
  // ask at the same time): under the first half the second half of K step kt + 2 (its buffer was
  // last read in step kt - 1, before that step's barrier), under the second half the first half
  // of K step kt + 3, into this step's buffer, which nobody reads behind the barrier.  In front
  // of the barrier this wave's part of K step kt + 1 has landed when at most the loads of one
  // step are outstanding; behind it everybody's has.  No fence: it would wait for every load.
  static_assert(NBUF == 3, "the requests' order is written for three buffers");
  constexpr int READ_SPAN = MF / 2;
  auto half = [&](const bf16x8* af, const bf16x8* bf, int rbuf, int rkc, bf16x8* raf, bf16x8* rbf, int kt_load, int lbuf, int l0) {
#pragma unroll
    for (int g = 0; g < MF; ++g) {
      const int i = g / TN16, j = g % TN16;
      multiply_16x16x32(acc[i][j], bf[j], af[i]);   // transposed
      if (g < READ_SPAN) {
#pragma unroll
        for (int r = (RD * g) / READ_SPAN; r < (RD * (g + 1)) / READ_SPAN; ++r) read_one(rbuf, rkc, raf, rbf, r);
      }
#pragma unroll
      for (int l = (LD / 2 * g) / MF; l < (LD / 2 * (g + 1)) / MF; ++l) load_one(kt_load, lbuf, l0 + l);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  int rb = 0;                                   // kt % NBUF
  for (int kt = 0; kt < ktiles; ++kt) {
    const int lb = rb == 0 ? NBUF - 1 : rb - 1, nb = rb == NBUF - 1 ? 0 : rb + 1;
    half(a[0], b[0], rb, 1, a[1], b[1], kt + 2, lb, LD / 2);
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(LD) : "memory");
    barrier_no_fence();
    half(a[1], b[1], nb, 0, a[0], b[0], kt + 3, rb, 0);
    rb = nb;
  }
  accumulators_settle();
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  const bool vec = MODE == OUT_SWIGLU ? (ldc % 2 == 0 && (uintptr_t)C % 4 == 0)
                 : MODE == OUT_BF16 ? (ldc % 4 == 0 && (uintptr_t)C % 8 == 0)
                                    : (ldc % 4 == 0 && (uintptr_t)C % 16 == 0);
  if constexpr (MODE == OUT_QKV) {
    store_wave_qkv<TM16, TN16>(C, ldc, M, N, m0 + wm * 32 * TM, n0 + wn * 32 * TN, lane, acc, qkv);
  } else {
    using S = Stage<MODE, TN16, 16>;
    static_assert(4 * S::BYTES <= NBUF * BUF, "the waves' strips fit in the LDS of the buffers");
    __syncthreads();      // nobody reads operands from the LDS any more
    const bool whole_rows = (ldc * S::ES) % 16 == 0 && (uintptr_t)C % 16 == 0 && n0 + wn * 32 * TN + 32 * TN <= N;
    // (a gating product has a copy of the stores for each activation)
    with_gate_activation<MODE>(qkv.gate_act, [&](auto act) {
      constexpr int ACT = decltype(act)::value;
      if (whole_rows) {
        store_wave_staged<MODE, TM16, TN16, ACT>(lds_bytes + wave * S::BYTES, C, ldc, M, m0 + wm * 32 * TM, n0 + wn * 32 * TN, lane, acc);
      } else {
#pragma unroll
        for (int i = 0; i < TM16; ++i)
#pragma unroll
          for (int j = 0; j < TN16; ++j)
            store_tile_t<MODE, ACT>(C, ldc, M, N, m0 + wm * 32 * TM + i * 16 + lrow, n0 + wn * 32 * TN + j * 16, lane, acc[i][j], vec);
      }
    });
  }
#endif
}

// (k_split > 0: K in `splits` cuts of k_split columns, MODE a float32 store, the partial products
// split_stride words apart from C on)
template <int MODE, int TM, int TN, int NBUF>
int launch_direct64(void* C, int64_t ldc, const bf16_t* A, int64_t lda, const bf16_t* W, int64_t ldw,
                    int M, int N, int K, const QkvArgs& qkv, hipStream_t stream, int k_split, int splits,
                    int64_t split_stride) {
  const size_t lds = (size_t)NBUF * (64 * TM + 64 * TN) * EROW;
  static bool raised = false;
  if (!raised) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_bf16_direct64_kernel<MODE, TM, TN, NBUF, false>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e == hipSuccess)
      e = hipFuncSetAttribute((const void*)gemm_bf16_direct64_kernel<MODE, TM, TN, NBUF, true>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return fail("gemm_bf16: cannot raise the LDS limit: %s", hipGetErrorString(e));
    raised = true;
  }
  const int64_t tiles = (int64_t)((N + 64 * TN - 1) / (64 * TN)) * ((M + 64 * TM - 1) / (64 * TM));
  dim3 grid((unsigned)((tiles + XCDS - 1) / XCDS * XCDS), k_split > 0 ? splits : 1);
  if (k_split > 0)
    gemm_bf16_direct64_kernel<MODE, TM, TN, NBUF, true><<<grid, 256, lds, stream>>>(C, ldc, A, lda, W, ldw, M, N, K, qkv,
                                                                                   k_split, split_stride);
  else
    gemm_bf16_direct64_kernel<MODE, TM, TN, NBUF, false><<<grid, 256, lds, stream>>>(C, ldc, A, lda, W, ldw, M, N, K, qkv,
                                                                                    0, 0);
  return 0;
}

// The large tiles take a product whose K is a multiple of 64, whose byte offsets fit 32
// bits, and which has enough of them.
inline bool large_fits(int64_t lda, int64_t ldw, int M, int N, int K) {
  return K % 64 == 0 && (int64_t)M * lda < (1ll << 30) && (int64_t)N * ldw < (1ll << 30);
}

// ------------------------------------------------------------------ skinny ---
constexpr int SK_WAVES = 8, SK_ROWS = 16, SK_UNROLL = 4;

// MT: number of 16-row groups of the batch (M <= 16 * MT).
template <int MODE, bool VEC, int MT>
__global__ __launch_bounds__(SK_WAVES * 64) void gemm_bf16_skinny_kernel(
    void* __restrict__ C, int64_t ldc, const bf16_t* __restrict__ A, int64_t lda,
    const bf16_t* __restrict__ W, int64_t ldw, int M, int N, int K) {
  __shared__ float partial[SK_WAVES][MT][64][4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r16 = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * SK_ROWS;
  const bool w_ok = n0 + r16 < N;
  const bf16_t* w_row = W + (int64_t)(w_ok ? n0 + r16 : 0) * ldw;
  const bf16_t* x_row[MT];
  bool x_ok[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    x_ok[t] = t * 16 + r16 < M;
    x_row[t] = A + (int64_t)(x_ok[t] ? t * 16 + r16 : 0) * lda;
  }

  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

  constexpr int KBLOCK = 32 * SK_UNROLL;
  for (int kb = wave * KBLOCK; kb < K; kb += SK_WAVES * KBLOCK) {
    Chunk w[SK_UNROLL];
#pragma unroll
    for (int s = 0; s < SK_UNROLL; ++s) w[s] = load_chunk<VEC>(w_row, w_ok, kb + s * 32 + g * 8, K);
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      Chunk x[SK_UNROLL];
#pragma unroll
      for (int s = 0; s < SK_UNROLL; ++s) x[s] = load_chunk<VEC>(x_row[t], x_ok[t], kb + s * 32 + g * 8, K);
#pragma unroll
      for (int s = 0; s < SK_UNROLL; ++s)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[s].v, x[s].v, acc[t], 0, 0, 0);
    }
  }

#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) partial[wave][t][lane][i] = acc[t][i];
  __syncthreads();
  // D layout of the 16x16 tile: register i of lane l is weight row 4*(l/16) + i, batch row l%16
  for (int idx = threadIdx.x; idx < MT * 64; idx += SK_WAVES * 64) {
    const int t = idx >> 6, l = idx & 63;
    const int m = t * 16 + (l & 15);
    if (m >= M) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = n0 + 4 * (l >> 4) + i;
      if (n >= N) continue;
      float s = 0.f;
#pragma unroll
      for (int w = 0; w < SK_WAVES; ++w) s += partial[w][t][l][i];
      store_out<MODE>(C, ldc, m, n, s);
    }
  }
}

// Which tiled kernel takes an aligned product: force_kernel 2 the 128 x 128 tiles, 4 the
// 256 x 256 tiles, 5 the 256 x 128 tiles, 6 the 256 x 192 tiles, 7 and 8 the 128 x 128 and 128 x 192 tiles
// of the kernel that loads straight into LDS, anything else the one expected to be fastest:
// rounds of tiles over the chip times the time of a tile, with the share of the matrix
// peak that each kernel was measured to reach on a busy CU (128 x 128: two workgroups a
// CU; the large tiles reach more the longer K is, and a tile of empty rows costs as
// much as a full one).
struct TiledPlan {
  int first;       // kernel of the columns 0 .. n1
  int n1;
  int second;      // kernel of the columns n1 .. N (0: there are none)
};

inline TiledPlan plan_tiled(int M, int N, int K, bool large_ok, bool may_split) {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    cus = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess &&
           prop.multiProcessorCount > 0) ? prop.multiProcessorCount : 256;
  }
  if (!large_ok) return TiledPlan{2, N, 0};
  const double fill = K >= 512 ? 1.0 : 0.6;            // the four-buffer pipeline needs a few steps to pay
  auto rounds = [&](double t, int slots) { return (double)(int64_t)((t + slots - 1) / slots); };
  // time of kernel k on n columns, in tile elements over the share of the peak
  auto cost = [&](int k, int n) {
    const int bm = k == 2 || k == 8 ? 128 : 256, bn = k == 2 ? 128 : k == 4 ? 256 : k == 5 ? 128 : 192;
    const double t = (double)((M + bm - 1) / bm) * ((n + bn - 1) / bn);
    // (128 x 192 tiles, the 256 x 128 kernel compiled for them: where they are at most one a CU.  2,048 rows of
    // 3,072 columns are 256 of them and 96 of 256 x 128: N 3,072 at K 2,048 / 3,072 / 8,192 33.2 / 48.9 / 97.0 us against
    // 35.6 / 53.3 / 101.9; 1,024 rows of N 6,144, K 4,096 52.2 against 56.6, of N 5,120, K 5,120 60.6 against 66.8;
    // in a second round they lose to every other tile)
    if (k == 8) return t <= cus ? 128.0 * 192 / (0.335 * fill) : 1e30;
    // (up to a tile a CU: the 128 x 128 tiles go to the kernel that loads straight into LDS)
    if (k == 2) return t <= cus ? 128.0 * 128 / (t <= 256 ? 0.30 : 0.22) : rounds(t, 2 * cus) * 2 * 128 * 128 / 0.31;
    return rounds(t, cus) * bm * bn / ((k == 4 ? 0.46 : k == 5 ? 0.42 : 0.44) * fill);
  };
  TiledPlan best{2, N, 0};
  double best_cost = cost(2, N);
  for (int k : {5, 6, 4, 8})
    if (cost(k, N) < best_cost || (k == 4 && cost(k, N) <= best_cost)) {
      best = TiledPlan{k, N, 0};
      best_cost = cost(k, N);
    }
  // A last round of large tiles that fills a part of the chip only costs as much as a
  // full one: the columns of the whole rounds go to the large tiles and the rest to a
  // second launch with the kernel that suits it (for 2,048 x 28,672: three rounds of
  // 256 x 256 and one of 256 x 128 in place of seven of 256 x 128).
  if (may_split) {
    const double launch = 3e-6 / (K * 2.05e-13);       // a second launch, in the same unit
    const int tile_rows = (M + 255) / 256;
    for (int a : {4, 6}) {
      const int bn = a == 4 ? 256 : 192;
      const int per_round = cus / tile_rows;           // tile columns that one round takes
      if (per_round < 1) continue;
      const int whole = (N / bn) / per_round;
      const int n1 = whole * per_round * bn;
      if (whole < 1 || n1 >= N) continue;
      for (int b : {2, 5, 6, 4, 8}) {
        const double c = cost(a, n1) + cost(b, N - n1) + launch;
        if (c < best_cost) {
          best = TiledPlan{a, n1, b};
          best_cost = c;
        }
      }
    }
  }
  return best;
}

template <int MODE>
int launch_tiled_kernel(int choice, void* C, int64_t ldc, const bf16_t* A, int64_t lda, const bf16_t* W, int64_t ldw,
                        int M, int N, int K, hipStream_t stream, const QkvArgs& qkv, const Partial& partial = Partial{},
                        bool forced = false) {
  if (choice == 6) return launch_direct<MODE, 4, 3>(C, ldc, A, lda, W, ldw, M, N, K, qkv, stream);
  if (choice == 4) return launch_direct<MODE, 4, 4>(C, ldc, A, lda, W, ldw, M, N, K, qkv, stream);
  if (choice == 5) return launch_direct64<MODE, 4, 2, 3>(C, ldc, A, lda, W, ldw, M, N, K, qkv, stream);
  if (choice == 7) return launch_direct64<MODE, 2, 2, 3>(C, ldc, A, lda, W, ldw, M, N, K, qkv, stream);
  if (choice == 8) return launch_direct64<MODE, 2, 3, 3>(C, ldc, A, lda, W, ldw, M, N, K, qkv, stream);
  return launch_pipelined<MODE>(C, ldc, A, lda, W, ldw, M, N, K, qkv, stream, partial, NormAfter{}, nullptr, forced);
}

template <int MODE>
int launch_aligned(void* C, int64_t ldc, const bf16_t* A, int64_t lda, const bf16_t* W, int64_t ldw,
                   int M, int N, int K, int force_kernel, hipStream_t stream, const QkvArgs& qkv = QkvArgs{},
                   const Partial& partial = Partial{}) {
  const bool large_ok = large_fits(lda, ldw, M, N, K);
  if (force_kernel == 2 || (force_kernel >= 4 && force_kernel <= 8))
    return launch_tiled_kernel<MODE>(force_kernel >= 4 && !large_ok ? 2 : force_kernel, C, ldc, A, lda, W, ldw, M, N, K,
                                     stream, qkv, partial, true);
  // (the q/k/v epilogue finds a column's head by its number: those products stay whole)
  const TiledPlan plan = plan_tiled(M, N, K, large_ok, MODE != OUT_QKV);
  if (int rc = launch_tiled_kernel<MODE>(plan.first, C, ldc, A, lda, W, ldw, M, plan.n1, K, stream, qkv, partial)) return rc;
  if (plan.second == 0) return 0;
  const int64_t skip = MODE == OUT_SWIGLU ? plan.n1 / 2 : plan.n1;         // output columns of the first part
  void* c2 = (MODE == OUT_BF16 || MODE == OUT_SWIGLU) ? (void*)((bf16_t*)C + skip) : (void*)((float*)C + skip);
  return launch_tiled_kernel<MODE>(plan.second, c2, ldc, A, lda, W + (int64_t)plan.n1 * ldw, ldw, M, N - plan.n1, K,
                                   stream, qkv);
}

// Up to 16 rows the streaming kernel always wins.  From 17 to 64 rows it re-reads the
// batch for every 16 weight rows, and the tiled kernel (which wastes matrix
// instructions but not bandwidth) wins once there are enough tiles to fill the chip, or
// weights enough for its cuts of K to fill it.  (This is the way of weights that lie as rows only:
// those that also lie in tiles go through hfee_gemm_skinny up to 64 rows.)
// (weights as rows, us, the streaming kernel against the tiled one with its cuts of K: N 6,144, K 4,096 at 17 /
// 33 / 64 rows 27.5 / 34.0 / 46.7 against 22.1 / 22.5 / 24.0; N 4,096, K 14,336 48.1 / 59.6 / 75.7 against 33.4 / 34.2 /
// 36.4; N 8,192, K 28,672 136 / 182 / 271 against 92 / 94 / 102; N 4,096, K 4,096 level up to 24 rows, 28.9 against 22.1
// at 64; N 3,072, K 2,048 14.7 / 16.6 / 19.6 against 17.4 / 18.2 / 18.8: from sixteen million weights on the tiled one)
inline bool skinny_pays(int M, int N, int K) {
  return M <= 16 || (M <= 64 && N < 16384 && (int64_t)N * K < (16ll << 20));
}

template <int MODE, bool VEC>
int launch(void* C, int64_t ldc, const bf16_t* A, int64_t lda, const bf16_t* W, int64_t ldw,
           int M, int N, int K, int force_kernel, hipStream_t stream, const Partial& partial) {
  const bool skinny = force_kernel == 1 || (force_kernel == 0 && skinny_pays(M, N, K));
  if (skinny) {
    dim3 grid((N + SK_ROWS - 1) / SK_ROWS);
    for (int m0 = 0; m0 < M; m0 += 64) {   // M > 64 only when the kernel was forced
      const int rows = M - m0 < 64 ? M - m0 : 64;
      const int g = (rows + 15) / 16;
      void* c = MODE == OUT_BF16 ? (void*)((bf16_t*)C + (int64_t)m0 * ldc) : (void*)((float*)C + (int64_t)m0 * ldc);
      const bf16_t* a = A + (int64_t)m0 * lda;
      if (g == 1) gemm_bf16_skinny_kernel<MODE, VEC, 1><<<grid, SK_WAVES * 64, 0, stream>>>(c, ldc, a, lda, W, ldw, rows, N, K);
      else if (g == 2) gemm_bf16_skinny_kernel<MODE, VEC, 2><<<grid, SK_WAVES * 64, 0, stream>>>(c, ldc, a, lda, W, ldw, rows, N, K);
      else if (g == 3) gemm_bf16_skinny_kernel<MODE, VEC, 3><<<grid, SK_WAVES * 64, 0, stream>>>(c, ldc, a, lda, W, ldw, rows, N, K);
      else gemm_bf16_skinny_kernel<MODE, VEC, 4><<<grid, SK_WAVES * 64, 0, stream>>>(c, ldc, a, lda, W, ldw, rows, N, K);
    }
  } else {
    dim3 grid((N + TBN - 1) / TBN, (M + TBM - 1) / TBM);
    if (grid.y > 65535) return fail("gemm_bf16: too many rows (%d)", M);
    if (VEC && force_kernel != 3)
      return launch_aligned<MODE>(C, ldc, A, lda, W, ldw, M, N, K, force_kernel, stream, QkvArgs{}, partial);
    gemm_bf16_tiled_kernel<MODE, VEC><<<grid, 256, 0, stream>>>(C, ldc, A, lda, W, ldw, M, N, K);
  }
  return 0;
}

}  // namespace

// How an aligned product of more than 64 rows is laid over the tiled kernels when nothing
// is forced: kernel of the first n1 columns, n1, kernel of the rest (0: none).  For
// tests and for reading a profile.
HFEE_API int hfee_gemm_bf16_plan(int M, int N, int K, int* first, int* n1, int* second) {
  HFEE_REQUIRE(M > 0 && N > 0 && K > 0 && first && n1 && second, "gemm_bf16_plan: bad arguments");
  const TiledPlan p = plan_tiled(M, N, K, large_fits(K, K, M, N, K), true);
  *first = p.first;
  *n1 = p.n1;
  *second = p.second;
  return 0;
}

// float32 words of scratch that hfee_gemm_bf16 can use for M x N x K (0: none): products with
// too few tiles for the chip are cut along K over more workgroups, which leave their partial
// products there for a second kernel to add up.
HFEE_API int hfee_gemm_bf16_scratch(int M, int N, int K) {
  if (skinny_pays(M, N, K)) return 0;                    // (the streaming kernel cuts nothing)
  const int splits = pipelined_splits(M, N, K);          // (fewer than 256 tiles of 128 x 128, at most 8 cuts: it fits an int)
  return splits > 1 ? splits * M * N : 0;
}

// C = A W^T for bfloat16 A [M, K] and W [N, K].
// out_mode: 0 bfloat16 store, 1 float32 store, 2 float32 accumulate, 3 gate (the
// rows of W alternate gate/up; C is [M, N/2] bfloat16 = activation(gate) * up, the
// activation being gate_act: GATE_SILU ...; aligned operands only).
// force_kernel: 0 choose by the sizes, 1 skinny, 2 tiled 128 x 128, 3 the simple tiled
// kernel, 4 tiled 256 x 256, 5 tiled 256 x 128, 6 tiled 256 x 192, 7 tiled 128 x 128 and 8 tiled 128 x 192 loaded
// straight into LDS (for tests of each kernel alone; 4 to 8 fall back to 2 where they do not apply).
// scratch: null, or hfee_gemm_bf16_scratch(M, N, K) float32 words, 16-byte aligned.
HFEE_API int hfee_gemm_bf16(void* C, int out_mode, int64_t ldc, const void* A, int64_t lda, const void* W,
                            int64_t ldw, int M, int N, int K, int force_kernel, float* scratch,
                            int64_t scratch_floats, int gate_act, hipStream_t stream) {
  Partial partial;
  partial.at = scratch;
  partial.floats = scratch != nullptr ? scratch_floats : 0;
  HFEE_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_bf16: bad sizes M=%d N=%d K=%d", M, N, K);
  HFEE_REQUIRE(lda >= K && ldw >= K, "gemm_bf16: a leading dimension is shorter than its row");
  HFEE_REQUIRE(out_mode >= 0 && out_mode <= 3, "gemm_bf16: unknown output mode %d", out_mode);
  HFEE_REQUIRE(ldc >= (out_mode == 3 ? N / 2 : N), "gemm_bf16: ldc is shorter than a row of the result");
  HFEE_REQUIRE(force_kernel >= 0 && force_kernel <= 8, "gemm_bf16: unknown kernel choice %d", force_kernel);
  if (M == 0) return 0;
  const bool vec = (K % 8 == 0) && (lda % 8 == 0) && (ldw % 8 == 0) &&
                   ((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0);
  if (out_mode == 3) {
    HFEE_REQUIRE(N % 2 == 0 && vec, "gemm_bf16: the gate needs an even N and aligned operands");
    HFEE_REQUIRE(gate_act >= 0 && gate_act < GATE_KINDS, "gemm_bf16: unknown activation %d", gate_act);
    QkvArgs gate{};
    gate.gate_act = gate_act;
    if (launch_aligned<OUT_SWIGLU>(C, ldc, (const bf16_t*)A, lda, (const bf16_t*)W, ldw, M, N, K, force_kernel, stream, gate)) return 1;
    HFEE_CHECK_LAUNCH("gemm_bf16");
    return 0;
  }
  const bf16_t* a = (const bf16_t*)A;
  const bf16_t* w = (const bf16_t*)W;
  int rc;
#define GO(MODE)                                                                                  \
  rc = vec ? launch<MODE, true>(C, ldc, a, lda, w, ldw, M, N, K, force_kernel, stream, partial)    \
           : launch<MODE, false>(C, ldc, a, lda, w, ldw, M, N, K, force_kernel, stream, partial)
  if (out_mode == OUT_BF16) GO(OUT_BF16);
  else if (out_mode == OUT_F32) GO(OUT_F32);
  else GO(OUT_ADD_F32);
#undef GO
  if (rc) return rc;
  HFEE_CHECK_LAUNCH("gemm_bf16");
  return 0;
}

// C (float32, the residual stream) += A W^T, and normed (bfloat16) = C_new / sqrt(mean(C_new^2) + eps)
// * norm_weight, the norm that reads the new rows next.  Where K is cut over workgroups (see
// hfee_gemm_bf16_scratch) the kernel that adds the partial products up also does the norm;
// otherwise the product and the norm are two launches, as if the caller had made them.
// C and normed: rows of N elements without gaps.  scratch as for hfee_gemm_bf16.
HFEE_API int hfee_gemm_bf16_add_norm(float* C, const void* A, int64_t lda, const void* W, int64_t ldw, int M, int N,
                                     int K, float* scratch, int64_t scratch_floats, void* normed,
                                     const void* norm_weight, int norm_weight_is_f32, float eps, hipStream_t stream) {
  HFEE_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_bf16_add_norm: bad sizes M=%d N=%d K=%d", M, N, K);
  HFEE_REQUIRE(C != nullptr && normed != nullptr && norm_weight != nullptr && eps >= 0.f,
               "gemm_bf16_add_norm: C, normed and the norm's weight are needed, and eps must not be negative");
  HFEE_REQUIRE(lda >= K && ldw >= K, "gemm_bf16_add_norm: a leading dimension is shorter than its row");
  if (M == 0) return 0;
  const bool vec = (K % 8 == 0) && (lda % 8 == 0) && (ldw % 8 == 0) && ((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0);
  bool done = false;
  if (vec && !skinny_pays(M, N, K)) {
    const TiledPlan plan = plan_tiled(M, N, K, large_fits(lda, ldw, M, N, K), true);
    if (plan.first == 2 && plan.second == 0) {
      Partial partial;
      partial.at = scratch;
      partial.floats = scratch != nullptr ? scratch_floats : 0;
      NormAfter norm;
      norm.normed = (bf16_t*)normed;
      norm.ldn = N;
      norm.weight = norm_weight;
      norm.weight_is_f32 = norm_weight_is_f32 != 0;
      norm.eps = eps;
      if (launch_pipelined<OUT_ADD_F32>(C, N, (const bf16_t*)A, lda, (const bf16_t*)W, ldw, M, N, K, QkvArgs{}, stream,
                                        partial, norm, &done))
        return 1;
      HFEE_CHECK_LAUNCH("gemm_bf16_add_norm");
      if (done) return 0;
      return hfee_rmsnorm(normed, DT_BF16, C, norm_weight, norm_weight_is_f32 ? DT_F32 : DT_BF16, nullptr, eps, M, N, stream);
    }
  }
  if (int rc = hfee_gemm_bf16(C, OUT_ADD_F32, N, A, lda, W, ldw, M, N, K, 0, scratch, scratch_floats, GATE_SILU, stream)) return rc;
  return hfee_rmsnorm(normed, DT_BF16, C, norm_weight, norm_weight_is_f32 ? DT_F32 : DT_BF16, nullptr, eps, M, N, stream);
}

// A W^T cut along K over workgroups, the partial products left as they are: *cuts matrices of
// float32 [M, N], one after the other in scratch, for a caller whose next kernel adds them up
// on its way (hfee_rope_cache_write_cuts).  *cuts = 0 and nothing launched where the product
// would not be cut (see hfee_gemm_bf16_scratch) or the scratch is too small: the caller then
// takes the plain product.
HFEE_API int hfee_gemm_bf16_cuts(const void* A, int64_t lda, const void* W, int64_t ldw, int M, int N, int K,
                                 float* scratch, int64_t scratch_floats, int* cuts, hipStream_t stream) {
  HFEE_REQUIRE(M > 0 && N > 0 && K > 0 && cuts != nullptr, "gemm_bf16_cuts: bad arguments");
  HFEE_REQUIRE(lda >= K && ldw >= K, "gemm_bf16_cuts: a leading dimension is shorter than its row");
  *cuts = 0;
  const bool vec = (K % 8 == 0) && (lda % 8 == 0) && (ldw % 8 == 0) && ((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0);
  if (!vec || skinny_pays(M, N, K) || scratch == nullptr || (uintptr_t)scratch % 16 != 0 || N % 4 != 0) return 0;
  const TiledPlan plan = plan_tiled(M, N, K, large_fits(lda, ldw, M, N, K), true);
  const int splits = pipelined_splits(M, N, K);
  if (plan.first != 2 || plan.second != 0 || splits < 2 || scratch_floats < (int64_t)splits * M * N) return 0;
  constexpr int TM = 2, TN = 2, STAGES = 3;
  const int k_split = ((K + splits - 1) / splits + 63) / 64 * 64;
  if (cuts_by_large_tiles(M, N, K, splits) && large_fits(lda, ldw, M, N, K)) {
    if (launch_direct64<OUT_F32, 4, 2, 3>(scratch, N, (const bf16_t*)A, lda, (const bf16_t*)W, ldw, M, N, K, QkvArgs{}, stream,
                                          k_split, splits, (int64_t)M * N))
      return 1;
  } else if (large_fits(lda, ldw, M, N, K)) {
    if (launch_direct64<OUT_F32, 2, 2, 3>(scratch, N, (const bf16_t*)A, lda, (const bf16_t*)W, ldw, M, N, K, QkvArgs{}, stream,
                                          k_split, splits, (int64_t)M * N))
      return 1;
  } else {
    const size_t lds = (size_t)2 * (64 * TM + 64 * TN) * PPITCH * sizeof(bf16_t);
    if (raise_pipelined_lds<OUT_F32>(lds)) return 1;
    const int64_t tiles = (int64_t)((N + 64 * TN - 1) / (64 * TN)) * ((M + 64 * TM - 1) / (64 * TM));
    dim3 grid((unsigned)((tiles + XCDS - 1) / XCDS * XCDS), splits);
    gemm_bf16_pipelined_kernel<OUT_F32, TM, TN, STAGES><<<grid, 256, lds, stream>>>(
        scratch, N, (const bf16_t*)A, lda, (const bf16_t*)W, ldw, M, N, K, QkvArgs{}, k_split, (int64_t)M * N);
  }
  HFEE_CHECK_LAUNCH("gemm_bf16_cuts");
  *cuts = splits;
  return 0;
}

// The q/k/v product of more than 64 rows: C = q part of A W^T rotated, k and v rotated
// and written into the paged cache by the product's epilogue (see qkv_epilogue.h).
// Operands must be aligned as the tiled kernels need them.  For the callers of
// hfee_gemm_skinny, which hands such products here.
HFEE_API int hfee_gemm_bf16_qkv(void* C, int64_t ldc, const void* A, int64_t lda, const void* W, int64_t ldw, int M,
                                int N, int K, const QkvArgs* qkv, int force_kernel, hipStream_t stream) {
  HFEE_REQUIRE(M > 0 && N > 0 && K > 0 && qkv != nullptr, "gemm_bf16_qkv: bad arguments");
  HFEE_REQUIRE((K % 8 == 0) && (lda % 8 == 0) && (ldw % 8 == 0) && ((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0),
               "gemm_bf16_qkv: K and the leading dimensions must be multiples of 8 and the operands 16-byte aligned");
  if (launch_aligned<OUT_QKV>(C, ldc, (const bf16_t*)A, lda, (const bf16_t*)W, ldw, M, N, K, force_kernel, stream, *qkv))
    return 1;
  HFEE_CHECK_LAUNCH("gemm_bf16_qkv");
  return 0;
}
