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

#include <type_traits>

using namespace hfee;

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

enum { OUT_BF16 = 0, OUT_F32 = 1, OUT_ADD_F32 = 2 };

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


// ---------------------------------------------------------- tiled, pipelined ---
// The prefill product for aligned operands.  Four waves in a 2x2 grid, each with
// TM x TN tiles of 32x32 (a workgroup tile of 64 TM x 64 TN), K in steps of 64.
// Global loads run STAGES K steps ahead of the matrix instructions (a ring of
// register stages), the LDS holds two steps.  Epilogues: bfloat16 store, float32
// store, float32 accumulate, and the SiLU gate for weights whose rows alternate
// gate/up (C[m, j] = silu(row 2j) * row 2j+1).
constexpr int PBK = 64, PPITCH = 72;   // pitch 144 bytes: no bank conflicts
constexpr int XCDS = 8;                // accelerator dies of an MI355X
enum { OUT_SWIGLU = 3 };

template <int TM, int TN>
struct PStage {
  u32x4 a[2 * TM], w[2 * TN];      // this thread's 16-byte chunks of the A tile and of the W tile
};

template <int MODE, int TM, int TN, int STAGES>
__global__ __launch_bounds__(256) void gemm_bf16_pipelined_kernel(void* __restrict__ C, int64_t ldc,
                                                                  const bf16_t* __restrict__ A, int64_t lda,
                                                                  const bf16_t* __restrict__ W, int64_t ldw,
                                                                  int M, int N, int K) {
  constexpr int BM = 64 * TM, BN = 64 * TN;
  extern __shared__ __attribute__((aligned(16))) bf16_t lds_tiles[];
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
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[ks & 1][i], b[ks & 1][j], acc[i][j], 0, 0, 0);
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

  // D layout of the 32x32 tile: register r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column l%32
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + wn * 32 * TN + j * 32 + lrow;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * 32 * TM + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        float v = acc[i][j][r];
        if (MODE == OUT_SWIGLU) {
          // the odd neighbour holds the up row: swap inside lane pairs (DPP quad_perm 1,0,3,2)
          const float up = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
          if ((lane & 1) == 0 && m < M && n < N)
            ((bf16_t*)C)[(int64_t)m * ldc + (n >> 1)] = float_to_bf16(v * __frcp_rn(1.0f + __expf(-v)) * up);
        } else if (m < M && n < N) {
          store_out<MODE>(C, ldc, m, n, v);
        }
      }
    }
}

template <int MODE>
int launch_pipelined(void* C, int64_t ldc, const bf16_t* A, int64_t lda, const bf16_t* W, int64_t ldw,
                     int M, int N, int K, hipStream_t stream) {
  // 128 x 128 tiles, two workgroups per CU.  (128 x 256 tiles halve the LDS reads per
  // matrix instruction but leave one wave per SIMD, and measured 20 % slower.)
  constexpr int TM = 2, TN = 2, STAGES = 3;
  const size_t lds = (size_t)2 * (64 * TM + 64 * TN) * PPITCH * sizeof(bf16_t);
  static bool raised = false;
  if (!raised) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_bf16_pipelined_kernel<MODE, TM, TN, STAGES>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return fail("gemm_bf16: cannot raise the LDS limit: %s", hipGetErrorString(e));
    raised = true;
  }
  const int64_t tiles = (int64_t)((N + 64 * TN - 1) / (64 * TN)) * ((M + 64 * TM - 1) / (64 * TM));
  if (tiles > (1 << 30)) return fail("gemm_bf16: too many tiles");
  dim3 grid((unsigned)((tiles + XCDS - 1) / XCDS * XCDS));
  gemm_bf16_pipelined_kernel<MODE, TM, TN, STAGES><<<grid, 256, lds, stream>>>(C, ldc, A, lda, W, ldw, M, N, K);
  return 0;
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

// Up to 16 rows the streaming kernel always wins.  From 17 to 64 rows it re-reads the
// batch for every 16 weight rows, and the tiled kernel (which wastes matrix
// instructions but not bandwidth) wins once there are enough tiles to fill the chip.
inline bool skinny_pays(int M, int N) { return M <= 16 || (M <= 64 && N < 16384); }

template <int MODE, bool VEC>
int launch(void* C, int64_t ldc, const bf16_t* A, int64_t lda, const bf16_t* W, int64_t ldw,
           int M, int N, int K, int force_kernel, hipStream_t stream) {
  const bool skinny = force_kernel == 1 || (force_kernel == 0 && skinny_pays(M, N));
  if (skinny) {
    const int mt = (M + 15) / 16;
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
    (void)mt;
  } else {
    dim3 grid((N + TBN - 1) / TBN, (M + TBM - 1) / TBM);
    if (grid.y > 65535) return fail("gemm_bf16: too many rows (%d)", M);
    if (VEC && force_kernel != 3)
      return launch_pipelined<MODE>(C, ldc, A, lda, W, ldw, M, N, K, stream);
    gemm_bf16_tiled_kernel<MODE, VEC><<<grid, 256, 0, stream>>>(C, ldc, A, lda, W, ldw, M, N, K);
  }
  return 0;
}

}  // namespace

HFEE_API int hfee_gemm_skinny(void* C, int64_t ldc, const void* A, int a_is_f32, int64_t lda, const void* W,
                              int64_t ldw, int M, int N, int K, int epi,
                              const void* norm_weight, int norm_weight_is_f32, float eps, const int* rows,
                              const int* positions, const int* token_segment, const int* block_tables,
                              int bt_stride, const float* cos_table, const float* sin_table, int half,
                              int table_positions, void* cache, int num_heads, int kv_heads, int head_dim,
                              int page_size, hipStream_t stream);

// out_mode: 0 bfloat16 store, 1 float32 store, 2 float32 accumulate, 3 SiLU gate (the
// rows of W alternate gate/up; C is [M, N/2] bfloat16; aligned operands and M > 64 only).
// force_kernel: 0 choose by M, 1 skinny, 2 tiled, 3 the simple tiled kernel (for tests
// of each kernel alone).
HFEE_API int hfee_gemm_bf16(void* C, int out_mode, int64_t ldc, const void* A, int64_t lda, const void* W,
                            int64_t ldw, int M, int N, int K, int force_kernel, hipStream_t stream) {
  HFEE_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_bf16: bad sizes M=%d N=%d K=%d", M, N, K);
  HFEE_REQUIRE(lda >= K && ldw >= K, "gemm_bf16: a leading dimension is shorter than its row");
  HFEE_REQUIRE(out_mode >= 0 && out_mode <= 3, "gemm_bf16: unknown output mode %d", out_mode);
  HFEE_REQUIRE(ldc >= (out_mode == 3 ? N / 2 : N), "gemm_bf16: ldc is shorter than a row of the result");
  HFEE_REQUIRE(force_kernel >= 0 && force_kernel <= 3, "gemm_bf16: unknown kernel choice %d", force_kernel);
  if (M == 0) return 0;
  const bool vec = (K % 8 == 0) && (lda % 8 == 0) && (ldw % 8 == 0) &&
                   ((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0);
  if (out_mode == 3) {
    HFEE_REQUIRE(N % 2 == 0 && vec, "gemm_bf16: the SiLU gate needs an even N and aligned operands");
    if (skinny_pays(M, N))
      return hfee_gemm_skinny(C, ldc, A, 0, lda, W, ldw, M, N, K, 3, nullptr, 0, 0.f, nullptr, nullptr, nullptr, nullptr,
                              0, nullptr, nullptr, 0, 0, nullptr, 0, 0, 0, 0, stream);
    if (launch_pipelined<OUT_SWIGLU>(C, ldc, (const bf16_t*)A, lda, (const bf16_t*)W, ldw, M, N, K, stream)) return 1;
    HFEE_CHECK_LAUNCH("gemm_bf16");
    return 0;
  }
  if (vec && M <= 64 && (force_kernel == 1 || (force_kernel == 0 && skinny_pays(M, N))))   // gemm_skinny.hip
    return hfee_gemm_skinny(C, ldc, A, 0, lda, W, ldw, M, N, K, out_mode, nullptr, 0, 0.f, nullptr, nullptr, nullptr,
                            nullptr, 0, nullptr, nullptr, 0, 0, nullptr, 0, 0, 0, 0, stream);
  const bf16_t* a = (const bf16_t*)A;
  const bf16_t* w = (const bf16_t*)W;
  int rc;
#define GO(MODE)                                                                                  \
  rc = vec ? launch<MODE, true>(C, ldc, a, lda, w, ldw, M, N, K, force_kernel, stream)             \
           : launch<MODE, false>(C, ldc, a, lda, w, ldw, M, N, K, force_kernel, stream)
  if (out_mode == OUT_BF16) GO(OUT_BF16);
  else if (out_mode == OUT_F32) GO(OUT_F32);
  else GO(OUT_ADD_F32);
#undef GO
  if (rc) return rc;
  HFEE_CHECK_LAUNCH("gemm_bf16");
  return 0;
}
