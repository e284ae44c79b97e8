// The decode-time matrix product: C[M,N] = A[M,K] * W[N,K]^T for M <= 64, bound by
// reading W once from HBM, with the neighbouring small operations folded in so that a
// decode step of a layer is five launches instead of ten.
//
// A workgroup owns 16 weight rows; its eight waves split K in blocks of 128 and
// stream their share of W straight from global memory into the A operand of
// v_mfma_f32_16x16x32_bf16 (lane l: row l%16, eight consecutive k).  The batch rows are
// the B operand.  Loads are issued one block ahead of the matrix instructions.
// Partial sums meet in LDS and are added in wave order (a fixed order).
//
// W comes in tiles (see WeightTiles in common.h): 16 rows x 32 columns are one kilobyte in
// the order in which a wave's lanes hold them as an operand, so that a load instruction of a
// wave reads one contiguous kilobyte, whole 128-byte lines that nobody else touches, and
// can carry the non-temporal hint.  With rows of W as they lie in a checkpoint the same
// instruction reads sixteen half lines, each of which a second instruction asks for again:
// a read-only stream of that pattern measures 5.9 TB/s on this GPU, the kilobytes 6.5.
//
// Folded in:
//   NORM   the RMSNorm in front of the product
//          (/root/reference/internal/ggml/ops.go:124-134): A is the float32 residual
//          stream; x * w is rounded to bfloat16 on the way into the operand, the sum of
//          squares rides along, and 1/sqrt(mean + eps) scales the finished sums.
//   EPI_ADD      C (float32) += result        (/root/reference/internal/llm/forward.go:106-107)
//   EPI_SWIGLU   rows of W alternate gate/up: C[m, j] = silu(gate_j) * up_j
//                                             (/root/reference/internal/ggml/ops.go:159-165)
//   EMIT   (with EPI_ADD) a norm that follows the residual add, in two halves so that
//          nobody waits for a whole row: the product that adds into the stream also
//          writes bfloat16(x_new * w_next) and, per workgroup, its columns' share of every
//          row's sum of squares.  The product that consumes the row (ROW SCALE) adds the
//          shares up, in a fixed order, and scales its finished sums by
//          1/sqrt(mean + eps): the same numbers as NORM gives, with no norm of its own.
//   EPI_QKV      rows of W are q, k, v heads with rotation pairs adjacent (2i, 2i+1):
//                rotate q and k at the token's position, write q to C, k and v into the
//                token's slot of the paged cache
//                                             (/root/reference/internal/llm/forward.go:96-101)
#include "common.h"
#include "qkv_epilogue.h"
#include "gemm_entry.h"

using namespace hfee;

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

enum { EPI_BF16 = 0, EPI_F32 = 1, EPI_ADD = 2, EPI_SWIGLU = 3, EPI_QKV = 4 };

constexpr int WAVES = 8, ROWS = 16;

union Chunk {
  u32x4 u;
  bf16x8 v;
  bf16_t e[8];
};

struct Args {
  void* C;
  int64_t ldc;
  const void* A;              // bfloat16 [M, K], or float32 rows when NORM
  int64_t lda;
  const bf16_t* W;            // in tiles of 16 rows x 32 columns
  int64_t w_stride;           // elements from one row of tiles to the next
  int M, N, K;
  const void* norm_weight;    // NORM: [K]
  int norm_weight_is_f32;
  float eps;
  const int* rows;            // NORM: row m of the product is row rows[m] of A (null: m)
  QkvArgs qkv;
  // EMIT (EPI_ADD only; emit_out null: nothing is emitted)
  const void* emit_weight;    // [N] weight of the norm that follows
  int emit_weight_is_f32;
  bf16_t* emit_out;           // [M, N] bfloat16(x_new * weight)
  int64_t ld_emit;
  float* emit_ss;             // [workgroups][SS_STRIDE] this workgroup's columns' sum of squares per row
  // ROW SCALE (scale_ss null: none)
  const float* scale_ss;      // [scale_blocks][SS_STRIDE] shares of the rows' sums of squares
  int scale_blocks;
  float scale_eps;
};

constexpr int SS_STRIDE = 64;   // rows of a product of this file

// A K block is U steps of 32 columns: what a wave asks for at once and keeps in flight while
// it multiplies the block before.
template <int U>
struct Block {                // one wave's operands for one K block
  Chunk w[U];
};

template <int MT, bool NORM, int U>
struct XBlock;

template <int MT, int U>
struct XBlock<MT, false, U> {
  Chunk x[MT][U];
};

template <int MT, int U>
struct XBlock<MT, true, U> {     // raw float32 activations and the norm weight
  f32x4 x[MT][U][2];
  f32x4 nw[U][2];
};

__device__ __forceinline__ f32x4 load_f4(const float* p) { return *reinterpret_cast<const f32x4*>(p); }

template <int MT, bool NORM, int U>
__device__ __forceinline__ void load_block(Block<U>& b, XBlock<MT, NORM, U>& xb, const bf16_t* __restrict__ w_row,
                                           const void* const* x_rows, const Args& a, int k) {
  // w_row points at this lane's place in the first tile of its row of tiles, x_rows at its
  // eight-element column group; 32 columns on is the next tile
#pragma unroll
  for (int s = 0; s < U; ++s)
    b.w[s].u = load_streamed(reinterpret_cast<const u32x4*>(w_row + (int64_t)(k + 32 * s) * WeightTiles::PER_COLUMN));
  if constexpr (!NORM) {
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int s = 0; s < U; ++s)
        xb.x[t][s].u = *reinterpret_cast<const u32x4*>((const bf16_t*)x_rows[t] + k + 32 * s);
  } else {
    const int kg = k + 8 * ((threadIdx.x & 63) >> 4);
#pragma unroll
    for (int s = 0; s < U; ++s) {
      if (a.norm_weight_is_f32) {
        xb.nw[s][0] = load_f4((const float*)a.norm_weight + kg + 32 * s);
        xb.nw[s][1] = load_f4((const float*)a.norm_weight + kg + 32 * s + 4);
      } else {
        Chunk c;
        c.u = *reinterpret_cast<const u32x4*>((const bf16_t*)a.norm_weight + kg + 32 * s);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          xb.nw[s][0][j] = bf16_to_float(c.e[j]);
          xb.nw[s][1][j] = bf16_to_float(c.e[4 + j]);
        }
      }
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        xb.x[t][s][0] = load_f4((const float*)x_rows[t] + k + 32 * s);
        xb.x[t][s][1] = load_f4((const float*)x_rows[t] + k + 32 * s + 4);
      }
    }
  }
}

template <int MT, bool NORM, int U>
__device__ __forceinline__ void compute_block(f32x4* acc, float* ss, const Block<U>& b, const XBlock<MT, NORM, U>& xb) {
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int s = 0; s < U; ++s) {
      if constexpr (!NORM) {
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b.w[s].v, xb.x[t][s].v, acc[t], 0, 0, 0);
      } else {
        Chunk c;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float v = xb.x[t][s][h][j];
            ss[t] = fmaf(v, v, ss[t]);
            c.e[4 * h + j] = float_to_bf16(v * xb.nw[s][h][j]);
          }
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b.w[s].v, c.v, acc[t], 0, 0, 0);
      }
    }
}

__device__ __forceinline__ float silu(float g) { return g / (1.0f + expf(-g)); }

// ROW SCALE: 1/sqrt(mean of squares + eps) of every batch row from the shares that the
// product before this one left, into `out` (LDS, SS_STRIDE floats).  All threads of the
// workgroup come here; the caller synchronises before it reads `out`.  Lane l of wave w
// takes batch rows l % 16 (+16, +32, +48) and the shares 4w + l/16, + 32, ...: every load
// is on its own (nobody waits for a sum before asking for the next share), a row's four
// lanes meet by shuffles and the waves in LDS, in an order that depends on nothing but
// the number of shares.
template <int TILES>
__device__ __forceinline__ void row_scales(const Args& a, float* out) {
  __shared__ float part[WAVES][SS_STRIDE];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, m16 = lane & 15, j = lane >> 4;
  float s[TILES];
  const float* p[TILES];
#pragma unroll
  for (int t = 0; t < TILES; ++t) {
    s[t] = 0.f;
    p[t] = a.scale_ss + min(t * 16 + m16, a.M - 1);      // rows beyond M repeat the last one; nobody uses them
  }
  // (no load stands under a condition: the compiler keeps a whole round of them in flight)
  constexpr int ROUND = 8;
  for (int b0 = wave * 4 + j; b0 < a.scale_blocks; b0 += ROUND * WAVES * 4) {
    float v[ROUND][TILES];
#pragma unroll
    for (int r = 0; r < ROUND; ++r) {
      const int b = min(b0 + r * WAVES * 4, a.scale_blocks - 1);       // past the end: a repeat that is not added
#pragma unroll
      for (int t = 0; t < TILES; ++t) v[r][t] = p[t][(int64_t)b * SS_STRIDE];
    }
#pragma unroll
    for (int r = 0; r < ROUND; ++r)
#pragma unroll
      for (int t = 0; t < TILES; ++t) s[t] += b0 + r * WAVES * 4 < a.scale_blocks ? v[r][t] : 0.f;
  }
#pragma unroll
  for (int t = 0; t < TILES; ++t) {
    float v = s[t];
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    if (j == 0) part[wave][t * 16 + m16] = v;
  }
  __syncthreads();
  if (threadIdx.x < TILES * 16) {
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) v += part[w][threadIdx.x];
    out[threadIdx.x] = 1.0f / sqrtf(v / (float)a.K + a.scale_eps);
  }
}

// The same in three parts, for kernels that end in an exchange through LDS anyway: the loads are
// asked for at the start and nothing waits for them there (row_scales' barrier, standing in
// front of the loop, kept every wave from asking for its next weights until the shares, which
// the product before has only just written, had come from memory: 1.4 us a product inside the
// decode step); the sums go into LDS together with the kernel's own partial sums, in front of the
// barrier that those need, and a finishing thread adds the waves' parts up for its row.  One
// round of loads: scale_blocks <= Shares<TILES>::BLOCKS (else row_scales).
template <int TILES>
struct Shares {
  static constexpr int ROUND = TILES == 1 ? 16 : 8;
  static constexpr int BLOCKS = ROUND * WAVES * 4;
  float v[ROUND][TILES];
};

template <int TILES>
__device__ __forceinline__ void ask_shares(const Args& a, Shares<TILES>& sh) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, m16 = lane & 15, j = lane >> 4;
#pragma unroll
  for (int r = 0; r < Shares<TILES>::ROUND; ++r) {
    const int b = min(wave * 4 + j + r * WAVES * 4, a.scale_blocks - 1);       // past the end: a repeat that is not added
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
      sh.v[r][t] = 0.f;
      if (r * WAVES * 4 < a.scale_blocks)        // (the same for everybody: whole rounds beyond the end are not asked for)
        sh.v[r][t] = a.scale_ss[(int64_t)b * SS_STRIDE + min(t * 16 + m16, a.M - 1)];
    }
  }
}

// part: [WAVES][SS_STRIDE] floats of LDS; the caller's barrier follows.
template <int TILES>
__device__ __forceinline__ void put_shares(const Args& a, const Shares<TILES>& sh, float (*part)[SS_STRIDE]) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, m16 = lane & 15, j = lane >> 4;
#pragma unroll
  for (int t = 0; t < TILES; ++t) {
    float v = 0.f;
#pragma unroll
    for (int r = 0; r < Shares<TILES>::ROUND; ++r) v += wave * 4 + j + r * WAVES * 4 < a.scale_blocks ? sh.v[r][t] : 0.f;
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    if (j == 0) part[wave][t * 16 + m16] = v;
  }
}

// after the barrier: 1/sqrt(mean of squares + eps) of batch row m
__device__ __forceinline__ float scale_of(const Args& a, const float (*part)[SS_STRIDE], int m) {
  float v = 0.f;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) v += part[w][m];
  return 1.0f / sqrtf(v / (float)a.K + a.scale_eps);
}

// What happens to four finished sums: weight rows n .. n+3 of batch row m.
template <int EPI>
__device__ __forceinline__ void epilogue(const Args& a, int m, int n, float* v) {
  if constexpr (EPI == EPI_BF16) {
    bf16_t* c = (bf16_t*)a.C + (int64_t)m * a.ldc + n;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (n + i < a.N) c[i] = float_to_bf16(v[i]);
  } else if constexpr (EPI == EPI_F32) {
    float* c = (float*)a.C + (int64_t)m * a.ldc + n;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (n + i < a.N) c[i] = v[i];
  } else if constexpr (EPI == EPI_ADD) {
    float* c = (float*)a.C + (int64_t)m * a.ldc + n;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (n + i < a.N) c[i] += v[i];
  } else if constexpr (EPI == EPI_SWIGLU) {
    // rows n, n+1 = gate, up of column n/2; rows n+2, n+3 of column n/2 + 1 (N is even)
    bf16_t* c = (bf16_t*)a.C + (int64_t)m * a.ldc + (n >> 1);
    c[0] = float_to_bf16(silu(v[0]) * v[1]);
    if (n + 2 < a.N) c[1] = float_to_bf16(silu(v[2]) * v[3]);
  } else {   // EPI_QKV
    qkv_store(a.qkv, a.C, a.ldc, m, n, v);
  }
}

// What the thread that finishes four sums (weight rows n .. n+3 of batch row m) has to
// read for them: asked for at the start of a kernel, it has arrived when the sums have.
template <int EPI>
struct Ahead {
  float old[4];          // EPI_ADD: what is added to
  float weight[4];       // EPI_ADD with EMIT: the weight of the norm that follows
  QkvPlace place;        // EPI_QKV
};

template <int EPI>
__device__ __forceinline__ Ahead<EPI> look_ahead(const Args& a, int m, int n, bool live) {
  Ahead<EPI> h;
  if constexpr (EPI == EPI_ADD) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool in = live && n + i < a.N;
      h.old[i] = in ? ((const float*)a.C)[(int64_t)m * a.ldc + n + i] : 0.f;
      h.weight[i] = !(in && a.emit_out != nullptr) ? 0.f
                    : a.emit_weight_is_f32 ? ((const float*)a.emit_weight)[n + i]
                                           : bf16_to_float(((const bf16_t*)a.emit_weight)[n + i]);
    }
  } else if constexpr (EPI == EPI_QKV) {
    if (live) h.place = qkv_place(a.qkv, a.C, a.ldc, m, n);
  }
  return h;
}

// What every kernel that looks ahead does with four finished sums of a whole wave's lanes
// (lane l: batch row m, weight rows n .. n+3, `live` if they exist): the residual add with
// the first half of the norm that follows it (EMIT), or the plain epilogue, with what
// look_ahead has brought.  `block`: this group of 16 weight rows (the row of the shares
// table).  All lanes of the wave come here together: the shares are summed by shuffles.
template <int EPI>
__device__ __forceinline__ void finish_rows_ahead(const Args& a, const Ahead<EPI>& h, int m, int n, bool live, float* v,
                                                  int block, int l) {
  if constexpr (EPI == EPI_ADD) {
    float ss = 0.f;
    if (live) {
      float* c = (float*)a.C + (int64_t)m * a.ldc + n;
      bf16_t* e = a.emit_out != nullptr ? a.emit_out + (int64_t)m * a.ld_emit + n : nullptr;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (n + i < a.N) {
          const float x = h.old[i] + v[i];
          c[i] = x;
          ss = fmaf(x, x, ss);
          if (e != nullptr) e[i] = float_to_bf16(x * h.weight[i]);
        }
      }
    }
    if (a.emit_out != nullptr) {
      ss += __shfl_xor(ss, 16, 64);          // the four column groups of this row
      ss += __shfl_xor(ss, 32, 64);
      if ((l >> 4) == 0 && m < a.M) a.emit_ss[(int64_t)block * SS_STRIDE + m] = ss;
    }
  } else if constexpr (EPI == EPI_QKV) {
    if (live) qkv_put(h.place, v);
  } else {
    if (live) epilogue<EPI>(a, m, n, v);
  }
}

// TWO_A_CU (at most 16 batch rows): blocks of half the size, so that the registers allow two
// workgroups a CU.  For launches of more workgroups than CUs and at most twice as many (5,120
// weight rows: 320): all of them are on the chip from the start and share the memory's
// bandwidth, where one a CU leaves a second round that fills a part of the chip only.
template <int MT, bool NORM, int EPI, bool TWO_A_CU = false>
__global__ __launch_bounds__(WAVES * 64, TWO_A_CU ? 4 : 2) void skinny_kernel(Args a) {
  // (two kilobytes of weights a wave and step of the loop for up to 16 batch rows, one beyond:
  // with 8 waves a CU and a block in flight that is 64 KB a CU on its way, what the memory's
  // latency takes at the CU's share of the bandwidth)
  constexpr int U = MT == 1 && !TWO_A_CU ? 8 : 4, KBLOCK = 32 * U;
  __shared__ float partial[WAVES][MT][64][4];
  __shared__ float ss_part[WAVES][MT][16];
  __shared__ float row_scale[SS_STRIDE];
  __shared__ float share_part[WAVES][SS_STRIDE];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r16 = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * ROWS;
  const bool scaled = !NORM && a.scale_ss != nullptr, late = scaled && a.scale_blocks <= Shares<MT>::BLOCKS;
  Shares<MT> shares;
  // rows beyond N lie in the last row of tiles (zeros), rows beyond M read a valid row; what
  // they produce is never stored
  const bf16_t* w_row = WeightTiles::lane_place(a.W, a.w_stride, n0 + r16, g);
  const void* x_rows[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    int m = min(t * 16 + r16, a.M - 1);
    if (NORM && a.rows) m = a.rows[m];
    x_rows[t] = NORM ? (const void*)((const float*)a.A + (int64_t)m * a.lda + g * 8)
                     : (const void*)((const bf16_t*)a.A + (int64_t)m * a.lda + g * 8);
  }

  f32x4 acc[MT];
  float ss[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    ss[t] = 0.f;
  }
  // the threads that will finish the sums (the first MT waves, four sums each) ask now for
  // what they will need then
  const int f_t = threadIdx.x >> 6, f_m = f_t * 16 + (lane & 15), f_n = n0 + 4 * (lane >> 4);
  const bool f_live = f_t < MT && f_m < a.M && f_n < a.N;
  const Ahead<EPI> ahead = look_ahead<EPI>(a, f_m, f_n, f_live);

  const int nfull = a.K / KBLOCK;
  {
    // One block ahead, and no further: the next block is asked for, the current one is
    // multiplied, and the copy into `cur` then waits for the block just asked for.  Forms
    // of this loop that keep two blocks a wave in flight all the time (two sets of registers
    // taking turns, in blocks of 128 or of 64 columns) were faster on one matrix in a loop and
    // slower inside the decode step, where the weights come from memory: 56.9 and 57.4 µs
    // against 53.5 for q/k/v + output + down of a layer of the 8B shape at batch 8.  (The
    // block number is kept per lane, as it was when this was measured.)
    Block<U> cur, nxt;
    XBlock<MT, NORM, U> xcur, xnxt;
    int kb = threadIdx.x >> 6;
    if (kb < nfull) load_block<MT, NORM, U>(cur, xcur, w_row, x_rows, a, kb * KBLOCK);
    // (behind the first loads of W, so that it costs no latency of its own)
    if (late) ask_shares<MT>(a, shares);
    else if (scaled) row_scales<MT>(a, row_scale);
    while (kb < nfull) {
      const int kn = kb + WAVES;
      if (kn < nfull) load_block<MT, NORM, U>(nxt, xnxt, w_row, x_rows, a, kn * KBLOCK);
      compute_block<MT, NORM, U>(acc, ss, cur, xcur);
      cur = nxt;
      xcur = xnxt;
      kb = kn;
    }
  }
  // the last, partial block (K is a multiple of 8: whole chunks are in or out)
  if (a.K % KBLOCK != 0 && wave == nfull % WAVES) {
    const int k0 = nfull * KBLOCK;
#pragma unroll
    for (int s = 0; s < U; ++s) {
      const int k = k0 + 32 * s + g * 8;      // this lane's first element of the chunk
      if (k0 + 32 * s >= a.K) break;          // uniform: the whole step is beyond K
      const bool in = k < a.K;
      Chunk w;
      w.u = u32x4{0u, 0u, 0u, 0u};
      if (in) w.u = load_streamed(reinterpret_cast<const u32x4*>(w_row + (int64_t)(k0 + 32 * s) * WeightTiles::PER_COLUMN));
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        Chunk c;
        c.u = u32x4{0u, 0u, 0u, 0u};
        if (in) {
          if constexpr (!NORM) {
            c.u = *reinterpret_cast<const u32x4*>((const bf16_t*)x_rows[t] + k0 + 32 * s);
          } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              const float v = ((const float*)x_rows[t])[k0 + 32 * s + j];
              const float nw = a.norm_weight_is_f32 ? ((const float*)a.norm_weight)[k + j]
                                                    : bf16_to_float(((const bf16_t*)a.norm_weight)[k + j]);
              ss[t] = fmaf(v, v, ss[t]);
              c.e[j] = float_to_bf16(v * nw);
            }
          }
        }
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w.v, c.v, acc[t], 0, 0, 0);
      }
    }
  }

  // ---- partial sums meet in LDS ---------------------------------------------------
#pragma unroll
  for (int t = 0; t < MT; ++t) {
#pragma unroll
    for (int i = 0; i < 4; ++i) partial[wave][t][lane][i] = acc[t][i];
    if (NORM) {
      float s = ss[t];
      s += __shfl_xor(s, 16, 64);
      s += __shfl_xor(s, 32, 64);
      if (g == 0) ss_part[wave][t][r16] = s;
    }
  }
  if (late) put_shares<MT>(a, shares, share_part);
  __syncthreads();

  // D layout of the 16x16 tile: register i of lane l is weight row 4*(l/16) + i, batch row l%16
  // (MT * 64 is a multiple of the wave size: whole waves walk the loop, as the shuffles of EMIT need)
  for (int idx = threadIdx.x; idx < MT * 64; idx += WAVES * 64) {
    const int t = idx >> 6, l = idx & 63;
    const int m = t * 16 + (l & 15);
    const int n = n0 + 4 * (l >> 4);
    const bool live = m < a.M && n < a.N;
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float s = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) s += partial[w][t][l][i];
      v[i] = s;
    }
    if (NORM) {
      float s = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) s += ss_part[w][t][l & 15];
      const float scale = 1.0f / sqrtf(s / (float)a.K + a.eps);
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] *= scale;
    } else if (a.scale_ss != nullptr) {
      const float scale = late ? scale_of(a, share_part, min(m, SS_STRIDE - 1)) : row_scale[min(m, SS_STRIDE - 1)];
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] *= scale;
    }

    finish_rows_ahead<EPI>(a, ahead, m, n, live, v, blockIdx.x, l);      // (idx == threadIdx.x: MT <= WAVES)
  }
}

// The CUs of the current device (256 if it cannot be asked).
inline int cu_count() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    cus = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess &&
           prop.multiProcessorCount > 0) ? prop.multiProcessorCount : 256;
  }
  return cus;
}

template <int MT, bool NORM>
void launch_epi(const Args& a, int epi, hipStream_t stream) {
  // (a workgroup takes a whole row of tiles: with 8 or 12 rows a workgroup, which spread 6,144
  // rows more evenly over 256 CUs, a wave's load is no longer a whole kilobyte, and that costs
  // more than the uneven rounds: q/k/v of the 8B shape 16.6 us against 12.7)
  dim3 grid((a.N + ROWS - 1) / ROWS);
  if constexpr (MT == 1 && !NORM) {
    const int cus = cu_count();
    if ((int)grid.x > cus && (int)grid.x <= 2 * cus) {
#define GO2(E) skinny_kernel<MT, NORM, E, true><<<grid, WAVES * 64, 0, stream>>>(a)
      switch (epi) {
        case EPI_BF16: GO2(EPI_BF16); break;
        case EPI_F32: GO2(EPI_F32); break;
        case EPI_ADD: GO2(EPI_ADD); break;
        case EPI_SWIGLU: GO2(EPI_SWIGLU); break;
        default: GO2(EPI_QKV); break;
      }
#undef GO2
      return;
    }
  }
#define GO(E) skinny_kernel<MT, NORM, E><<<grid, WAVES * 64, 0, stream>>>(a)
  switch (epi) {
    case EPI_BF16: GO(EPI_BF16); break;
    case EPI_F32: GO(EPI_F32); break;
    case EPI_ADD: GO(EPI_ADD); break;
    case EPI_SWIGLU: GO(EPI_SWIGLU); break;
    default: GO(EPI_QKV); break;
  }
#undef GO
}


// ------------------------------------------------------------ 17 to 64 rows ---
// With more than 16 batch rows the streaming kernel reads the batch again for every 16
// weight rows, and that traffic (from L2) outgrows the weights.  Here K is cut into
// slices of 1,024 columns (the last one may be shorter: a multiple of 256 columns), each with
// workgroups of its own.  A workgroup keeps its slice
// of the batch, all rows, in LDS; each of its waves walks over groups of 16 weight rows
// on its own: the weights come straight from global memory through a ring of 4 or 16 loads
// that runs across group boundaries, the batch operands from LDS; no barrier stands in
// the loop.  With more than one slice a wave leaves its share of a row group's sums in a
// scratch buffer and goes on; a second, short kernel (one wave for 16 batch rows of a row
// group, so that the whole chip takes part) adds the shares in the order of the slices and
// runs the epilogue.  Nobody waits for anybody, and nothing is counted.
constexpr int MID_KS = 1024, MID_STEPS = MID_KS / 32;
// Loads a wave keeps in flight: four.  Measured inside the decode step at 64 rows (q/k/v, output,
// down of the 8B shape): 20.3 / 14.2 / 27.2 µs with 8, 15.0 / 13.8 / 27.1 with 4, 19.7 / 15.2 / 30.4
// with 2; at 24 and 32 rows 4 against 16: 4.41 against 4.46 ms a step, 4.70 against 4.73; at 24
// and 48 rows 4 against 8: 4.35 against 4.44, 5.29 against 5.36.
// The loop is unrolled over eight steps (whole turns of the ring), and the last slice of K is
// a whole number of these: K is a multiple of 256 columns.  (The same loop over 16 steps with
// a last turn of 8, written as one body for both, measured 3 % slower over the whole step at
// 64 rows: 5.91 ms against 5.73.)
constexpr int MID_RING = 4, MID_HALF = 8;
// (the kernel for many weight rows, below, keeps its own count: at 24 and 32 rows 4.36 and 4.68 ms
// a step with 8, 4.41 and 4.70 with 16, 4.40 and 4.74 with 4; at 48 rows 5.28 with 8 and 5.33 with
// 4; at 64 rows 5.94 with 8 and 5.75 with 4)
constexpr int mid_ring(int mt) { return mt >= 4 ? 4 : 8; }
constexpr int MID_PITCH = MID_KS + 8;        // LDS row pitch of the batch slice in elements: rows 16 bytes askew

constexpr size_t mid_lds_bytes(int mt) { return (size_t)mt * 16 * MID_PITCH * sizeof(bf16_t); }

template <int MT, int EPI>
__global__ __launch_bounds__(WAVES * 64) void mid_kernel(Args a, int row_groups, int slices, float* __restrict__ scratch) {
  extern __shared__ __attribute__((aligned(16))) char mid_lds[];
  bf16_t* xs = (bf16_t*)mid_lds;                                                    // [MT * 16][MID_PITCH]
  __shared__ float row_scale[SS_STRIDE];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r16 = lane & 15, g = lane >> 4;
  const int slice = blockIdx.x % slices;                     // the host launches a multiple of `slices`
  const int stride = (gridDim.x / slices) * WAVES;           // waves of this slice
  const int k0 = slice * MID_KS;

  // ---- the batch slice is asked for first: it comes from L2 and must not wait in line
  // behind the first weights, which come from memory (a wave's loads return in order).
  // Every workgroup of a slice wants the same rows: each starts at another one.
  constexpr int FILL = MT * 16 * (MID_KS / 8) / (WAVES * 64);      // 16-byte chunks a thread brings
  static_assert(MT * 16 * (MID_KS / 8) % (WAVES * 64) == 0, "the batch slice is whole rounds of the workgroup");
  constexpr int FILL_ROWS = WAVES * 64 / (MID_KS / 8);             // rows a round of the workgroup covers
  const int fill_row = threadIdx.x / (MID_KS / 8), fill_c = threadIdx.x % (MID_KS / 8);
  const int fill_first = (blockIdx.x / slices) % FILL;
  u32x4 fill[FILL];
#pragma unroll
  for (int it = 0; it < FILL; ++it) {
    const int row = ((it + fill_first) % FILL) * FILL_ROWS + fill_row;
    fill[it] = u32x4{0u, 0u, 0u, 0u};                             // rows beyond M are zeros
    if (row < a.M && k0 + fill_c * 8 < a.K)                       // (the last slice may be half a slice)
      fill[it] = *reinterpret_cast<const u32x4*>((const bf16_t*)a.A + (int64_t)row * a.lda + k0 + fill_c * 8);
  }

  // ---- then the first weights: behind every wave's requests for the batch, also in the
  // queue of loads that the waves of a CU share (the barrier waits for the issue, not the data)
  __syncthreads();
  auto row_ptr = [&](int rg) {       // rows beyond N are zeros of the last row of tiles; what they produce is never stored
    return WeightTiles::lane_place(a.W, a.w_stride, rg * ROWS + r16, g) + (int64_t)k0 * WeightTiles::PER_COLUMN;
  };
  // (row groups are dealt out so that every workgroup of a slice gets as many, within one)
  const int per_slice = gridDim.x / slices;
  int rg = blockIdx.x / slices + per_slice * wave;
  const bf16_t* w_cur = row_ptr(min(rg, row_groups - 1));
  static_assert(MID_HALF % MID_RING == 0 && MID_STEPS % MID_HALF == 0, "a ring slot means the same step in every turn of the loop");
  Chunk ring[MID_RING];
#pragma unroll
  for (int st = 0; st < MID_RING; ++st) ring[st].u = load_streamed(reinterpret_cast<const u32x4*>(w_cur + st * WeightTiles::TILE));

#pragma unroll
  for (int it = 0; it < FILL; ++it) {
    const int row = ((it + fill_first) % FILL) * FILL_ROWS + fill_row;
    *reinterpret_cast<u32x4*>(xs + row * MID_PITCH + fill_c * 8) = fill[it];
  }
  if (a.scale_ss != nullptr && (slices == 1 || blockIdx.x == gridDim.x - 1)) {
    // (with slices, the finishing kernel scales the rows: one workgroup here works the scales
    // out for it and leaves them behind the shares, so that not every workgroup there adds
    // up all the shares of every row again)
    row_scales<MT>(a, row_scale);
    if (slices > 1) {
      __syncthreads();
      if (threadIdx.x < MT * 16) scratch[(int64_t)row_groups * slices * MT * 256 + threadIdx.x] = row_scale[threadIdx.x];
    }
  }
  __syncthreads();

  const bf16_t* x_lane = xs + r16 * MID_PITCH + g * 8;
  const int steps = min(MID_STEPS, (a.K - k0) / 32);      // of this slice: 32, or fewer in a last, shorter one
  while (rg < row_groups) {
    const int rg_next = rg + stride;
    const bf16_t* w_next = row_ptr(rg_next < row_groups ? rg_next : rg);    // past the end: a repeat that nobody uses
    f32x4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int h = 0; h < steps; h += MID_HALF) {
#pragma unroll
      for (int s = 0; s < MID_HALF; ++s) {
        const int st = h + s;
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          const bf16x8 b = *reinterpret_cast<const bf16x8*>(x_lane + t * 16 * MID_PITCH + st * 32);
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ring[s % MID_RING].v, b, acc[t], 0, 0, 0);
        }
        const int ahead = st + MID_RING;
        const bf16_t* src = ahead < steps ? w_cur + ahead * WeightTiles::TILE : w_next + (ahead - steps) * WeightTiles::TILE;
        ring[s % MID_RING].u = load_streamed(reinterpret_cast<const u32x4*>(src));
      }
      // The order of issue, spelled out (groups: 0x008 matrix, 0x100 LDS read, 0x020 global
      // load): the batch operands of a step are read under the products of the step before,
      // and a ring slot is refilled as soon as its step has been multiplied.
      __builtin_amdgcn_sched_group_barrier(0x100, MT, 0);
#pragma unroll
      for (int s = 0; s < MID_HALF; ++s) {
        if (s + 1 < MID_HALF) __builtin_amdgcn_sched_group_barrier(0x100, MT, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, MT, 0);
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      }
    }

    const int n = rg * ROWS + 4 * g;
    if (slices > 1) {
      // this slice's share: register i of lane l (weight row 4*(l/16) + i, batch row l%16) of
      // tile t at [row group][slice][t][l][i], a kilobyte a store
      float* mine = scratch + ((int64_t)(rg * slices + slice) * MT) * 256 + lane * 4;
#pragma unroll
      for (int t = 0; t < MT; ++t) *reinterpret_cast<f32x4*>(mine + t * 256) = acc[t];
    } else {
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const int m = t * 16 + r16;
        float v[4] = {acc[t][0], acc[t][1], acc[t][2], acc[t][3]};
        if (a.scale_ss != nullptr) {
          const float scale = row_scale[m];
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] *= scale;
        }
        const bool live = m < a.M && n < a.N;
        finish_rows_ahead<EPI>(a, look_ahead<EPI>(a, m, n, live), m, n, live, v, rg, lane);
      }
    }
    rg = rg_next;
    w_cur = w_next;
  }
}

// The second kernel of a product cut into slices: wave (row group, t) adds the slices'
// shares of batch rows 16t .. 16t+15, in the order of the slices, and runs the epilogue.
// What the epilogue reads and all shares are asked for together.
template <int MT, int EPI>
__global__ __launch_bounds__(WAVES * 64) void mid_finish_kernel(Args a, int row_groups, int slices,
                                                                const float* __restrict__ scratch) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r16 = lane & 15, g = lane >> 4;
  const int unit = blockIdx.x * WAVES + wave;
  const int rg = unit / MT, t = unit - rg * MT;
  const bool here = rg < row_groups;                       // (whole waves)
  const int m = t * 16 + r16, n = rg * ROWS + 4 * g;
  const bool live = here && m < a.M && n < a.N;
  const Ahead<EPI> ahead = look_ahead<EPI>(a, m, n, live);
  // (the rows' scales: left behind the shares by the kernel before)
  const float scale = a.scale_ss != nullptr ? scratch[(int64_t)row_groups * slices * MT * 256 + m] : 1.f;
  const float* share = scratch + ((int64_t)min(rg, row_groups - 1) * slices * MT + t) * 256 + lane * 4;
  const int64_t step = (int64_t)MT * 256;
  f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
  constexpr int TOGETHER = 8;
  for (int s0 = 0; s0 < slices; s0 += TOGETHER) {
    f32x4 part[TOGETHER];
#pragma unroll
    for (int j = 0; j < TOGETHER; ++j)                     // past the end: a repeat that is not added
      part[j] = *reinterpret_cast<const f32x4*>(share + min(s0 + j, slices - 1) * step);
#pragma unroll
    for (int j = 0; j < TOGETHER; ++j)
      if (s0 + j < slices) acc += part[j];
  }
  float v[4] = {acc[0], acc[1], acc[2], acc[3]};
  if (a.scale_ss != nullptr) {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] *= scale;
  }
  if (here) finish_rows_ahead<EPI>(a, ahead, m, n, live, v, rg, lane);
}

// Returns true if the kernels for 17 to 64 rows took the product.
template <int MT>
bool launch_mid_rows(const Args& a, int epi, float* scratch, int64_t scratch_floats, int num_cus, hipStream_t stream) {
  const int row_groups = (a.N + ROWS - 1) / ROWS, slices = (a.K + MID_KS - 1) / MID_KS;
  if (slices > 1 && (scratch == nullptr || scratch_floats < (int64_t)row_groups * slices * MT * 256 + SS_STRIDE)) return false;
  int per_slice = num_cus / slices;                         // workgroups per slice: eight row groups at a time each
  if (per_slice < 1) per_slice = 1;
  // (all of a slice's share of the CUs, also where that leaves waves of a workgroup without a row
  // group: q/k/v at 64 rows on 256 workgroups of six busy waves instead of 192 of eight, the output
  // product on 256 of four instead of 128; a decode step at batch 64 5.744 -> 5.717 ms)
  if (per_slice > row_groups) per_slice = row_groups;
  const size_t lds = mid_lds_bytes(MT);
  const int finish_grid = (row_groups * MT + WAVES - 1) / WAVES;
#define GO(E)                                                                                                  \
  do {                                                                                                         \
    static bool raised = false;                                                                                \
    if (!raised) {                                                                                             \
      if (hipFuncSetAttribute((const void*)mid_kernel<MT, E>, hipFuncAttributeMaxDynamicSharedMemorySize,      \
                              (int)lds) != hipSuccess)                                                        \
        return false;                                                                                          \
      raised = true;                                                                                           \
    }                                                                                                          \
    mid_kernel<MT, E><<<per_slice * slices, WAVES * 64, lds, stream>>>(a, row_groups, slices, scratch);        \
    if (slices > 1) mid_finish_kernel<MT, E><<<finish_grid, WAVES * 64, 0, stream>>>(a, row_groups, slices, scratch); \
  } while (0)
  switch (epi) {
    case EPI_BF16: GO(EPI_BF16); break;
    case EPI_F32: GO(EPI_F32); break;
    case EPI_ADD: GO(EPI_ADD); break;
    case EPI_SWIGLU: GO(EPI_SWIGLU); break;
    default: GO(EPI_QKV); break;
  }
#undef GO
  return true;
}

// ------------------------------------------- 17 to 64 rows, many weight rows ---
// Where the weight rows alone fill the chip (gate/up, the vocabulary head) nothing has to be
// cut along K, and the shares, their buffer and the second kernel fall away: a product of
// 28,672 weight rows and 64 batch rows in four slices writes and reads a quarter of the
// weights' bytes again as shares.  Here a wave owns a group of 16 weight rows over the whole
// of K and a workgroup's eight waves walk K together, 512 columns at a time: the batch's
// columns of the moment lie in LDS, twice, so that the next 512 are brought (through
// registers, from L2) under the products of these; one barrier a slice.  The weights come as
// above, through a ring of loads that runs on across slices and row groups.
constexpr int WIDE_KS = 512, WIDE_STEPS = WIDE_KS / 32, WIDE_PITCH = WIDE_KS + 8;

constexpr int WIDE_MIN_GROUPS_A_CU = 6;
// (up to 48 rows from four on: gate/up of the 1B shape, 1,024 row groups on 256 workgroups of four busy
// waves, a decode step at batch 20 / 24 / 32 / 40 / 48 1.181 / 1.210 / 1.288 / 1.329 / 1.405 -> 1.139 / 1.166 /
// 1.240 / 1.326 / 1.399 ms; at 64 rows the pair of kernels stays, 1.591 against 1.616)
constexpr int WIDE_MIN_GROUPS_A_CU_FEW_ROWS = 4;       // of eight: below, the kernels above with their slices of K spread better

constexpr size_t mid_wide_lds_bytes(int mt) { return (size_t)2 * mt * 16 * WIDE_PITCH * sizeof(bf16_t); }

template <int MT, int EPI>
__global__ __launch_bounds__(WAVES * 64) void mid_wide_kernel(Args a, int row_groups, int busy) {
  extern __shared__ __attribute__((aligned(16))) char wide_lds[];
  bf16_t* xs = (bf16_t*)wide_lds;                                    // [2][MT * 16][WIDE_PITCH]
  __shared__ float row_scale[SS_STRIDE];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r16 = lane & 15, g = lane >> 4;
  const int slices = a.K / WIDE_KS, tiles = a.K / 32;

  // a slice of the batch: MT * 16 rows of 64 chunks of 16 bytes, a row a wave and round
  constexpr int FILL = MT * 16 / WAVES;
  auto ask = [&](u32x4* fill, int slice) {
#pragma unroll
    for (int it = 0; it < FILL; ++it) {
      const int row = it * WAVES + wave;
      fill[it] = u32x4{0u, 0u, 0u, 0u};                              // rows beyond M are zeros
      if (row < a.M) fill[it] = *reinterpret_cast<const u32x4*>((const bf16_t*)a.A + (int64_t)row * a.lda + slice * WIDE_KS + lane * 8);
    }
  };
  auto put = [&](const u32x4* fill, int buf) {
#pragma unroll
    for (int it = 0; it < FILL; ++it)
      *reinterpret_cast<u32x4*>(xs + ((buf * MT * 16) + it * WAVES + wave) * WIDE_PITCH + lane * 8) = fill[it];
  };
  auto row_ptr = [&](int rg) {       // rows beyond N are zeros of the last row of tiles; what they produce is never stored
    return WeightTiles::lane_place(a.W, a.w_stride, min(rg, row_groups - 1) * ROWS + r16, g);
  };

  // the batch first (from L2: it must not wait in line behind weights from memory), then the ring
  u32x4 fill[FILL];
  ask(fill, 0);
  // `busy` waves of a workgroup take a row group each in every round; the others only help to bring
  // the batch (1,792 row groups over 256 CUs are seven a workgroup: with eight, 224 workgroups would
  // leave 32 CUs without work)
  const int stride = gridDim.x * busy;
  const bool works = wave < busy;
  const bf16_t* w_cur = row_ptr(blockIdx.x * busy + wave);
  constexpr int RING = mid_ring(MT);          // (8 or 16 loads a wave in flight at 64 rows: the step within 1 %)
  static_assert(WIDE_STEPS % RING == 0, "a ring slot must mean the same step in every slice");
  Chunk ring[RING];
  if (works) {
#pragma unroll
    for (int st = 0; st < RING; ++st) ring[st].u = load_streamed(reinterpret_cast<const u32x4*>(w_cur + st * WeightTiles::TILE));
  }
  put(fill, 0);
  // (the rows' shares meet at the first slice's barrier: see ask_shares; with one slice there is none)
  __shared__ float share_part[WAVES][SS_STRIDE];
  bool late = a.scale_ss != nullptr && slices > 1 && a.scale_blocks <= Shares<MT>::BLOCKS;
  Shares<MT> shares;
  if (late) ask_shares<MT>(a, shares);
  else if (a.scale_ss != nullptr) row_scales<MT>(a, row_scale);
  __syncthreads();

  int buf = 0;
  for (int first = blockIdx.x * busy; first < row_groups; first += stride) {      // (the same for all waves: barriers inside)
    const int rg = works ? first + wave : row_groups;
    const bf16_t* w_next = row_ptr(rg + stride);                     // past the end: a repeat that nobody uses
    f32x4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < slices; ++s) {
      ask(fill, s + 1 < slices ? s + 1 : 0);
      const bf16_t* x_lane = xs + (buf * MT * 16 + r16) * WIDE_PITCH + g * 8;
      if (works) {                 // (the same for the whole wave)
#pragma unroll
        for (int st = 0; st < WIDE_STEPS; ++st) {
#pragma unroll
          for (int t = 0; t < MT; ++t) {
            const bf16x8 b = *reinterpret_cast<const bf16x8*>(x_lane + t * 16 * WIDE_PITCH + st * 32);
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ring[st % RING].v, b, acc[t], 0, 0, 0);
          }
          const int ahead = s * WIDE_STEPS + st + RING;
          const bf16_t* src = ahead < tiles ? w_cur + (int64_t)ahead * WeightTiles::TILE : w_next + (int64_t)(ahead - tiles) * WeightTiles::TILE;
          ring[st % RING].u = load_streamed(reinterpret_cast<const u32x4*>(src));
        }
        // (the order of issue as in the kernel above: LDS reads of a step under the products of the
        // step before, a ring slot refilled as soon as its step has been multiplied)
        __builtin_amdgcn_sched_group_barrier(0x100, MT, 0);
#pragma unroll
        for (int st = 0; st < WIDE_STEPS; ++st) {
          if (st + 1 < WIDE_STEPS) __builtin_amdgcn_sched_group_barrier(0x100, MT, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, MT, 0);
          __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
      }
      put(fill, buf ^ 1);          // read last in the slice before this one: everybody has passed that barrier
      if (late && s == 0) put_shares<MT>(a, shares, share_part);
      __syncthreads();
      if (late && s == 0) {        // (read after the next slice's barrier at the earliest)
        if (threadIdx.x < MT * 16) row_scale[threadIdx.x] = scale_of(a, share_part, threadIdx.x);
        late = false;
      }
      buf ^= 1;
    }
    if (rg < row_groups) {
      const int n = rg * ROWS + 4 * g;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const int m = t * 16 + r16;
        float v[4] = {acc[t][0], acc[t][1], acc[t][2], acc[t][3]};
        if (a.scale_ss != nullptr) {
          const float scale = row_scale[m];
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] *= scale;
        }
        const bool live = m < a.M && n < a.N;
        finish_rows_ahead<EPI>(a, look_ahead<EPI>(a, m, n, live), m, n, live, v, rg, lane);
      }
    }
    w_cur = w_next;
  }
}

// Returns true if the kernel for 17 to 64 rows and many weight rows took the product.
template <int MT>
bool launch_mid_wide(const Args& a, int epi, int num_cus, hipStream_t stream) {
  const int row_groups = (a.N + ROWS - 1) / ROWS;
  const int per = (row_groups + num_cus * WAVES - 1) / (num_cus * WAVES);      // rounds of a workgroup, all but equal
  // (gate/up of the 8B shape: seven waves on 256 CUs instead of eight on 224: a decode step at batch 64
  // 5.73 -> 5.61 ms, at 32 4.68 -> 4.60, at 24 4.38 -> 4.30, the two libraries in turn on one box)
  int busy = (row_groups + num_cus * per - 1) / (num_cus * per);                // waves of a workgroup with a row group a round
  if (busy > WAVES) busy = WAVES;
  const int grid = (row_groups + busy * per - 1) / (busy * per);
  const size_t lds = mid_wide_lds_bytes(MT);
#define GO(E)                                                                                                  \
  do {                                                                                                         \
    static bool raised = false;                                                                                \
    if (!raised) {                                                                                             \
      if (hipFuncSetAttribute((const void*)mid_wide_kernel<MT, E>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                              (int)lds) != hipSuccess)                                                        \
        return false;                                                                                          \
      raised = true;                                                                                           \
    }                                                                                                          \
    mid_wide_kernel<MT, E><<<grid, WAVES * 64, lds, stream>>>(a, row_groups, busy);                            \
  } while (0)
  switch (epi) {
    case EPI_BF16: GO(EPI_BF16); break;
    case EPI_F32: GO(EPI_F32); break;
    case EPI_ADD: GO(EPI_ADD); break;
    case EPI_SWIGLU: GO(EPI_SWIGLU); break;
    default: GO(EPI_QKV); break;
  }
#undef GO
  return true;
}

// ------------------------------------------------------------ wide products ---
// For products with many weight rows (gate/up, the vocabulary head) and at most 16
// batch rows.  Workgroups are persistent: each walks several groups of 16 weight
// rows.  The batch rows are turned into matrix operands once per workgroup and stay
// in registers (with the norm folded in if asked: this makes the fusion free), so
// the loop streams W only; loads run a fixed number of steps ahead, across the
// boundary between row groups.  K must be exactly STEPS * 32 * WAVES, so that the
// loop has no condition in it.
template <int STEPS, bool NORM, int EPI>
__global__ __launch_bounds__(WAVES * 64) void wide_kernel(Args a, int row_groups) {
  // (loads in flight a wave; it must divide STEPS.  Measured inside the decode step, gate/up of the
  // 8B shape: 44.7 µs with 16, 43.0 with 8, 43.8 with 4)
  constexpr int RING = STEPS % 8 == 0 ? 8 : STEPS % 10 == 0 ? 10 : STEPS % 6 == 0 ? 6 : 4;
  static_assert(STEPS % RING == 0, "a ring slot must mean the same step in every row group");
  __shared__ float partial[WAVES][64][4];
  __shared__ float ss_part[WAVES][16];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r16 = lane & 15, g = lane >> 4;
  // local step s of this wave covers columns koff(s) .. koff(s)+31: blocks of four
  // steps are dealt to the waves in turn
  auto koff = [&](int s) { return ((((s >> 2) * WAVES + wave) << 2) + (s & 3)) * 32; };

  // ---- the batch rows as operands, once -------------------------------------------
  Chunk b[STEPS];
  float ss = 0.f;
  {
    int m = min(r16, a.M - 1);
    if (NORM && a.rows) m = a.rows[m];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int k = koff(s) + g * 8;
      if constexpr (!NORM) {
        b[s].u = *reinterpret_cast<const u32x4*>((const bf16_t*)a.A + (int64_t)m * a.lda + k);
      } else {
        const float* xr = (const float*)a.A + (int64_t)m * a.lda + k;
        const f32x4 x0 = load_f4(xr), x1 = load_f4(xr + 4);
        float nw[8];
        if (a.norm_weight_is_f32) {
          const f32x4 n0 = load_f4((const float*)a.norm_weight + k), n1 = load_f4((const float*)a.norm_weight + k + 4);
#pragma unroll
          for (int i = 0; i < 4; ++i) { nw[i] = n0[i]; nw[4 + i] = n1[i]; }
        } else {
          Chunk c;
          c.u = *reinterpret_cast<const u32x4*>((const bf16_t*)a.norm_weight + k);
#pragma unroll
          for (int i = 0; i < 8; ++i) nw[i] = bf16_to_float(c.e[i]);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          ss = fmaf(x0[i], x0[i], ss);
          ss = fmaf(x1[i], x1[i], ss);
          b[s].e[i] = float_to_bf16(x0[i] * nw[i]);
          b[s].e[4 + i] = float_to_bf16(x1[i] * nw[4 + i]);
        }
      }
    }
  }
  float scale = 1.f;
  if (NORM) {
    ss += __shfl_xor(ss, 16, 64);
    ss += __shfl_xor(ss, 32, 64);
    if (g == 0) ss_part[wave][r16] = ss;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) t += ss_part[w][r16];
    scale = 1.0f / sqrtf(t / (float)a.K + a.eps);     // for this lane's batch row (lane % 16)
  }

  // ---- stream W ---------------------------------------------------------------------
  auto row_ptr = [&](int rg) { return WeightTiles::lane_place(a.W, a.w_stride, rg * ROWS + r16, g); };
  int rg = blockIdx.x;                       // the host launches at most row_groups workgroups
  const bf16_t* w_cur = row_ptr(rg);
  Chunk ring[RING];
#pragma unroll
  for (int s = 0; s < RING; ++s) ring[s].u = load_streamed(reinterpret_cast<const u32x4*>(w_cur + koff(s) * WeightTiles::PER_COLUMN));
  __shared__ float share_part[WAVES][SS_STRIDE];
  const bool scaled = !NORM && a.scale_ss != nullptr;
  bool late = scaled && a.scale_blocks <= Shares<1>::BLOCKS;      // the shares meet at the first row group's barrier
  Shares<1> shares;
  if (late) {
    ask_shares<1>(a, shares);
  } else if (scaled) {
    __shared__ float row_scale[SS_STRIDE];
    row_scales<1>(a, row_scale);
    __syncthreads();
    scale = row_scale[min(r16, a.M - 1)];
  }

  while (rg < row_groups) {
    const int rg_next = rg + gridDim.x;
    // after the last group the loads ahead re-read it: harmless, and the loop stays free of conditions
    const bf16_t* w_next = row_ptr(rg_next < row_groups ? rg_next : rg);
    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ring[s % RING].v, b[s].v, acc, 0, 0, 0);
      const int ahead = s + RING;          // refill the slot RING steps ahead
      ring[s % RING].u = ahead < STEPS ? load_streamed(reinterpret_cast<const u32x4*>(w_cur + koff(ahead) * WeightTiles::PER_COLUMN))
                                       : load_streamed(reinterpret_cast<const u32x4*>(w_next + koff(ahead - STEPS) * WeightTiles::PER_COLUMN));
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) partial[wave][lane][i] = acc[i];
    if (late) put_shares<1>(a, shares, share_part);
    __syncthreads();
    if (late) {
      scale = scale_of(a, share_part, min(r16, a.M - 1));
      late = false;
    }
    if (wave == 0) {
      // register i of lane l: weight row 4*(l/16) + i, batch row l%16
      const int m = r16, n = rg * ROWS + 4 * g;
      if (m < a.M && n < a.N) {
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float t = 0.f;
#pragma unroll
          for (int w = 0; w < WAVES; ++w) t += partial[w][lane][i];
          v[i] = t * scale;
        }
        epilogue<EPI>(a, m, n, v);
      }
    }
    __syncthreads();
    rg = rg_next;
    w_cur = w_next;
  }
}

template <bool NORM, int EPI>
bool launch_wide_steps(const Args& a, int row_groups, int grid, hipStream_t stream) {
  const int steps = a.K / (32 * WAVES);      // local steps per wave; K == steps * 32 * WAVES was checked
  if (steps == 4) wide_kernel<4, NORM, EPI><<<grid, WAVES * 64, 0, stream>>>(a, row_groups);
  else if (steps == 8) wide_kernel<8, NORM, EPI><<<grid, WAVES * 64, 0, stream>>>(a, row_groups);
  else if (steps == 12) wide_kernel<12, NORM, EPI><<<grid, WAVES * 64, 0, stream>>>(a, row_groups);
  else if (steps == 16) wide_kernel<16, NORM, EPI><<<grid, WAVES * 64, 0, stream>>>(a, row_groups);
  else if (steps == 20 || steps == 32) {
    // (with the norm folded in, the float32 rows on their way to operands need more registers
    // than a wave of eight a CU has: those products stay with the streaming kernel)
    if constexpr (NORM) return false;
    else if (steps == 20) wide_kernel<20, false, EPI><<<grid, WAVES * 64, 0, stream>>>(a, row_groups);
    else wide_kernel<32, false, EPI><<<grid, WAVES * 64, 0, stream>>>(a, row_groups);
  } else return false;      // other widths: the streaming kernel takes them
  return true;
}

// Returns true if the wide kernel took the product.
bool launch_wide(const Args& a, bool norm, int epi, hipStream_t stream) {
  static int num_cus = 0;
  if (num_cus == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return false;
    num_cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
  }
  const int row_groups = (a.N + ROWS - 1) / ROWS;
  if (a.M > 16 || a.K % (128 * WAVES) != 0 || a.K > 32 * 32 * WAVES) return false;
  // from two row groups a workgroup on: the workgroups then share the weight rows evenly, where
  // one row group each leaves a second round that fills a part of the chip only (q/k/v of the 8B
  // shape, 384 row groups: 1.5 us a layer inside the decode step; and better than the streaming
  // kernel with two workgroups a CU: 3.465 ms a step against 3.52)
  const int per = (row_groups + num_cus - 1) / num_cus;       // row groups per workgroup, all but equal
  if (per < 2) return false;
  const int grid = (row_groups + per - 1) / per;
#define GO(NORM_, E) return launch_wide_steps<NORM_, E>(a, row_groups, grid, stream)
  if (norm) {
    switch (epi) {
      case EPI_BF16: GO(true, EPI_BF16);
      case EPI_F32: GO(true, EPI_F32);
      case EPI_ADD: GO(true, EPI_ADD);
      case EPI_SWIGLU: GO(true, EPI_SWIGLU);
      default: GO(true, EPI_QKV);
    }
  }
  switch (epi) {
    case EPI_BF16: GO(false, EPI_BF16);
    case EPI_F32: GO(false, EPI_F32);
    case EPI_ADD: GO(false, EPI_ADD);
    case EPI_SWIGLU: GO(false, EPI_SWIGLU);
    default: GO(false, EPI_QKV);
  }
#undef GO
}

}  // namespace

// One entry point for every variant.  a_is_f32 != 0 selects the fused RMSNorm (M <= 16).
// epi: 0 bfloat16 store, 1 float32 store, 2 float32 accumulate, 3 SiLU gate, 4 q/k/v.
// emit_out (with epi 2): also write bfloat16(C_new * emit_weight) to emit_out [M, N] and this
// product's shares of the rows' sums of squares to emit_ss (ceil(N / 16) x 64 floats).
// scale_ss: shares left by such a product (scale_blocks x 64 floats) over rows of width K:
// the finished sums are scaled by 1 / sqrt(sum / K + scale_eps).
// scratch: for 17 to 64 rows and K a multiple of 256, a faster pair of kernels that needs
// ceil(N / 16) * ceil(K / 1024) * ceil(M / 16) * 256 + 64 floats of scratch (none for K <= 1,024);
// without it, or for other sizes, or where it would not pay, the streaming kernel takes
// the product (force_mid: 1 takes the pair of kernels with slices of K wherever it applies,
// 2 the kernel for many weight rows: for tests).
HFEE_API int hfee_gemm_skinny(void* C, int64_t ldc, const void* A, int a_is_f32, int64_t lda, const void* W,
                              int64_t w_stride, int M, int N, int K, int epi,
                              const void* norm_weight, int norm_weight_is_f32, float eps, const int* rows,
                              const int* positions, const int* token_segment, const int* block_tables,
                              int bt_stride, const float* cos_table, const float* sin_table, int half,
                              int table_positions, void* cache, int num_heads, int kv_heads, int head_dim,
                              int page_size, const void* emit_weight, int emit_weight_is_f32, void* emit_out,
                              int64_t ld_emit, float* emit_ss, const float* scale_ss, int scale_blocks,
                              float scale_eps, float* scratch, int64_t scratch_floats, int force_mid,
                              hipStream_t stream) {
  HFEE_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_skinny: bad sizes M=%d N=%d K=%d", M, N, K);
  if (M == 0) return 0;
  HFEE_REQUIRE(epi >= 0 && epi <= 4, "gemm_skinny: unknown epilogue %d", epi);
  HFEE_REQUIRE(M <= 64, "gemm_skinny: at most 64 rows, got %d", M);
  HFEE_REQUIRE(K % 8 == 0 && lda % 8 == 0 && (uintptr_t)A % 16 == 0 && (uintptr_t)W % 16 == 0,
               "gemm_skinny: K and lda must be multiples of 8 and the operands 16-byte aligned");
  HFEE_REQUIRE(lda >= K, "gemm_skinny: lda is shorter than a row");
  HFEE_REQUIRE(w_stride == WeightTiles::row_stride(K),
               "gemm_skinny: the weight must come in tiles of 16 x 32 (%lld elements a row of tiles for K = %d, got %lld)",
               (long long)WeightTiles::row_stride(K), K, (long long)w_stride);
  const bool norm = a_is_f32 != 0;
  if (norm) {
    HFEE_REQUIRE(M <= 16, "gemm_skinny: the fused norm takes at most 16 rows, got %d", M);
    HFEE_REQUIRE(norm_weight != nullptr && eps >= 0.f, "gemm_skinny: the fused norm needs its weight");
    HFEE_REQUIRE((uintptr_t)norm_weight % 16 == 0, "gemm_skinny: the norm weight must be 16-byte aligned");
  } else {
    HFEE_REQUIRE(rows == nullptr, "gemm_skinny: a row gather needs the fused norm");
  }
  Args a{};
  a.C = C; a.ldc = ldc; a.A = A; a.lda = lda; a.W = (const bf16_t*)W; a.w_stride = w_stride;
  a.M = M; a.N = N; a.K = K;
  a.norm_weight = norm_weight; a.norm_weight_is_f32 = norm_weight_is_f32; a.eps = eps; a.rows = rows;
  if (epi == EPI_SWIGLU) {
    HFEE_REQUIRE(N % 2 == 0 && ldc >= N / 2, "gemm_skinny: the SiLU gate needs an even N and ldc >= N/2");
  } else if (epi == EPI_QKV) {
    HFEE_REQUIRE(head_dim > 0 && head_dim % 4 == 0 && num_heads > 0 && kv_heads > 0 &&
                 N == (num_heads + 2 * kv_heads) * head_dim, "gemm_skinny: q/k/v rows do not match the heads");
    HFEE_REQUIRE(ldc >= (int64_t)num_heads * head_dim && ldc % 4 == 0 && (uintptr_t)C % 8 == 0,
                 "gemm_skinny: the q output is too narrow or not 8-byte aligned");
    HFEE_REQUIRE(positions != nullptr, "gemm_skinny: q/k/v needs positions");
    HFEE_REQUIRE(half >= 0 && 2 * half <= head_dim, "gemm_skinny: rotary width exceeds the head");
    HFEE_REQUIRE(cos_table == nullptr || table_positions > 0, "gemm_skinny: empty rotation table");
    if (make_cache_layout(&a.qkv.lay, kv_heads, head_dim, page_size)) return 1;
    HFEE_REQUIRE(cache == nullptr || (token_segment != nullptr && block_tables != nullptr),
                 "gemm_skinny: writing the cache needs block tables");
    a.qkv.positions = positions; a.qkv.token_segment = token_segment; a.qkv.block_tables = block_tables;
    a.qkv.bt_stride = bt_stride; a.qkv.cos_table = cos_table; a.qkv.sin_table = sin_table; a.qkv.half = half;
    a.qkv.cache = cache; a.qkv.num_heads = num_heads;
  } else {
    HFEE_REQUIRE(ldc >= N, "gemm_skinny: ldc is shorter than a row");
  }
  if (emit_out != nullptr) {
    HFEE_REQUIRE(epi == EPI_ADD && !norm, "gemm_skinny: a following norm is emitted by the accumulating product only");
    HFEE_REQUIRE(emit_weight != nullptr && emit_ss != nullptr && ld_emit >= N, "gemm_skinny: incomplete arguments for the emitted norm");
    a.emit_weight = emit_weight; a.emit_weight_is_f32 = emit_weight_is_f32; a.emit_out = (bf16_t*)emit_out;
    a.ld_emit = ld_emit; a.emit_ss = emit_ss;
  }
  if (scale_ss != nullptr) {
    HFEE_REQUIRE(!norm && scale_blocks > 0 && scale_eps >= 0.f, "gemm_skinny: a row scale needs its shares and no norm of its own");
    a.scale_ss = scale_ss; a.scale_blocks = scale_blocks; a.scale_eps = scale_eps;
  }
  const int mt = (M + 15) / 16;
  // Where the kernels with the batch in LDS win, from fits to measured times in microseconds
  // (1,024 to 15,360 weight rows, K from 2,048 to 14,336, 17 to 64 batch rows): the streaming
  // kernel takes the weights' time at 5 TB/s, a launch, and 0.052 a batch row and 1,024
  // columns for reading the batch again with every 16 weight rows (more where the row
  // groups outnumber the CUs); the pair of kernels takes 16.5, or the weights' time at
  // 4.65 TB/s and 4 where that is more, whatever the number of batch rows.
  const double weight_mb = 2e-6 * (double)N * (double)K;
  const double rounds = ((N + ROWS - 1) / ROWS) / 256.0;
  const double t_streaming = weight_mb / 5.0 + 3.0 + 0.052 * (K / 1024.0) * (rounds > 1.0 ? rounds : 1.0) * M;
  const double t_pair = weight_mb * 0.215 + 4.0 > 16.5 ? weight_mb * 0.215 + 4.0 : 16.5;
  const bool mid_pays = t_pair < 0.95 * t_streaming;
  static int num_cus = 0;
  if (num_cus == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    num_cus = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess &&
               prop.multiProcessorCount > 0) ? prop.multiProcessorCount : 256;
  }
  // weight rows enough for most of the CUs to have eight row groups each: nothing is cut along K
  const bool wide_rows = (N + ROWS - 1) / ROWS >= WIDE_MIN_GROUPS_A_CU * num_cus ||
                         ((N + ROWS - 1) / ROWS >= WIDE_MIN_GROUPS_A_CU_FEW_ROWS * num_cus && mt <= 3);
  if (!norm && mt > 1 && K % WIDE_KS == 0 && (force_mid == 2 || (force_mid == 0 && wide_rows))) {
    const bool took = mt == 2 ? launch_mid_wide<2>(a, epi, num_cus, stream)
                    : mt == 3 ? launch_mid_wide<3>(a, epi, num_cus, stream)
                              : launch_mid_wide<4>(a, epi, num_cus, stream);
    if (took) {
      HFEE_CHECK_LAUNCH("gemm_skinny(17 to 64 rows, many weight rows)");
      return 0;
    }
  }
  if (!norm && mt > 1 && K % 256 == 0 && (mid_pays || force_mid == 1)) {
    const bool took = mt == 2 ? launch_mid_rows<2>(a, epi, scratch, scratch_floats, num_cus, stream)
                    : mt == 3 ? launch_mid_rows<3>(a, epi, scratch, scratch_floats, num_cus, stream)
                              : launch_mid_rows<4>(a, epi, scratch, scratch_floats, num_cus, stream);
    if (took) {
      HFEE_CHECK_LAUNCH("gemm_skinny(17 to 64 rows)");
      return 0;
    }
  }
  if (emit_out == nullptr && launch_wide(a, norm, epi, stream)) {
    HFEE_CHECK_LAUNCH("gemm_skinny(wide)");
    return 0;
  }
  if (norm) launch_epi<1, true>(a, epi, stream);
  else if (mt == 1) launch_epi<1, false>(a, epi, stream);
  else if (mt == 2) launch_epi<2, false>(a, epi, stream);
  else if (mt == 3) launch_epi<3, false>(a, epi, stream);
  else launch_epi<4, false>(a, epi, stream);
  HFEE_CHECK_LAUNCH("gemm_skinny");
  return 0;
}

// The q/k/v product of more than 64 rows (a prompt's portion) with the same epilogue, through
// the tiled kernels: W as rows [N, K] with leading dimension ldw, not in tiles.
HFEE_API int hfee_gemm_qkv_rows(void* C, int64_t ldc, const void* A, int64_t lda, const void* W, int64_t ldw, int M,
                                int N, int K, const int* positions, const int* token_segment, const int* block_tables,
                                int bt_stride, const float* cos_table, const float* sin_table, int half,
                                int table_positions, void* cache, int num_heads, int kv_heads, int head_dim,
                                int page_size, hipStream_t stream) {
  HFEE_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_qkv_rows: bad sizes M=%d N=%d K=%d", M, N, K);
  HFEE_REQUIRE(head_dim > 0 && head_dim % 4 == 0 && num_heads > 0 && kv_heads > 0 &&
               N == (num_heads + 2 * kv_heads) * head_dim, "gemm_qkv_rows: q/k/v rows do not match the heads");
  HFEE_REQUIRE(ldc >= (int64_t)num_heads * head_dim && ldc % 4 == 0 && (uintptr_t)C % 8 == 0,
               "gemm_qkv_rows: the q output is too narrow or not 8-byte aligned");
  HFEE_REQUIRE(lda >= K && ldw >= K, "gemm_qkv_rows: a leading dimension is shorter than its row");
  HFEE_REQUIRE(positions != nullptr, "gemm_qkv_rows: q/k/v needs positions");
  HFEE_REQUIRE(half >= 0 && 2 * half <= head_dim, "gemm_qkv_rows: rotary width exceeds the head");
  HFEE_REQUIRE(cos_table == nullptr || table_positions > 0, "gemm_qkv_rows: empty rotation table");
  QkvArgs q{};
  if (make_cache_layout(&q.lay, kv_heads, head_dim, page_size)) return 1;
  HFEE_REQUIRE(cache == nullptr || (token_segment != nullptr && block_tables != nullptr),
               "gemm_qkv_rows: writing the cache needs block tables");
  q.positions = positions; q.token_segment = token_segment; q.block_tables = block_tables;
  q.bt_stride = bt_stride; q.cos_table = cos_table; q.sin_table = sin_table; q.half = half;
  q.cache = cache; q.num_heads = num_heads;
  return hfee_gemm_bf16_qkv(C, ldc, A, lda, W, ldw, M, N, K, &q, 0, stream);
}
