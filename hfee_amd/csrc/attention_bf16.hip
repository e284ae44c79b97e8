// Paged causal attention on the matrix cores, bfloat16 in, float32 softmax and
// accumulation.  Compiled once per head size (HFEE_HEAD_DIM, a multiple of 16).
//
// The formulas are the reference's (/root/reference/internal/llm/forward.go:144-178):
// head h reads KV head h / (H/K); scores are dot * scale over the keys
// 0..pos (the range is the mask; a window narrows it), softmax, weighted sum of
// the values.  The softmax runs online over tiles of 32 keys.
//
// One wave owns 32 query slots.  Per key tile it computes S^T = K Q^T with
// v_mfma_f32_32x32x16_bf16 (the key rows come straight from the page as the A
// operand, 16 bytes per lane), keeps each query's running maximum and sum in the
// lane that holds that query's column, and feeds P^T back as the B operand of
// O^T += V^T P^T without leaving registers: the A operand of that product is the
// transposed value page, whose 4-key runs are contiguous.  The k index of a matrix
// instruction is only a label shared by its two operands, so the keys that a lane
// happens to hold after the first product (8b + 4G + i) need no shuffle.
//
//   prefill: a slot is a position of one segment's portion, all for one head;
//   decode:  a slot is one of the heads that share a KV head, all at one position;
//            the keys may be split over several waves whose partial results a
//            second kernel joins.
#include "common.h"

#include <climits>
#include <type_traits>

#ifndef HFEE_HEAD_DIM
#error "compile with -DHFEE_HEAD_DIM=<multiple of 16>"
#endif

using namespace hfee;

HFEE_DEFINE_LAST_ERROR

namespace {

constexpr int HD = HFEE_HEAD_DIM;
static_assert(HD % 16 == 0 && HD >= 16 && HD <= 256, "head size must be a multiple of 16 in 16..256");
constexpr int NC = HD / 16;            // 16-wide chunks of the head for Q K^T
constexpr int NDT = (HD + 31) / 32;    // 32-wide tiles of the head for P V
constexpr float LOG2E = 1.4426950408889634f;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

union Op {          // one matrix-instruction operand: eight bfloat16
  u32x4 u;
  u32x2 h[2];
  bf16x8 v;
  bf16_t e[8];
};

struct Tile {
  // running state of 32 query slots; this lane's slot is lane % 32
  float m;              // reference of the exponentials: at most SLACK below the running maximum (log2 domain)
  float l;              // running sum
  f32x16 o[NDT];        // O^T: register r of tile t is dim 32t + 8*(r/4) + 4*(lane/32) + r%4
};

// The operands of one tile of 32 keys: the key rows for S^T = K Q^T and the value
// columns for O^T += V^T P^T.  Step u of P V covers keys k0+16u .. k0+16u+15; a lane's
// operand slots 0..3 are keys 16u + 4G + 0..3 and slots 4..7 keys 16u + 8 + 4G + 0..3
// (as P holds them after the first product): the cache stores a value column's slots
// in exactly that order, so the operand is one 16-byte load.
struct TileOps {
  Op k[NC];
  Op v[2][NDT];
};

// The operand of s_waitcnt that waits until at most n vector memory operations are outstanding
// and for nothing else (gfx9 encoding: vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8).
constexpr int vmcnt_only(int n) { return (n & 15) | (7 << 4) | (15 << 8) | ((n >> 4) << 14); }
// The same, and until every LDS read of this wave has returned (lgkmcnt 0).
constexpr int vmcnt_and_lds_reads(int n) { return (n & 15) | (7 << 4) | (0 << 8) | ((n >> 4) << 14); }

// 64 consecutive entries of a sequence's block table, one per lane, so that a tile's
// page numbers come from a register shuffle instead of a load that the tile's own loads
// would have to wait for.
struct PageWindow {
  int base;      // first block held; -1: nothing yet
  int page;      // this lane's entry: block base + lane

  __device__ __forceinline__ void fill(const int* __restrict__ bt, int bt_stride, int block) {
    base = block;
    const int mine = block + (int)(threadIdx.x & 63);
    page = mine < bt_stride ? bt[mine] : 0;
  }
  // the page of `block`, which must lie in base .. base + 63
  __device__ __forceinline__ int of(int block) const { return __shfl(page, block - base, 64); }
};

// What of a lane's addresses does not change from tile to tile (in elements from the
// start of a page): the tile adds the page and a uniform slot offset.
struct LaneOffsets {
  int64_t key;              // this lane's key row within a page (k0 % page_size == 0), its half of a chunk
  int64_t value[NDT];       // this lane's value column of each 32-wide part of the head, its half of the slots
};

__device__ __forceinline__ LaneOffsets lane_offsets(const CacheLayout& lay, int kvh) {
  const int lane = threadIdx.x & 63, r32 = lane & 31, G = lane >> 5;
  LaneOffsets o;
  o.key = lay.key_offset(0, kvh, r32 & (lay.page_size - 1), 0) + G * 8;
#pragma unroll
  for (int t = 0; t < NDT; ++t)
    o.value[t] = lay.value_column(0, kvh, min(32 * t + r32, HD - 1)) + 8 * G;   // rows beyond the head repeat its last one
  return o;
}

// Issues every load of the tile k0 .. k0+31 into registers.  kv_first..kv_last: the keys
// whose pages may be touched at all (a window group has given back the pages before
// kv_first; nothing exists after kv_last): a page without such a key is replaced by page
// 0.  What is read beside the keys that a slot sees is masked or multiplied by zero (the
// cache never holds anything but finite numbers).  The tile lies in at most two pages;
// their numbers are scalars out of the page window, and a lane's address is one of two
// bases plus what lane_offsets worked out once.
template <bool STREAMED>
__device__ __forceinline__ void load_tile(TileOps& ops, const bf16_t* __restrict__ cache, const CacheLayout& lay,
                                          const LaneOffsets& off, const int* __restrict__ bt, int bt_stride,
                                          PageWindow& pages, int k0, int kv_first, int kv_last) {
  const int r32 = threadIdx.x & 31;
  const int block_a = k0 >> lay.page_shift, block_b = (k0 + 16) >> lay.page_shift;
  if (pages.base < 0 || block_a < pages.base || block_b >= pages.base + 64) pages.fill(bt, bt_stride, block_a);
  const bool ok_a = k0 <= kv_last && k0 + 15 >= kv_first, ok_b = k0 + 16 <= kv_last && k0 + 31 >= kv_first;
  const int page_a = ok_a ? __builtin_amdgcn_readlane(pages.page, __builtin_amdgcn_readfirstlane(block_a - pages.base)) : 0;
  const int page_b = ok_b ? __builtin_amdgcn_readlane(pages.page, __builtin_amdgcn_readfirstlane(block_b - pages.base)) : 0;
  const bf16_t* base_a = cache + (int64_t)page_a * lay.page_stride;
  const bf16_t* base_b = cache + (int64_t)page_b * lay.page_stride;
  const int in_page = k0 & (lay.page_size - 1);
  // (a key's chunk c, 16 dims, lies a chunk stride on; the tile's place in its page adds slots of 16 dims)
  const bf16_t* krow = (r32 < 16 ? base_a : base_b) + off.key + in_page * 16;
  const int64_t chunk_stride = lay.key_chunk_stride();
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    if constexpr (STREAMED) ops.k[c].u = load_streamed(reinterpret_cast<const u32x4*>(krow + c * chunk_stride));
    else ops.k[c].u = *reinterpret_cast<const u32x4*>(krow + c * chunk_stride);
  }
  const bf16_t* vbase[2] = {base_a + in_page, base_b + ((k0 + 16) & (lay.page_size - 1))};
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int t = 0; t < NDT; ++t) {
      if constexpr (STREAMED) ops.v[u][t].u = load_streamed(reinterpret_cast<const u32x4*>(vbase[u] + off.value[t]));
      else ops.v[u][t].u = *reinterpret_cast<const u32x4*>(vbase[u] + off.value[t]);
    }
}

// Adds the keys k0 .. k0+31 to the running state.  q_op: this slot's query, pre-loaded
// as NC operands.  pos: this slot's position (keys lo..pos are visible; -1 for an unused
// slot).  key_op(c) and value_op(u, t) hand over the tile's operands: from registers, or
// from a tile in LDS that several waves share.
struct Nothing {
  __device__ __forceinline__ void operator()() const {}
};

// under_scores(): what the caller wants issued behind the score products, while the matrix pipe
// works on them (a request for a tile to come).
template <class KeyOp, class ValueOp, class Under = Nothing>
__device__ __forceinline__ void compute_tile_with(Tile& st, const Op* q_op, KeyOp key_op, ValueOp value_op, int k0,
                                                  int pos, int lo, float scale_log2, bool all_visible,
                                                  Under under_scores = Nothing()) {
  const int lane = threadIdx.x & 63, G = lane >> 5;

  // ---- S^T = K Q^T ------------------------------------------------------------
  // All key operands are asked for before the first product, and all value operands behind
  // them, before the exponentials: where they come from LDS, a read takes a hundred cycles
  // and more to arrive, and read two at a time between the products, as the compiler
  // orders them on its own, every pair's latency stood in the chain.
  f32x16 s;
#pragma unroll
  for (int r = 0; r < 16; ++r) s[r] = 0.f;
  bf16x8 k_ops[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) k_ops[c] = key_op(c);
  bf16x8 v_ops[2][NDT];
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int t = 0; t < NDT; ++t) v_ops[u][t] = value_op(u, t);
  __builtin_amdgcn_sched_barrier(0);          // (the reads stay in front of the products)
#pragma unroll
  for (int c = 0; c < NC; ++c) s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k_ops[c], q_op[c].v, s, 0, 0, 0);
  __builtin_amdgcn_sched_barrier(0);
  under_scores();
  __builtin_amdgcn_sched_barrier(0);

  // ---- mask, running maximum and sum ------------------------------------------
  // all_visible (the same for the whole wave): every key of the tile is visible to every
  // slot in use, so the comparisons are left out.  (A slot that is not in use then holds
  // numbers without meaning; they stay in its own lanes and are never stored.)
  // (the scale, which is positive, is applied to the maximum here and to each score
  // inside its exponential below: one multiplication fewer per score)
  float tile_max = -INFINITY;
  if (all_visible) {
#pragma unroll
    for (int r = 0; r < 16; ++r) tile_max = fmaxf(tile_max, s[r]);
  } else {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int key = k0 + 8 * (r >> 2) + 4 * G + (r & 3);
      const bool visible = key <= pos && key >= lo;
      s[r] = visible ? s[r] : -INFINITY;
      tile_max = fmaxf(tile_max, s[r]);
    }
  }
  tile_max *= scale_log2;          // (of this lane's half of the slot's keys)
  // st.m is the reference that the exponentials are taken against, not always the exact
  // maximum: it moves (and the sums are rescaled) only when some slot's scores rise more
  // than SLACK above it, for every slot of the wave at once.  Below that the terms are at
  // most 2^SLACK, which float32 sums and bfloat16 factors hold as well as terms below 1;
  // the quotient o / l does not depend on the reference.  After the first tiles a
  // maximum seldom moves that far, so the rescaling of O is rare, and only then do the
  // two lanes of a slot have to agree on the maximum.
  constexpr float SLACK = 8.0f;
  if (__builtin_amdgcn_ballot_w64(tile_max > st.m + SLACK) != 0) {
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, 64));
    const float m_new = fmaxf(st.m, tile_max);
    // 2^x by the hardware instruction alone: its arguments here are <= 0, and a result
    // too small for a normal number may become zero
    const float alpha = m_new == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f(st.m - m_new);   // st.m == -inf gives 0
    st.l *= alpha;
    st.m = m_new;
#pragma unroll
    for (int t = 0; t < NDT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) st.o[t][r] *= alpha;
  }
  const float m_use = st.m == -INFINITY ? 0.f : st.m;
  float psum = 0.f;
  Op p[2];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const float e = __builtin_amdgcn_exp2f(fmaf(s[r], scale_log2, -m_use));
    psum += e;
    p[r >> 3].e[r & 7] = float_to_bf16(e);
  }
  st.l += psum;          // this lane's half of the slot's keys: the halves meet in finish_sum

  // ---- O^T += V^T P^T ----------------------------------------------------------
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int t = 0; t < NDT; ++t)
      st.o[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v_ops[u][t], p[u].v, st.o[t], 0, 0, 0);
}

__device__ __forceinline__ void compute_tile(Tile& st, const Op* q_op, const TileOps& ops, int k0, int pos, int lo,
                                             float scale_log2, bool all_visible) {
  compute_tile_with(st, q_op, [&](int c) { return ops.k[c].v; }, [&](int u, int t) { return ops.v[u][t].v; }, k0, pos, lo,
                    scale_log2, all_visible);
}

// The tiles first, first + step, ... < end of one sequence.  AHEAD: each tile's loads
// are issued while the tile before it is computed (two tiles' operands in registers:
// for kernels that run one wave per SIMD anyway); otherwise tile by tile.
// all_first..all_last: the keys that every slot in use sees (a tile inside this range
// needs no mask).  STREAMED: nobody else reads these keys in this launch (a decode step: one
// workgroup per sequence, KV head and stretch of keys), so they are loaded as a stream.
template <bool AHEAD, bool STREAMED>
__device__ __forceinline__ void attend_tiles(Tile& st, const Op* q_op, const bf16_t* __restrict__ cache,
                                             const CacheLayout& lay, const int* __restrict__ bt, int bt_stride,
                                             const LaneOffsets& off, int first, int end, int step, int kv_first, int kv_last,
                                             int pos, int lo, float scale_log2, int all_first, int all_last) {
  if (first >= end) return;
  PageWindow pages;
  pages.base = -1;
  if constexpr (AHEAD) {
    TileOps cur, nxt;
    load_tile<STREAMED>(cur, cache, lay, off, bt, bt_stride, pages, first * 32, kv_first, kv_last);
    for (int t = first; t < end; t += step) {
      const int tn = t + step;
      if (tn < end) load_tile<STREAMED>(nxt, cache, lay, off, bt, bt_stride, pages, tn * 32, kv_first, kv_last);
      compute_tile(st, q_op, cur, t * 32, pos, lo, scale_log2, t * 32 >= all_first && t * 32 + 31 <= all_last);
      cur = nxt;
    }
  } else {
    for (int t = first; t < end; t += step) {
      TileOps cur;
      load_tile<STREAMED>(cur, cache, lay, off, bt, bt_stride, pages, t * 32, kv_first, kv_last);
      compute_tile(st, q_op, cur, t * 32, pos, lo, scale_log2, t * 32 >= all_first && t * 32 + 31 <= all_last);
    }
  }
}

__device__ __forceinline__ void load_query(Op* q_op, const bf16_t* __restrict__ qrow, bool ok) {
  const int G = (threadIdx.x & 63) >> 5;
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    q_op[c].u = u32x4{0u, 0u, 0u, 0u};
    if (ok) q_op[c].u = *reinterpret_cast<const u32x4*>(qrow + c * 16 + G * 8);
  }
}

// The sum of a slot's terms: each of its two lanes has added up its own half of the keys.
__device__ __forceinline__ float finish_sum(const Tile& st) { return st.l + __shfl_xor(st.l, 32, 64); }

__device__ __forceinline__ void init_tile(Tile& st) {
  st.m = -INFINITY;
  st.l = 0.f;
#pragma unroll
  for (int t = 0; t < NDT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) st.o[t][r] = 0.f;
}

// ------------------------------------------------------------------- prefill ---
// work: per workgroup 4 ints: first row of the tile in the batch, number of rows
// in the tile (<= 32), position of the first row, block-table row (segment).
__global__ __launch_bounds__(64) void prefill_kernel(bf16_t* __restrict__ out, int64_t ld_out,
                                                     const bf16_t* __restrict__ q, int64_t ldq,
                                                     const bf16_t* __restrict__ cache, CacheLayout lay,
                                                     const int* __restrict__ work, int num_tiles,
                                                     const int* __restrict__ block_tables, int bt_stride,
                                                     int num_heads, float scale_log2, int window) {
  const int lane = threadIdx.x & 63, r32 = lane & 31, G = lane >> 5;
  // Workgroups go to the eight XCDs in turn, and each XCD has an L2 of its own.  Every
  // XCD gets a contiguous run of the work, ordered by KV head first: the keys and values
  // of a head are then read through one L2 (with eight KV heads, one head per XCD).
  // Within a head the later row tiles, which see more keys, come first.
  int tile, h;
  {
    const int total = num_tiles * num_heads, per_xcd = (total + 7) / 8;
    const int u = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (u >= total) return;
    const int group = num_heads / lay.kv_heads, per_kv = num_tiles * group;
    const int kv = u / per_kv, rest = u - kv * per_kv;
    tile = num_tiles - 1 - rest / group;
    h = kv * group + rest % group;
  }
  const int* wk = work + 4 * tile;
  const int row0 = wk[0], rows = wk[1], pos0 = wk[2], seg = wk[3];
  const int kvh = h / (num_heads / lay.kv_heads);
  const int* bt = block_tables + (int64_t)seg * bt_stride;

  const bool slot_ok = r32 < rows;
  const int pos = slot_ok ? pos0 + r32 : -1;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  Op q_op[NC];
  load_query(q_op, q + (int64_t)(row0 + (slot_ok ? r32 : 0)) * ldq + h * HD, slot_ok);

  Tile st;
  init_tile(st);
  const int kv_last = pos0 + rows - 1;
  const int kv_first = window > 0 ? max(0, pos0 - window + 1) : 0;
  // every row in use sees the keys from the last row's window start to the first row's position
  attend_tiles<false, false>(st, q_op, cache, lay, bt, bt_stride, lane_offsets(lay, kvh), kv_first >> 5, (kv_last >> 5) + 1, 1, kv_first, kv_last, pos, lo,
               scale_log2, window > 0 ? max(0, kv_last - window + 1) : 0, pos0);

  const float l_slot = finish_sum(st);
  if (slot_ok) {
    const float inv = 1.0f / l_slot;
    bf16_t* orow = out + (int64_t)(row0 + r32) * ld_out + h * HD;
#pragma unroll
    for (int t = 0; t < NDT; ++t)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int d = 32 * t + 8 * b + 4 * G;
        if (d < HD) {
          bf16_t v4[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) v4[i] = float_to_bf16(st.o[t][4 * b + i] * inv);
          *reinterpret_cast<u32x2*>(orow + d) = *reinterpret_cast<const u32x2*>(v4);
        }
      }
  }
}

// --------------------------------------------- prefill, key tiles shared in LDS ---
// The heads that share a KV head read the same keys and values.  A workgroup takes a
// tile of 32 rows for up to four such heads, one wave a head, and brings every key
// tile into LDS once: each lane asks for exactly the 16 bytes that it would have loaded
// as its own operand, but straight into LDS (lane l of a 1 KB block), and every wave
// then reads its operands from there, a block being one operand of the whole wave,
// contiguous.  Two tiles of LDS: the next tile's loads are in flight while this one is
// multiplied, without a register for them.  Lanes whose key or value does not exist
// read a place that does (masked keys count for nothing; the cache never holds anything
// but finite numbers, so a masked value times zero is zero).
constexpr int KV_BLOCKS = NC + 2 * NDT;           // 1 KB blocks of one key tile: keys, then values
constexpr int SHARED_WAVES = 4;
// key tiles of LDS where loads are waited for by count: four (three of them on their way) where
// two workgroups of four tiles fit a CU's 160 KB (head sizes up to 128: 16 KB a tile), else three
// (prefill attention of the 8B shape, 2,048 tokens: 67.6 us a layer with three, 65.0 with four)
constexpr int SHARED_TILES = HD <= 128 ? 4 : 3;
static_assert(SHARED_TILES == 3 || SHARED_TILES == 4, "the waits are written for three or four tiles");

__device__ __forceinline__ void request_tile(char* __restrict__ tile_lds, const bf16_t* __restrict__ cache,
                                             const CacheLayout& lay, const LaneOffsets& off,
                                             const int* __restrict__ bt, int bt_stride, PageWindow& pages, int k0,
                                             int kv_first, int kv_last, int wave, int waves) {
  typedef __attribute__((address_space(3))) void* lds_ptr;
  typedef const __attribute__((address_space(1))) void* global_ptr;
  const int r32 = threadIdx.x & 31;
  {
    const int b0 = k0 >> lay.page_shift, b1 = (k0 + 31) >> lay.page_shift;
    if (pages.base < 0 || b0 < pages.base || b1 >= pages.base + 64) pages.fill(bt, bt_stride, b0);
  }
  // Keys outside kv_first..kv_last read page 0.  A key's slot in its page is
  // (k0 + r32) % page_size = k0 % page_size + r32 % page_size: k0 is a multiple of 32.
  const int key = k0 + r32;
  const bool key_ok = key <= kv_last && key >= kv_first;
  const int key_page = pages.of(key >> lay.page_shift);
  const bf16_t* krow = cache + (key_ok ? key_page * lay.page_stride : 0) + off.key +
                       (int64_t)(k0 & (lay.page_size - 1)) * 16;
  const int64_t chunk_stride = lay.key_chunk_stride();
  const bf16_t* vbase[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int kb = k0 + 16 * u;
    const bool ok = kb <= kv_last && kb + 15 >= kv_first;
    const int page = pages.of(kb >> lay.page_shift);
    vbase[u] = cache + (ok ? page * lay.page_stride + (kb & (lay.page_size - 1)) : 0);
  }
  // the blocks are dealt to the waves in turn (the test is uniform over a wave)
  int turn = 0;
#pragma unroll
  for (int b = 0; b < KV_BLOCKS; ++b) {
    if (turn == wave) {
      const bf16_t* src = b < NC ? krow + b * chunk_stride : vbase[(b - NC) / NDT] + off.value[(b - NC) % NDT];
      __builtin_amdgcn_global_load_lds((global_ptr)src, (lds_ptr)(tile_lds + b * 1024), 16, 0, 0);
    }
    turn = turn + 1 == waves ? 0 : turn + 1;
  }
}

// The same request when the number of waves is known at compile time: which blocks a
// wave brings, and from where in a page each of its lanes reads them, never changes, so
// it is worked out once (WaveBlocks).  A tile of 32 keys lies in at most two pages (of its
// first and of its last 16 keys); their numbers come out of the page window as scalars,
// and a request is a choice between two bases, an addition and the load: no branch, no
// shuffle, no multiplication per lane.
template <int WAVES>
struct WaveBlocks {
  static constexpr int J = (KV_BLOCKS + WAVES - 1) / WAVES;
  int count;                 // blocks of this wave
  uint32_t lane_off[J];      // this lane's bytes from the start of a page
  bool second[J];            // this lane reads the page of the tile's last 16 keys
  int kind[J];               // 0 keys, 1 values of the first 16 keys, 2 values of the last 16 keys
};

template <int WAVES>
__device__ __forceinline__ WaveBlocks<WAVES> wave_blocks(const CacheLayout& lay, int kvh, int wave) {
  const int lane = threadIdx.x & 63, r32 = lane & 31, G = lane >> 5;
  WaveBlocks<WAVES> w;
  w.count = 0;
#pragma unroll
  for (int j = 0; j < WaveBlocks<WAVES>::J; ++j) {
    const int b = min(wave + WAVES * j, KV_BLOCKS - 1);
    if (wave + WAVES * j < KV_BLOCKS) w.count = j + 1;
    if (b < NC) {
      w.kind[j] = 0;
      w.second[j] = r32 >= 16;
      w.lane_off[j] = (uint32_t)(lay.key_offset(0, kvh, r32 & (lay.page_size - 1), b * 16 + G * 8) * 2);
    } else {
      const int u = (b - NC) / NDT, t = (b - NC) % NDT;
      w.kind[j] = 1 + u;
      w.second[j] = u != 0;
      // rows beyond the head repeat its last one
      w.lane_off[j] = (uint32_t)((lay.value_column(0, kvh, min(32 * t + r32, HD - 1)) + 8 * G) * 2);
    }
  }
  return w;
}

// BUFFER: the loads are buffer loads over the whole cache layer (which must be smaller than
// 4 GB: a lane's place is 32 bits from the layer's start).  The compiler does not connect
// them with the reads of the LDS that follow, as it does the global loads into LDS, before
// which it waits for every load in flight: the caller waits by count (and must).
template <int WAVES, bool BUFFER>
__device__ __forceinline__ void request_wave_blocks(char* __restrict__ tile_lds, const bf16_t* __restrict__ cache,
                                                    __amdgpu_buffer_rsrc_t rsrc, const CacheLayout& lay,
                                                    const WaveBlocks<WAVES>& w, const int* __restrict__ bt, int bt_stride,
                                                    PageWindow& pages, int k0, int kv_first, int kv_last, int wave) {
  typedef __attribute__((address_space(3))) void* lds_ptr;
  typedef const __attribute__((address_space(1))) void* global_ptr;
  const int block_a = k0 >> lay.page_shift, block_b = (k0 + 16) >> lay.page_shift;
  if (pages.base < 0 || block_a < pages.base || block_b >= pages.base + 64) {
    pages.fill(bt, bt_stride, block_a);
    // (every 64 pages.  The window is waited for here, where it is loaded: a load that may or may
    // not be on its way when the loop comes round makes the compiler wait for every load in flight,
    // the tiles to come among them, in front of each use of the window, in every step)
    if constexpr (BUFFER) __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
  }
  if constexpr (BUFFER && NC % WAVES == 0) {
    // A wave issues an instruction every four to five cycles, and what is computed per request
    // stands in every step's chain.  With the key chunks a whole number of rounds of the waves, a
    // wave's first NC / WAVES blocks are keys and the rest values, whichever wave it is: a key
    // block's lanes choose between the two pages once for all key blocks, and everything that is
    // the same for all lanes goes into the load's scalar offset; a value block lies in one page,
    // so its lanes' offsets never change at all.  (The layer is smaller than 4 GB here.)
    // (No look at kv_first..kv_last: a block table holds page 0 where a sequence has no page, or
    // no longer has one, and whatever a page holds is finite; keys out of range are masked.)
    const uint32_t page_bytes = (uint32_t)lay.page_stride * 2u;
    const uint32_t a32 = (uint32_t)__builtin_amdgcn_readlane(pages.page, __builtin_amdgcn_readfirstlane(block_a - pages.base)) * page_bytes;
    const uint32_t b32 = (uint32_t)__builtin_amdgcn_readlane(pages.page, __builtin_amdgcn_readfirstlane(block_b - pages.base)) * page_bytes;
    const uint32_t in_a = (uint32_t)(k0 & (lay.page_size - 1)), in_b = (uint32_t)((k0 + 16) & (lay.page_size - 1));
    const uint32_t s_key = in_a * 16u * 2u, s_va = a32 + in_a * 2u, s_vb = b32 + in_b * 2u;     // (a slot of a key chunk: 16 dims)
    const uint32_t lane_page = w.second[0] ? b32 : a32;            // (block 0 of a wave is a key block)
#pragma unroll
    for (int j = 0; j < WaveBlocks<WAVES>::J; ++j) {
      lds_ptr dst = (lds_ptr)(tile_lds + (wave + WAVES * j) * 1024);
      if (j < NC / WAVES) __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, dst, 16, lane_page + w.lane_off[j], s_key, 0, 0);
      else __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, dst, 16, w.lane_off[j], w.kind[j] == 2 ? s_vb : s_va, 0, 0);
    }
    return;
  }
  // pages outside kv_first..kv_last may have been given back: page 0 is read instead
  const bool ok_a = k0 <= kv_last && k0 + 15 >= kv_first, ok_b = k0 + 16 <= kv_last && k0 + 31 >= kv_first;
  const int page_a = ok_a ? __builtin_amdgcn_readlane(pages.page, __builtin_amdgcn_readfirstlane(block_a - pages.base)) : 0;
  const int page_b = ok_b ? __builtin_amdgcn_readlane(pages.page, __builtin_amdgcn_readfirstlane(block_b - pages.base)) : 0;
  // (the two pages' byte offsets as scalars that the compiler takes as given: it would
  // otherwise choose between the page numbers per lane and multiply in every lane)
  const uint64_t bytes_a = (uint64_t)page_a * (uint64_t)lay.page_stride * 2, bytes_b = (uint64_t)page_b * (uint64_t)lay.page_stride * 2;
  const uint32_t a_lo = __builtin_amdgcn_readfirstlane((uint32_t)bytes_a), a_hi = __builtin_amdgcn_readfirstlane((uint32_t)(bytes_a >> 32));
  const uint32_t b_lo = __builtin_amdgcn_readfirstlane((uint32_t)bytes_b), b_hi = __builtin_amdgcn_readfirstlane((uint32_t)(bytes_b >> 32));
  const int in_page = k0 & (lay.page_size - 1);
  // what the tile's place in its page adds: rows of keys, slots of values
  const uint32_t add[3] = {(uint32_t)(in_page * 16 * 2), (uint32_t)(in_page * 2),
                           (uint32_t)(((k0 + 16) & (lay.page_size - 1)) * 2)};
#pragma unroll
  for (int j = 0; j < WaveBlocks<WAVES>::J; ++j) {
    if (KV_BLOCKS % WAVES == 0 || j < w.count) {
      const uint32_t in_layer = w.lane_off[j] + (w.kind[j] == 0 ? add[0] : w.kind[j] == 1 ? add[1] : add[2]);
      if constexpr (BUFFER) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_ptr)(tile_lds + (wave + WAVES * j) * 1024), 16,
                                                 (w.second[j] ? b_lo : a_lo) + in_layer, 0, 0, 0);
      } else {
        const uint64_t page_bytes = ((uint64_t)(w.second[j] ? b_hi : a_hi) << 32) | (w.second[j] ? b_lo : a_lo);
        const char* src = (const char*)cache + page_bytes + in_layer;
        __builtin_amdgcn_global_load_lds((global_ptr)src, (lds_ptr)(tile_lds + (wave + WAVES * j) * 1024), 16, 0, 0);
      }
    }
  }
}

// The same as a static member of a class template: nothing is deduced at the call.  (The host
// pass of the compiler takes the call of the function template in the first specialization of
// the kernel below that makes it and reports no match in the second.)
template <int WAVES, bool BUFFER>
struct RequestBlocks {
  static __device__ __forceinline__ void go(char* __restrict__ tile_lds, const bf16_t* __restrict__ cache,
                                            __amdgpu_buffer_rsrc_t rsrc, const CacheLayout& lay, const WaveBlocks<WAVES>& w,
                                            const int* __restrict__ bt, int bt_stride, PageWindow& pages, int k0, int kv_first,
                                            int kv_last, int wave) {
    request_wave_blocks<WAVES, BUFFER>(tile_lds, cache, rsrc, lay, w, bt, bt_stride, pages, k0, kv_first, kv_last, wave);
  }
};

// work: per row tile 4 ints (first row, rows <= 32, first position, block-table row).
// WAVES: the waves of a workgroup if they are SHARED_WAVES, 0 for any other number.
// RING: key tiles come through buffer loads (layer_bytes < 4 GB) into a ring of SHARED_TILES
// tiles of LDS and are waited for by count (WAVES must divide a tile's blocks).
// (At most 256 registers a lane, so that two workgroups share a CU and take turns at the
// matrix pipe; without the second number the compiler took 262 with the accumulators in the
// other half of the register file, one workgroup a CU and a hundred moves between the halves
// a step.  History of this kernel at the 8B shape, 2,048 tokens, us a layer: 85 with one tile
// ahead behind a fence; 81.5 with the ring; 71.5 within 256 registers; 67.6 with a tile's
// sixteen operand reads in front of its products; 65.0 with four tiles.)
// IDLERS: some waves of a workgroup may have nothing to multiply at a key tile (a wave without a
// head, or a row tile of earlier rows) and skip it.  Where the heads of a KV head fill the waves
// the kernel holds no trace of that: the check in every step's chain, and what the compiler made
// of the loop around it, cost 16 to 20 % at four heads to a KV head (69 -> 81 us a layer at
// 2,048 tokens, 275 -> 330 at 8,192, 1,093 -> 1,267 at 32,768).
template <int WAVES, bool RING, bool IDLERS = true>
__global__ __launch_bounds__(SHARED_WAVES * 64, 2) void prefill_shared_kernel(
    bf16_t* __restrict__ out, int64_t ld_out, const bf16_t* __restrict__ q, int64_t ldq,
    const bf16_t* __restrict__ cache, uint32_t layer_bytes, CacheLayout lay, const int* __restrict__ work, int num_tiles,
    const int* __restrict__ runs, int num_runs,
    const int* __restrict__ block_tables, int bt_stride, int num_heads, float scale_log2, int window) {
  extern __shared__ __attribute__((aligned(1024))) char kv_lds[];     // two tiles of KV_BLOCKS KB
  const int lane = threadIdx.x & 63, r32 = lane & 31, G = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), waves = blockDim.x >> 6;
  const int group = num_heads / lay.kv_heads, chunks = (group + waves - 1) / waves;
  // What the waves of a workgroup share a key tile for: the heads of a KV head over one row
  // tile, or (runs: heads that share no keys with another) up to four row tiles of one head
  // that follow one another in a sequence, run (first tile, count): the keys of the last of
  // them are the keys of all, and a wave leaves out the tiles beyond its own rows.
  const bool by_rows = runs != nullptr;
  // Workgroups go to the eight XCDs in turn; every XCD gets a contiguous run of the work,
  // ordered by KV head first (its keys then live in one L2), later row tiles first.
  int tile, last_tile, kvh, chunk;
  {
    const int per_kv = by_rows ? num_runs : num_tiles * chunks, total = per_kv * lay.kv_heads, per_xcd = (total + 7) / 8;
    const int u = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (u >= total) return;
    kvh = u / per_kv;
    const int rest = u - kvh * per_kv;
    if (by_rows) {
      const int* run = runs + 2 * (num_runs - 1 - rest);
      tile = run[0];
      last_tile = tile + run[1] - 1;
      chunk = 0;
    } else {
      tile = last_tile = num_tiles - 1 - rest / chunks;
      chunk = rest % chunks;
    }
  }
  // the keys that the workgroup walks: from the first tile's first key to the last tile's last
  const int wg_pos0 = work[4 * tile + 2], wg_last = work[4 * last_tile + 2] + work[4 * last_tile + 1] - 1;
  const bool head_ok = by_rows ? tile + wave <= last_tile : chunk * waves + wave < group;      // a wave without work still loads its share
  const int* wk = work + 4 * (by_rows && head_ok ? tile + wave : tile);
  const int row0 = wk[0], rows = wk[1], pos0 = wk[2], seg = wk[3];
  const int* bt = block_tables + (int64_t)seg * bt_stride;
  const int h = by_rows ? kvh : kvh * group + (head_ok ? chunk * waves + wave : 0);

  const bool slot_ok = r32 < rows && head_ok;
  const int pos = slot_ok ? pos0 + r32 : -1;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  Op q_op[NC];
  load_query(q_op, q + (int64_t)(row0 + (slot_ok ? r32 : 0)) * ldq + h * HD, slot_ok);

  Tile st;
  init_tile(st);
  const int kv_last = wg_last;
  const int kv_first = window > 0 ? max(0, wg_pos0 - window + 1) : 0;
  const int t_first = kv_first >> 5, t_end = (kv_last >> 5) + 1;
  const int my_last = pos0 + rows - 1;                                    // this wave's last key
  const int all_first = window > 0 ? max(0, my_last - window + 1) : 0;   // every row in use sees all_first .. pos0
  PageWindow pages;
  pages.base = -1;
  constexpr int TILE_BYTES = KV_BLOCKS * 1024;
  const LaneOffsets off = lane_offsets(lay, kvh);
  const WaveBlocks<WAVES == 0 ? 1 : WAVES> mine = wave_blocks<WAVES == 0 ? 1 : WAVES>(lay, kvh, wave);
  // (a raw buffer of 32-bit data over the layer; only the ring's loads go through it)
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)cache, 0, (int)layer_bytes, 0x00020000);
  // (a wave without work, or of earlier rows, sees nothing of the tiles from t_mine on)
  const int t_mine = !IDLERS ? INT_MAX : head_ok ? (my_last >> 5) + 1 : INT_MIN;
  auto compute = [&](auto checked, int t, const char* tile_at, auto under_scores) {
    if constexpr (IDLERS && decltype(checked)::value) {
      if (t >= t_mine) {
        under_scores();
        return;
      }
    }
    const char* cur = tile_at + lane * 16;
    compute_tile_with(
        st, q_op, [&](int c) { return *reinterpret_cast<const bf16x8*>(cur + c * 1024); },
        [&](int u, int tt) { return *reinterpret_cast<const bf16x8*>(cur + (NC + u * NDT + tt) * 1024); }, t * 32, pos, lo,
        scale_log2, t * 32 >= all_first && t * 32 + 31 <= pos0, under_scores);
  };
  if constexpr (RING) {
    // Every wave brings the same number of blocks of a tile, so a wave can wait for its loads by
    // count: SHARED_TILES tiles of LDS, all but one of them on their way.  The keys come from the
    // L2, whose latency is as long as a tile takes to multiply.  (With global loads into LDS the
    // compiler puts a wait for every load in flight in front of the first read of LDS that
    // follows them, so that every step waited for the tile it had just asked for.)
    static_assert(WAVES != 0 && KV_BLOCKS % (WAVES == 0 ? 1 : WAVES) == 0, "a wave's loads of a tile must be a fixed number");
    constexpr int W = WAVES == 0 ? 1 : WAVES, MINE = KV_BLOCKS / W;     // loads a wave issues for a tile
    auto request = [&](int t) {
      RequestBlocks<W, true>::go(kv_lds + ((t - t_first) % SHARED_TILES) * TILE_BYTES, cache, rsrc, lay, mine, bt, bt_stride,
                                   pages, t * 32, kv_first, kv_last, wave);
    };
    // Nothing is on its way when the loop begins but what the loop itself asks for: the compiler
    // keeps count of the loads whose registers it knows (the queries'), and one of those in
    // flight across the loop's edge makes it wait, in front of every product, until only the
    // loads of that very step are outstanding, which is one tile ahead again and no more.
    request(t_first);
    if (t_first + 1 < t_end) request(t_first + 1);
    if (SHARED_TILES == 4 && t_first + 2 < t_end) request(t_first + 2);
    __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
    // A wave's tiles first, in a loop that holds no check (in front of every tile's products it
    // cost 16 to 20 %), then the tiles that only its fellows multiply: it still waits, meets the
    // others at the barrier and brings its share of the tiles to come.
    const int t_split = min(t_end, max(t_first, t_mine));
    auto arrive = [&](int t) {
      // this wave's blocks of tile t have landed (those of the tiles after it may still be on their way) ...
      const int behind = min(SHARED_TILES - 2, t_end - 1 - t);          // tiles asked for after tile t
      // (the wait is the compiler's own builtin, not text it cannot read: it then knows that
      // the loads of before the loop, the queries, have arrived, and does not wait for them,
      // and with them for every load behind them, in front of every product)
      // (and this wave's own LDS reads of tile t - 1 have returned: the products that consume them
      // stand before this point, but nothing else would make a read that is still on its way
      // come back before another wave's load lands in the place it reads)
      if (behind >= 2) __builtin_amdgcn_s_waitcnt(vmcnt_and_lds_reads(2 * MINE));
      else if (behind == 1) __builtin_amdgcn_s_waitcnt(vmcnt_and_lds_reads(MINE));
      else __builtin_amdgcn_s_waitcnt(vmcnt_and_lds_reads(0));
      // ... and after the barrier everybody's have, and nobody reads tile t - 1 any more, whose
      // place the next request takes.  (No fence: it would wait for every load in flight.)
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
    };
    for (int t = t_first; t < t_split; ++t) {
      arrive(t);
      // (the request behind the tile's score products: asked for right after the barrier, the
      // sixteen loads of a workgroup's four waves meet at the CU's one path into LDS, and a wave
      // stands four hundred cycles at its four loads before it reads its first operand)
      compute(std::false_type{}, t, kv_lds + ((t - t_first) % SHARED_TILES) * TILE_BYTES, [&]() {
        if (t + SHARED_TILES - 1 < t_end) request(t + SHARED_TILES - 1);
      });
    }
    if constexpr (IDLERS) {
      for (int t = t_split; t < t_end; ++t) {
        arrive(t);
        if (t + SHARED_TILES - 1 < t_end) request(t + SHARED_TILES - 1);
      }
    }
  } else {
    auto request = [&](int t) {
      char* dst = kv_lds + ((t - t_first) & 1) * TILE_BYTES;
      if constexpr (WAVES != 0)
        request_wave_blocks<WAVES, false>(dst, cache, rsrc, lay, mine, bt, bt_stride, pages, t * 32,
                                          kv_first, kv_last, wave);
      else request_tile(dst, cache, lay, off, bt, bt_stride, pages, t * 32, kv_first, kv_last, wave, waves);
    };
    request(t_first);
    __syncthreads();               // waits for the loads too
    for (int t = t_first; t < t_end; ++t) {
      if (t + 1 < t_end) request(t + 1);
      compute(std::true_type{}, t, kv_lds + ((t - t_first) & 1) * TILE_BYTES, Nothing());
      __syncthreads();             // the next tile has landed; nobody reads this one any more
    }
  }

  const float l_slot = finish_sum(st);
  if (slot_ok) {
    const float inv = 1.0f / l_slot;
    bf16_t* orow = out + (int64_t)(row0 + r32) * ld_out + h * HD;
#pragma unroll
    for (int t = 0; t < NDT; ++t)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int d = 32 * t + 8 * b + 4 * G;
        if (d < HD) {
          bf16_t v4[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) v4[i] = float_to_bf16(st.o[t][4 * b + i] * inv);
          *reinterpret_cast<u32x2*>(orow + d) = *reinterpret_cast<const u32x2*>(v4);
        }
      }
  }
}

// ------------------------------ prefill, a row tile's keys in two halves ---
// At a few thousand tokens the launch above is as long as its longest workgroup: the last
// row tile of a 2,048-token prompt walks 64 key tiles one after the other while most of the
// chip has long finished (half of the time of the kernel is the tail).  Here a workgroup
// has eight waves: four heads of a KV head over the first half of the row tile's key tiles,
// and the same four heads over the second half, each half with its own ring of tiles in
// LDS, both walking in step (one barrier a step for all eight).  At the end the second
// half's state goes through the LDS to the first half's waves, which join the two (the
// reference of the exponentials is per half; the quotient does not depend on it) and store.
// One workgroup a CU, two waves a SIMD as before; the longest chain is half as long.
// For four heads (or a multiple) to a KV head, head sizes up to 128 (two rings of four
// tiles fit the LDS), a layer that 32 bits address.
constexpr bool HALVES_FIT = KV_BLOCKS % SHARED_WAVES == 0 && 2 * 4 * KV_BLOCKS <= 160;
constexpr int HALVES_TILES = 4;
constexpr int JOIN_FLOATS = NDT * 16 + 2;          // a lane's share of a wave's state: O, reference, sum

__global__ __launch_bounds__(2 * SHARED_WAVES * 64, 1) void prefill_halves_kernel(
    bf16_t* __restrict__ out, int64_t ld_out, const bf16_t* __restrict__ q, int64_t ldq,
    const bf16_t* __restrict__ cache, uint32_t layer_bytes, CacheLayout lay, const int* __restrict__ work, int num_tiles,
    const int* __restrict__ block_tables, int bt_stride, int num_heads, float scale_log2, int window) {
  extern __shared__ __attribute__((aligned(1024))) char kv_lds[];     // two rings of HALVES_TILES tiles
  if constexpr (HALVES_FIT) {
    constexpr int W = SHARED_WAVES, MINE = KV_BLOCKS / W, TILE_BYTES = KV_BLOCKS * 1024, RING_BYTES = HALVES_TILES * TILE_BYTES;
    const int lane = threadIdx.x & 63, r32 = lane & 31, G = lane >> 5;
    const int wave8 = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wave = wave8 & (W - 1), half = wave8 >> 2;
    const int group = num_heads / lay.kv_heads, chunks = group / W;
    int tile, kvh, chunk;
    {
      const int per_kv = num_tiles * chunks, total = per_kv * lay.kv_heads, per_xcd = (total + 7) / 8;
      const int u = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
      if (u >= total) return;
      kvh = u / per_kv;
      const int rest = u - kvh * per_kv;
      tile = num_tiles - 1 - rest / chunks;
      chunk = rest % chunks;
    }
    const int* wk = work + 4 * tile;
    const int row0 = wk[0], rows = wk[1], pos0 = wk[2], seg = wk[3];
    const int* bt = block_tables + (int64_t)seg * bt_stride;
    const int h = kvh * group + chunk * W + wave;
    const bool slot_ok = r32 < rows;
    const int pos = slot_ok ? pos0 + r32 : -1;
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    Op q_op[NC];
    load_query(q_op, q + (int64_t)(row0 + (slot_ok ? r32 : 0)) * ldq + h * HD, slot_ok);

    Tile st;
    init_tile(st);
    const int kv_last = pos0 + rows - 1;
    const int kv_first = window > 0 ? max(0, pos0 - window + 1) : 0;
    const int t_first = kv_first >> 5, t_end = (kv_last >> 5) + 1;
    // the first half takes the odd tile: it is the one that joins and stores at the end
    const int t_mid = t_first + (t_end - t_first + 1) / 2;
    const int my_first = half == 0 ? t_first : t_mid, my_end = half == 0 ? t_mid : t_end;
    const int common = t_end - t_mid;                       // steps that both halves take
    const int all_first = window > 0 ? max(0, kv_last - window + 1) : 0;
    PageWindow pages;
    pages.base = -1;
    const WaveBlocks<W> mine = wave_blocks<W>(lay, kvh, wave);
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)cache, 0, (int)layer_bytes, 0x00020000);
    char* ring = kv_lds + half * RING_BYTES;
    auto request = [&](int t) {
      RequestBlocks<W, true>::go(ring + ((t - my_first) % HALVES_TILES) * TILE_BYTES, cache, rsrc, lay, mine, bt, bt_stride,
                                   pages, t * 32, kv_first, kv_last, wave);
    };
    // (as in the kernel above: nothing but the ring's own loads is on its way inside the loop)
    if (my_first < my_end) request(my_first);
    if (my_first + 1 < my_end) request(my_first + 1);
    if (my_first + 2 < my_end) request(my_first + 2);
    __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
    auto arrive = [&](int t) {
      const int behind = min(HALVES_TILES - 2, my_end - 1 - t);
      if (behind >= 2) __builtin_amdgcn_s_waitcnt(vmcnt_and_lds_reads(2 * MINE));
      else if (behind == 1) __builtin_amdgcn_s_waitcnt(vmcnt_and_lds_reads(MINE));
      else __builtin_amdgcn_s_waitcnt(vmcnt_and_lds_reads(0));
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
    };
    auto step = [&](int t) {
      arrive(t);
      const char* cur = ring + ((t - my_first) % HALVES_TILES) * TILE_BYTES + lane * 16;
      compute_tile_with(
          st, q_op, [&](int c) { return *reinterpret_cast<const bf16x8*>(cur + c * 1024); },
          [&](int u, int tt) { return *reinterpret_cast<const bf16x8*>(cur + (NC + u * NDT + tt) * 1024); }, t * 32, pos, lo,
          scale_log2, t * 32 >= all_first && t * 32 + 31 <= pos0, [&]() {
            if (t + HALVES_TILES - 1 < my_end) request(t + HALVES_TILES - 1);
          });
    };
    for (int i = 0; i < common; ++i) step(my_first + i);
    if (t_mid - t_first > common) {                         // (the same for the whole workgroup)
      if (half == 0) {
        step(my_first + common);
      } else {
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
      }
    }

    // ---- the second half's state to the first half's waves, through the LDS (every ring is done with)
    __syncthreads();
    float* mine_at = reinterpret_cast<float*>(kv_lds) + (size_t)wave * JOIN_FLOATS * 64 + lane;
    if (half == 1) {
#pragma unroll
      for (int t = 0; t < NDT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) mine_at[(t * 16 + r) * 64] = st.o[t][r];
      mine_at[(NDT * 16) * 64] = st.m;
      mine_at[(NDT * 16 + 1) * 64] = st.l;
    }
    __syncthreads();
    if (half == 1) return;
    {
      const float m1 = mine_at[(NDT * 16) * 64], l1 = mine_at[(NDT * 16 + 1) * 64];
      const float m_new = fmaxf(st.m, m1);
      const float m_use = m_new == -INFINITY ? 0.f : m_new;
      // (a half without keys has a reference of minus infinity, a sum and an output of zero: its factor is zero)
      const float f0 = st.m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(st.m - m_use);
      const float f1 = m1 == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m1 - m_use);
      st.l = st.l * f0 + l1 * f1;
#pragma unroll
      for (int t = 0; t < NDT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) st.o[t][r] = st.o[t][r] * f0 + mine_at[(t * 16 + r) * 64] * f1;
    }
    const float l_slot = finish_sum(st);
    if (slot_ok) {
      const float inv = 1.0f / l_slot;
      bf16_t* orow = out + (int64_t)(row0 + r32) * ld_out + h * HD;
#pragma unroll
      for (int t = 0; t < NDT; ++t)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          const int d = 32 * t + 8 * b + 4 * G;
          if (d < HD) {
            bf16_t v4[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) v4[i] = float_to_bf16(st.o[t][4 * b + i] * inv);
            *reinterpret_cast<u32x2*>(orow + d) = *reinterpret_cast<const u32x2*>(v4);
          }
        }
    }
  }
}

// Joins the splits of one (segment, head) in ascending split order: lane s holds the
// weight of split s, every lane then walks the splits for its own dims.  One wave.
// COHERENT: the partial results were written by other workgroups of this launch, so
// they are read at device scope.
template <bool COHERENT>
__device__ __forceinline__ float read_partial(const float* p) {
  if constexpr (COHERENT) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else return *p;
}

// (The splits' outputs are asked for eight splits at a time, the first eight together with
// the maxima and sums: a join of up to eight splits costs one latency, not one a split.)
template <bool COHERENT>
__device__ __forceinline__ void combine_head(bf16_t* __restrict__ orow, const float* __restrict__ pr, int num_splits) {
  constexpr int NJ = (HD + 63) / 64, TOGETHER = 8;
  const int lane = threadIdx.x & 63;
  float m = -INFINITY, l = 0.f;
  float o[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) o[j] = 0.f;
  auto fetch = [&](float (&part)[TOGETHER][NJ], int first, int last) {     // splits first .. first+7, none beyond `last`
#pragma unroll
    for (int u = 0; u < TOGETHER; ++u) {
      const float* src = pr + (int64_t)min(first + u, last) * (HD + 2);
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int d = lane + 64 * j;                      // (no load under a condition: they all go out together)
        const float v = read_partial<COHERENT>(src + min(d, HD - 1));
        part[u][j] = d < HD ? v : 0.f;
      }
    }
  };
  for (int s0 = 0; s0 < num_splits; s0 += 64) {          // 64 splits at a time
    const int mine = s0 + lane;
    const int count = min(64, num_splits - s0);
    float part[TOGETHER][NJ];
    fetch(part, s0, s0 + count - 1);
    const float ms = mine < num_splits ? read_partial<COHERENT>(pr + (int64_t)mine * (HD + 2) + HD) : -INFINITY;
    const float ls = mine < num_splits ? read_partial<COHERENT>(pr + (int64_t)mine * (HD + 2) + HD + 1) : 0.f;
    const float m_new = fmaxf(m, wave_max(ms));
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float rescale = exp2f(m - m_use);
    const float f = exp2f(ms - m_use);                    // this lane's split weight
    l = l * rescale + wave_sum(ls * f);
#pragma unroll
    for (int j = 0; j < NJ; ++j) o[j] *= rescale;
    for (int c0 = 0; c0 < count; c0 += TOGETHER) {
      if (c0 > 0) fetch(part, s0 + c0, s0 + count - 1);
#pragma unroll
      for (int u = 0; u < TOGETHER; ++u) {
        const float fs = __shfl(f, min(c0 + u, 63), 64);
        if (c0 + u < count) {                             // in the order of the splits
#pragma unroll
          for (int j = 0; j < NJ; ++j) o[j] += part[u][j] * fs;
        }
      }
    }
    m = m_new;
  }
  const float inv = 1.0f / l;
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const int d = lane + 64 * j;
    if (d < HD) orow[d] = float_to_bf16(o[j] * inv);
  }
}

// -------------------------------------------------------------------- decode ---
// One workgroup of up to four waves per (decode segment, KV head, split).  The slots
// are the heads of the group, 32 at a time.  The workgroup's key tiles are dealt to its
// waves in turn; their running states meet in LDS and are joined in wave order.  With
// one split the result is final; otherwise it goes to `partial` as HD + 2 floats per
// (segment, head, split): the unnormalised output, the maximum, the sum.
constexpr int DECODE_MAX_WAVES = 4;      // each wave holds two tiles' operands: registers allow no more

template <bool AHEAD>
__global__ __launch_bounds__(DECODE_MAX_WAVES * 64, AHEAD ? 1 : 2) void decode_kernel(
    bf16_t* __restrict__ out, int64_t ld_out, const bf16_t* __restrict__ q, int64_t ldq,
    const bf16_t* __restrict__ cache, CacheLayout lay, const int* __restrict__ seg_rows,
    const int* __restrict__ seg_positions, const int* __restrict__ seg_tables,
    const int* __restrict__ block_tables, int bt_stride, int num_heads, float scale_log2, int window,
    float* __restrict__ partial, int num_splits, int* __restrict__ counters) {
  extern __shared__ float lds[];   // [waves][slots][HD + 2]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r32 = lane & 31, G = lane >> 5;
  const int waves = blockDim.x >> 6;
  const int sidx = blockIdx.x, kvh = blockIdx.y, split = blockIdx.z;
  const int group = num_heads / lay.kv_heads;
  const int slots = min(group, 32);
  // (without seg_rows and seg_tables, segment i is row i with block table i: the block table's
  // address then waits for no load, and the chain to the first key is one latency shorter)
  const int row = seg_rows != nullptr ? seg_rows[sidx] : sidx, pos = seg_positions[sidx];
  const int* bt = block_tables + (int64_t)(seg_tables != nullptr ? seg_tables[sidx] : sidx) * bt_stride;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;

  // key tiles of this split: a contiguous share of the tiles lo/32 .. pos/32
  const int tile_first = lo >> 5, tile_count = (pos >> 5) - tile_first + 1;
  const int per = (tile_count + num_splits - 1) / num_splits;
  const int t_begin = tile_first + split * per;
  const int t_end = min(tile_first + tile_count, t_begin + per);

  const LaneOffsets off = lane_offsets(lay, kvh);
  for (int g0 = 0; g0 < group; g0 += 32) {
    const bool slot_ok = g0 + r32 < group;
    const int h = kvh * group + g0 + (slot_ok ? r32 : 0);
    Op q_op[NC];
    load_query(q_op, q + (int64_t)row * ldq + h * HD, slot_ok);
    Tile st;
    init_tile(st);
    // (keys and values as a stream: every load instruction covers whole lines, and nobody else
    // reads them in this launch: 5.5 -> 6.3 TB/s where the cache is larger than the memory-side cache)
    attend_tiles<AHEAD, true>(st, q_op, cache, lay, bt, bt_stride, off, t_begin + wave, t_end, waves, lo, pos, slot_ok ? pos : -1, lo,
                 scale_log2, lo, pos);

    // this wave's state into LDS
    const float l_slot = finish_sum(st);
    if (g0 > 0) __syncthreads();
    if (slot_ok) {
      float* mine = lds + (int64_t)(wave * slots + r32) * (HD + 2);
#pragma unroll
      for (int t = 0; t < NDT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int d = 32 * t + 8 * (r >> 2) + 4 * G + (r & 3);
          if (d < HD) mine[d] = st.o[t][r];
        }
      if (G == 0) {
        mine[HD] = st.m;
        mine[HD + 1] = l_slot;
      }
    }
    __syncthreads();

    // join the waves: thread -> (slot, four consecutive dims)
    const int valid = min(32, group - g0);
    for (int idx = threadIdx.x; idx < valid * (HD / 4); idx += blockDim.x) {
      const int sl = idx / (HD / 4), d = 4 * (idx - sl * (HD / 4));
      float m = -INFINITY;
      for (int w = 0; w < waves; ++w) m = fmaxf(m, lds[(int64_t)(w * slots + sl) * (HD + 2) + HD]);
      const float m_use = m == -INFINITY ? 0.f : m;
      float l = 0.f, o[4] = {0.f, 0.f, 0.f, 0.f};
      for (int w = 0; w < waves; ++w) {
        const float* src = lds + (int64_t)(w * slots + sl) * (HD + 2);
        const float f = exp2f(src[HD] - m_use);
        l += src[HD + 1] * f;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] += src[d + i] * f;
      }
      const int head = kvh * group + g0 + sl;
      if (num_splits == 1) {
        const float inv = 1.0f / l;
        bf16_t v4[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v4[i] = float_to_bf16(o[i] * inv);
        *reinterpret_cast<u32x2*>(out + (int64_t)row * ld_out + head * HD + d) = *reinterpret_cast<const u32x2*>(v4);
      } else {
        // stores of device scope: they go through to memory, where the workgroup that
        // joins the splits (on any XCD) reads them
        float* pr = partial + ((int64_t)(sidx * num_heads + head) * num_splits + split) * (HD + 2);
#pragma unroll
        for (int i = 0; i < 4; ++i) __hip_atomic_store(pr + d + i, o[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (d == 0) {
          __hip_atomic_store(pr + HD, m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(pr + HD + 1, l, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
  }

  // The split that finishes last joins the splits of its (segment, KV head), so that no
  // second launch is needed: every workgroup publishes its partial results and counts
  // itself; nobody waits for anybody.  The counter is back at zero afterwards.
  if (num_splits > 1 && counters != nullptr) {
    __shared__ int is_last;
    // The partial results were stored at device scope and are complete when the store
    // counter is zero; the joining workgroup reads them with loads of device scope.  No
    // fence: a release would write the whole L2 back and an acquire would empty it, under
    // the workgroups that still stream keys.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    int* counter = counters + sidx * lay.kv_heads + kvh;
    if (threadIdx.x == 0) is_last = atomicAdd(counter, 1) == num_splits - 1;
    __syncthreads();
    if (is_last) {
      for (int hh = wave; hh < group; hh += waves)
        combine_head<true>(out + (int64_t)row * ld_out + (kvh * group + hh) * HD,
                           partial + (int64_t)(sidx * num_heads + kvh * group + hh) * num_splits * (HD + 2), num_splits);
      if (threadIdx.x == 0) atomicExch(counter, 0);
    }
  }
}

// The same join as a launch of its own (for callers that bring no counters).
__global__ __launch_bounds__(64) void combine_kernel(bf16_t* __restrict__ out, int64_t ld_out,
                                                     const int* __restrict__ seg_rows,
                                                     const float* __restrict__ partial, int num_heads,
                                                     int num_splits) {
  const int sidx = blockIdx.x, h = blockIdx.y;
  combine_head<false>(out + (int64_t)(seg_rows != nullptr ? seg_rows[sidx] : sidx) * ld_out + h * HD,
                      partial + (int64_t)(sidx * num_heads + h) * num_splits * (HD + 2), num_splits);
}

}  // namespace

HFEE_API int hfee_attention_bf16_head_dim() { return HD; }

// Whether this head size has the prefill kernel with a row tile's keys in two halves (variant 3).
HFEE_API int hfee_attention_bf16_halves() { return HALVES_FIT ? 1 : 0; }

// log2 of the bytes of a cache layer from which on the kernels that address the whole layer through one
// 32-bit offset (the ring of key tiles in LDS, the two halves) leave the work to the others.
HFEE_API int hfee_attention_bf16_layer_limit_log2() { return 32; }

// The most row tiles in a run of `runs` (hfee_attention_bf16_prefill): one wave a row tile.
HFEE_API int hfee_attention_bf16_run_tiles() { return SHARED_WAVES; }

static int check_common(const char* name, int64_t ld_out, int64_t ldq, int num_heads, int kv_heads,
                        int page_size, int window, float scale, const void* out, const void* q, CacheLayout* lay) {
  HFEE_REQUIRE(scale > 0.f && scale < INFINITY, "%s: the score scale must be positive, got %g", name, (double)scale);
  HFEE_REQUIRE(num_heads > 0 && kv_heads > 0 && num_heads % kv_heads == 0,
               "%s: %d heads are not a multiple of %d kv heads", name, num_heads, kv_heads);
  HFEE_REQUIRE(num_heads <= 65535, "%s: too many heads", name);
  HFEE_REQUIRE(window >= 0, "%s: negative window", name);
  HFEE_REQUIRE(ldq >= (int64_t)num_heads * HD && ld_out >= (int64_t)num_heads * HD, "%s: q/out row too short", name);
  HFEE_REQUIRE(ldq % 8 == 0 && (uintptr_t)q % 16 == 0, "%s: q rows must be 16-byte aligned", name);
  HFEE_REQUIRE(ld_out % 4 == 0 && (uintptr_t)out % 8 == 0, "%s: out rows must be 8-byte aligned", name);
  return make_cache_layout(lay, kv_heads, HD, page_size);
}

// work: num_tiles x 4 int32 (first row, rows <= 32, first position, block-table row).
// variant: 0 choose, 1 one wave per (tile, head), 2 key tiles shared in LDS by the heads
// of a KV head, 3 the same with a row tile's keys in two halves (for tests of each kernel alone).
HFEE_API int hfee_attention_bf16_prefill(void* out, int64_t ld_out, const void* q, int64_t ldq,
                                         const void* cache, int cache_pages, const int* work, int num_tiles,
                                         const int* runs, int num_runs,
                                         const int* block_tables, int bt_stride, int num_heads, int kv_heads,
                                         int page_size, float scale, int window, int variant, hipStream_t stream) {
  HFEE_REQUIRE(num_tiles >= 0, "attention_bf16_prefill: bad tile count");
  HFEE_REQUIRE(variant >= 0 && variant <= 3, "attention_bf16_prefill: unknown kernel choice %d", variant);
  HFEE_REQUIRE(cache_pages > 0, "attention_bf16_prefill: a cache layer of %d pages", cache_pages);
  if (num_tiles == 0) return 0;
  CacheLayout lay;
  if (check_common("attention_bf16_prefill", ld_out, ldq, num_heads, kv_heads, page_size, window, scale, out, q, &lay))
    return 1;
  HFEE_REQUIRE((int64_t)num_tiles * num_heads < (1ll << 30), "attention_bf16_prefill: too much work for one launch");
  const int group = num_heads / kv_heads;
  HFEE_REQUIRE(runs == nullptr || num_runs > 0, "attention_bf16_prefill: runs of row tiles without their number");
  const int64_t layer_bytes = (int64_t)cache_pages * lay.page_stride * 2;
  // heads that share no keys with another: the row tiles of a head that follow one another
  // share them instead, four at a time, where the caller has listed such runs
  const bool by_rows = group == 1 && runs != nullptr && variant != 1 && KV_BLOCKS % SHARED_WAVES == 0 &&
                       layer_bytes < (1ll << 32);
  // a row tile's keys in two halves, eight waves a workgroup: four heads (or a multiple) to a KV
  // head; the caller asks for it where the longest row tile of the step is much longer than the
  // chip's share of the whole step (it knows the positions)
  const bool halves_fit = HALVES_FIT && !by_rows && group % SHARED_WAVES == 0 && layer_bytes < (1ll << 32);
  HFEE_REQUIRE(variant != 3 || halves_fit, "attention_bf16_prefill: the kernel with a row tile's keys in two halves takes "
               "four heads or a multiple to a KV head, head sizes up to 128 and a layer below 4 GB");
  if (variant == 3) {
    constexpr size_t lds = (size_t)2 * HALVES_TILES * KV_BLOCKS * 1024;
    static bool raised_halves = false;
    if (!raised_halves) {
      hipError_t e = hipFuncSetAttribute((const void*)prefill_halves_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      HFEE_REQUIRE(e == hipSuccess, "attention_bf16_prefill: cannot raise the LDS limit: %s", hipGetErrorString(e));
      raised_halves = true;
    }
    dim3 grid((unsigned)(((int64_t)num_tiles * (group / SHARED_WAVES) * kv_heads + 7) / 8 * 8));
    prefill_halves_kernel<<<grid, 2 * SHARED_WAVES * 64, lds, stream>>>(
        (bf16_t*)out, ld_out, (const bf16_t*)q, ldq, (const bf16_t*)cache, (uint32_t)layer_bytes, lay, work, num_tiles,
        block_tables, bt_stride, num_heads, scale * LOG2E, window);
  } else if (!by_rows && (variant == 1 || (variant == 0 && group == 1))) {      // nothing to share: one wave per (tile, head)
    dim3 grid((unsigned)(((int64_t)num_tiles * num_heads + 7) / 8 * 8));
    prefill_kernel<<<grid, 64, 0, stream>>>((bf16_t*)out, ld_out, (const bf16_t*)q, ldq, (const bf16_t*)cache, lay,
                                            work, num_tiles, block_tables, bt_stride, num_heads, scale * LOG2E, window);
  } else {
    const bool can_ring = KV_BLOCKS % SHARED_WAVES == 0 && layer_bytes < (1ll << 32);
    // (two or three heads to a KV head: four waves all the same, of which the others only bring
    // their shares of the tiles, so that the ring applies: 16 heads over 8 KV heads 92 -> 69 µs
    // at 2,048 tokens, 24 heads 96 -> 76)
    const int waves = by_rows || (can_ring && group >= 2) ? SHARED_WAVES : group < SHARED_WAVES ? group : SHARED_WAVES;
    const int chunks = (group + waves - 1) / waves;
    // the ring of tiles with loads waited for by count: four waves that bring equal shares of a
    // tile, and a layer that 32 bits address
    const bool ring = waves == SHARED_WAVES && KV_BLOCKS % SHARED_WAVES == 0 && layer_bytes < (1ll << 32);
    const size_t lds = (size_t)(ring ? SHARED_TILES : 2) * KV_BLOCKS * 1024;
    static bool raised = false;
    if (!raised) {
      const int most = SHARED_TILES * KV_BLOCKS * 1024;
      hipError_t e = hipFuncSetAttribute((const void*)prefill_shared_kernel<0, false>,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, most);
      if (e == hipSuccess)
        e = hipFuncSetAttribute((const void*)prefill_shared_kernel<SHARED_WAVES, false>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, most);
      if (e == hipSuccess && KV_BLOCKS % SHARED_WAVES == 0)
        e = hipFuncSetAttribute((const void*)prefill_shared_kernel<SHARED_WAVES, KV_BLOCKS % SHARED_WAVES == 0>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, most);
      if (e == hipSuccess && KV_BLOCKS % SHARED_WAVES == 0)
        e = hipFuncSetAttribute((const void*)prefill_shared_kernel<SHARED_WAVES, KV_BLOCKS % SHARED_WAVES == 0, false>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, most);
      HFEE_REQUIRE(e == hipSuccess, "attention_bf16_prefill: cannot raise the LDS limit: %s", hipGetErrorString(e));
      raised = true;
    }
    dim3 grid((unsigned)(((int64_t)(by_rows ? num_runs : num_tiles * chunks) * kv_heads + 7) / 8 * 8));
    const int* runs_or_none = by_rows ? runs : nullptr;
    // (every wave has a head at every key tile: the heads of a KV head are whole rounds of the waves)
    const bool all_busy = !by_rows && group % waves == 0;
#define GO(W, R, ...)                                                                                               \
  prefill_shared_kernel<W, R, ##__VA_ARGS__><<<grid, waves * 64, lds, stream>>>((bf16_t*)out, ld_out, (const bf16_t*)q, ldq, \
                                                                (const bf16_t*)cache, (uint32_t)(ring ? layer_bytes : 0),  \
                                                                lay, work, num_tiles, runs_or_none, num_runs, block_tables, \
                                                                bt_stride, num_heads, scale * LOG2E, window)
    if (ring && all_busy) GO(SHARED_WAVES, (KV_BLOCKS % SHARED_WAVES == 0), false);
    else if (ring) GO(SHARED_WAVES, (KV_BLOCKS % SHARED_WAVES == 0));
    else if (waves == SHARED_WAVES) GO(SHARED_WAVES, false);
    else GO(0, false);
#undef GO
  }
  HFEE_CHECK_LAUNCH("attention_bf16_prefill");
  return 0;
}

// seg_rows / seg_positions / seg_tables: per decode segment its row in the batch,
// its position and its block-table row (seg_rows or seg_tables null: segment i is row i,
// has block table i).  partial: at least
// num_segments * num_heads * num_splits * (head_dim + 2) floats when num_splits > 1.
// counters: null, or at least num_segments * kv_heads int32 that are zero (and are zero
// again when the kernel has run): the splits are then joined by the workgroup that
// finishes last instead of by a second launch.
HFEE_API int hfee_attention_bf16_decode(void* out, int64_t ld_out, const void* q, int64_t ldq, const void* cache,
                                        const int* seg_rows, const int* seg_positions, const int* seg_tables,
                                        int num_segments, const int* block_tables, int bt_stride,
                                        int num_heads, int kv_heads, int page_size, float scale, int window,
                                        float* partial, int64_t partial_floats, int num_splits, int waves,
                                        int* counters, int num_counters, hipStream_t stream) {
  HFEE_REQUIRE(num_segments >= 0, "attention_bf16_decode: bad segment count");
  if (num_segments == 0) return 0;
  HFEE_REQUIRE(seg_positions != nullptr, "attention_bf16_decode: the segments' positions are missing");
  CacheLayout lay;
  if (check_common("attention_bf16_decode", ld_out, ldq, num_heads, kv_heads, page_size, window, scale, out, q, &lay))
    return 1;
  HFEE_REQUIRE(num_splits >= 1 && num_splits <= 65535, "attention_bf16_decode: bad split count %d", num_splits);
  HFEE_REQUIRE(kv_heads <= 65535, "attention_bf16_decode: too many kv heads");
  if (num_splits > 1) {
    const int64_t need = (int64_t)num_segments * num_heads * num_splits * (HD + 2);
    HFEE_REQUIRE(partial != nullptr && partial_floats >= need,
                 "attention_bf16_decode: the partial buffer holds %lld floats, %lld needed",
                 (long long)partial_floats, (long long)need);
  }
  dim3 grid(num_segments, kv_heads, num_splits);
  const bool in_kernel_join = counters != nullptr && num_counters >= num_segments * kv_heads;
  const int group = num_heads / kv_heads;
  const size_t per_wave = (size_t)(group < 32 ? group : 32) * (HD + 2) * sizeof(float);
  HFEE_REQUIRE(waves >= 1 && waves <= DECODE_MAX_WAVES, "attention_bf16_decode: 1..%d waves, got %d",
               DECODE_MAX_WAVES, waves);
  while (waves > 1 && waves * per_wave > 60 * 1024) waves /= 2;     // the waves' states must fit in LDS
  const size_t lds = waves * per_wave;
  static bool raised = false;
  if (lds > 48 * 1024 && !raised) {
    const int most = (int)(DECODE_MAX_WAVES * 32 * (HD + 2) * sizeof(float) < 160 * 1024
                               ? DECODE_MAX_WAVES * 32 * (HD + 2) * sizeof(float) : 160 * 1024);
    hipError_t e = hipFuncSetAttribute((const void*)decode_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, most);
    if (e == hipSuccess)
      e = hipFuncSetAttribute((const void*)decode_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, most);
    HFEE_REQUIRE(e == hipSuccess, "attention_bf16_decode: cannot raise the LDS limit: %s", hipGetErrorString(e));
    raised = true;
  }
  // With more workgroups than CUs, the form that holds one tile's operands (two workgroups
  // fit a CU and hide each other's loads); else the form that asks for the next tile while it
  // multiplies this one (one workgroup a CU, and nobody else to hide its loads).
  static int num_cus = 0;
  if (num_cus == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    num_cus = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess &&
               prop.multiProcessorCount > 0) ? prop.multiProcessorCount : 256;
  }
  const bool ahead = (int64_t)num_segments * kv_heads * num_splits <= num_cus;
  if (ahead)
    decode_kernel<true><<<grid, waves * 64, lds, stream>>>(
        (bf16_t*)out, ld_out, (const bf16_t*)q, ldq, (const bf16_t*)cache, lay, seg_rows, seg_positions, seg_tables,
        block_tables, bt_stride, num_heads, scale * LOG2E, window, partial, num_splits, in_kernel_join ? counters : nullptr);
  else
    decode_kernel<false><<<grid, waves * 64, lds, stream>>>(
        (bf16_t*)out, ld_out, (const bf16_t*)q, ldq, (const bf16_t*)cache, lay, seg_rows, seg_positions, seg_tables,
        block_tables, bt_stride, num_heads, scale * LOG2E, window, partial, num_splits, in_kernel_join ? counters : nullptr);
  HFEE_CHECK_LAUNCH("attention_bf16_decode");
  if (num_splits > 1 && !in_kernel_join) {
    dim3 cgrid(num_segments, num_heads);
    combine_kernel<<<cgrid, 64, 0, stream>>>((bf16_t*)out, ld_out, seg_rows, partial, num_heads, num_splits);
    HFEE_CHECK_LAUNCH("attention_bf16_decode(combine)");
  }
  return 0;
}
