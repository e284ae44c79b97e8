// Picking the next token on the device: greedy, or temperature sampling with
// repeat penalty, top-k, top-p and min-p.
//
// The rules and their order are the reference's
// (/root/reference/internal/llm/sampler.go:54-130): repeat penalty on each distinct
// recent id (logit > 0: divide, else multiply); temperature <= 0: the first maximum;
// else the top_k largest logits, prob = exp((logit - max) / temperature) normalised,
// top_p keeps the shortest prefix (in descending order) whose cumulative probability
// reaches it, min_p cuts what falls below min_p * prob[0], and the draw is
// proportional to what is kept.
//
// Nothing is sorted.  A prefix of the descending order is the set {key > t} plus the
// first r ties at t (ties taken in ascending id), so each rule becomes a search for
// its threshold: a radix select on counts for top_k, a bit-by-bit bisection on
// probability mass for top_p.  All sums run in a fixed order (thread-owned contiguous
// chunks, then a fixed tree), so a row's result is the same in every batch.
//
// A row of a large vocabulary goes through sample_slices_kernel first, 32 workgroups a row
// (penalty, maximum, and each slice's own top_k for a small top_k); sample_kernel then
// works on what the slices left.  Smaller vocabularies: sample_kernel alone.
//
// The random number is counter based: splitmix64 of (seed, draw index), one stream
// per request, independent of what else is sampled in the same call.
#include "common.h"
#include "no_alloc_entry.h"

#include <atomic>

using namespace hfee;

namespace {

constexpr int THREADS = 1024;

struct SampleParams {          // one per row; 12 x 4 bytes, filled by the host
  float temperature;
  int top_k;
  float top_p;
  float min_p;
  float repeat_penalty;
  int history_offset;          // into the flat history array
  int history_length;          // ids to penalise (already cut to repeat_last_n)
  uint32_t seed_lo, seed_hi;
  uint32_t draw_lo, draw_hi;   // index of this draw in the request's stream
  int logits_row;
};

__device__ __forceinline__ uint32_t order_key(float v) {   // larger float <=> larger key
  const uint32_t b = __float_as_uint(v);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

__device__ __forceinline__ double uniform_from(uint64_t seed, uint64_t draw) {
  uint64_t z = seed + (draw + 1) * 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  z ^= z >> 31;
  return (double)(z >> 11) * (1.0 / 9007199254740992.0);
}

// Exclusive prefix sums over the block in thread order; *total gets the sum.
template <typename T>
__device__ __forceinline__ T block_exclusive_scan(T v, T* wave_totals, T* total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  T incl = v;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const T up = __shfl_up(incl, off, 64);
    if (lane >= off) incl += up;
  }
  __syncthreads();
  if (lane == 63) wave_totals[wave] = incl;
  __syncthreads();
  T before = 0, all = 0;
  for (int w = 0; w < THREADS / 64; ++w) {
    const T wt = wave_totals[w];
    if (w < wave) before += wt;
    all += wt;
  }
  *total = all;
  return before + incl - v;
}

struct MaxIdx {
  float v;
  int i;
};

__device__ __forceinline__ MaxIdx better(MaxIdx a, MaxIdx b) {   // greater value, then smaller id
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}

// The sum of a wave's 64 values, the same in every lane's return value: four steps inside
// the rows of 16 lanes and two across them, all in the data path of the vector unit (a
// shuffle goes through the LDS crossbar and takes ten times as long; the bisection for
// top_p waits for 32 such sums in turn).  A fixed tree: the same sum for the same values.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_add(float v) {
  return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xf, false));
}
__device__ __forceinline__ float wave_total(float v) {
  v = dpp_add<0xB1, 0xf>(v);          // quad_perm [1, 0, 3, 2]
  v = dpp_add<0x4E, 0xf>(v);          // quad_perm [2, 3, 0, 1]
  v = dpp_add<0x141, 0xf>(v);         // row_half_mirror
  v = dpp_add<0x140, 0xf>(v);         // row_mirror: every lane has its row's sum
  v = dpp_add<0x142, 0xa>(v);         // row_bcast 15: rows 1 and 3 add the row before
  v = dpp_add<0x143, 0xc>(v);         // row_bcast 31: rows 2 and 3 add rows 0 + 1
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int dpp_add(int v) {
  return v + __builtin_amdgcn_update_dpp(0, v, CTRL, ROW_MASK, 0xf, false);
}
__device__ __forceinline__ int wave_total(int v) {
  v = dpp_add<0xB1, 0xf>(v);
  v = dpp_add<0x4E, 0xf>(v);
  v = dpp_add<0x141, 0xf>(v);
  v = dpp_add<0x140, 0xf>(v);
  v = dpp_add<0x142, 0xa>(v);
  v = dpp_add<0x143, 0xc>(v);
  return __builtin_amdgcn_readlane(v, 63);
}


// One pass of the block over lg[0 .. V-1]: see(j, lg[j]) for every j, ascending within a
// thread.  Rows that are 16-byte aligned are read four logits a load, four loads in flight;
// others one logit a load, eight in flight.
template <typename F>
__device__ __forceinline__ void scan_logits(const float* __restrict__ lg, int V, F see) {
  const int stride = blockDim.x;
  if (((uintptr_t)lg & 15) == 0) {
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    const f32x4* lg4 = reinterpret_cast<const f32x4*>(lg);
    const int quads = V >> 2;
    int i = threadIdx.x;
    for (; i + 3 * stride < quads; i += 4 * stride) {
      f32x4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = lg4[i + u * stride];
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int c = 0; c < 4; ++c) see(4 * (i + u * stride) + c, v[u][c]);
    }
    for (; i < quads; i += stride) {
      const f32x4 v = lg4[i];
#pragma unroll
      for (int c = 0; c < 4; ++c) see(4 * i + c, v[c]);
    }
    for (int j = 4 * quads + threadIdx.x; j < V; j += stride) see(j, lg[j]);
  } else {
    int j = threadIdx.x;
    for (; j + 7 * stride < V; j += 8 * stride) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = lg[j + u * stride];
#pragma unroll
      for (int u = 0; u < 8; ++u) see(j + u * stride, v[u]);
    }
    for (; j < V; j += stride) see(j, lg[j]);
  }
}

__device__ MaxIdx block_argmax_raw(const float* __restrict__ lg, int V, MaxIdx* scratch) {
  MaxIdx best{-INFINITY, 0x7fffffff};
  // (ascending j per thread: strict '>' keeps the first)
  scan_logits(lg, V, [&](int j, float v) { if (v > best.v) best = MaxIdx{v, j}; });
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    MaxIdx o{__shfl_xor(best.v, off, 64), __shfl_xor(best.i, off, 64)};
    best = better(best, o);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) scratch[wave] = best;
  __syncthreads();
  MaxIdx r = scratch[0];
  for (int w = 1; w < (int)(blockDim.x + 63) / 64; ++w) r = better(r, scratch[w]);
  return r;                         // id 0x7fffffff: every logit is NaN or -inf
}

__device__ MaxIdx block_argmax(const float* __restrict__ lg, int V, MaxIdx* scratch) {
  MaxIdx r = block_argmax_raw(lg, V, scratch);
  if (r.i == 0x7fffffff) r.i = 0;
  return r;
}

__global__ __launch_bounds__(THREADS) void argmax_kernel(int* __restrict__ out, const float* __restrict__ logits,
                                                         int64_t ld, int V) {
  __shared__ MaxIdx scratch[16];
  const MaxIdx r = block_argmax(logits + (int64_t)blockIdx.x * ld, V, scratch);
  if (threadIdx.x == 0) out[blockIdx.x] = r.i;
}

// A row over `parts` workgroups, so that a few rows still use the whole chip: each
// leaves the first maximum of its stretch in `partial`, counts itself, and the one that
// arrives last takes the best of them (greater value, then smaller id: the same id whatever
// the order of arrival) and sets the counter back to zero.
constexpr int ARGMAX_THREADS = 256;

__global__ __launch_bounds__(ARGMAX_THREADS) void argmax_parts_kernel(int* __restrict__ out,
                                                                      const float* __restrict__ logits, int64_t ld,
                                                                      int V, int parts, MaxIdx* __restrict__ partial,
                                                                      int* __restrict__ counters) {
  __shared__ MaxIdx scratch[16];
  __shared__ int last;
  const int row = blockIdx.x / parts, part = blockIdx.x - row * parts;
  const int stretch = (V + parts - 1) / parts;
  const int j0 = min(V, part * stretch), j1 = min(V, j0 + stretch);
  MaxIdx r = block_argmax_raw(logits + (int64_t)row * ld + j0, j1 - j0, scratch);
  if (threadIdx.x == 0) {
    if (r.i != 0x7fffffff) r.i += j0;
    MaxIdx* mine = partial + (int64_t)row * parts + part;
    __hip_atomic_store(&mine->v, r.v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&mine->i, r.i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    last = __hip_atomic_fetch_add(counters + row, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT) == parts - 1;
  }
  __syncthreads();
  if (!last) return;
  MaxIdx best{-INFINITY, 0x7fffffff};
  for (int p = threadIdx.x; p < parts; p += ARGMAX_THREADS) {
    const MaxIdx* theirs = partial + (int64_t)row * parts + p;
    MaxIdx o{__hip_atomic_load(&theirs->v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT),
             __hip_atomic_load(&theirs->i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)};
    best = better(best, o);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    MaxIdx o{__shfl_xor(best.v, off, 64), __shfl_xor(best.i, off, 64)};
    best = better(best, o);
  }
  __syncthreads();                                   // (block_argmax_raw's use of scratch is over)
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = best;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < ARGMAX_THREADS / 64; ++w) best = better(best, scratch[w]);
    out[row] = best.i == 0x7fffffff ? 0 : best.i;
    __hip_atomic_store(counters + row, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// The rules after top_k run either over the whole block (1,024 threads, sums joined through
// LDS with barriers) or, when top_k has gathered its few entries into LDS, over one wave
// (64 lanes, sums joined by shuffles, no barrier at all).
template <typename T, bool WAVE>
__device__ __forceinline__ T team_exclusive_scan(T v, T* wave_totals, T* total) {
  if constexpr (!WAVE) {
    return block_exclusive_scan<T>(v, wave_totals, total);
  } else {
    const int lane = threadIdx.x & 63;
    T incl = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const T up = __shfl_up(incl, off, 64);
      if (lane >= off) incl += up;
    }
    *total = __shfl(incl, 63, 64);
    return incl - v;
  }
}

// The team's sum alone (no prefix).
template <bool WAVE>
__device__ __forceinline__ float team_total(float v, float* scratch) {
  if constexpr (WAVE) {
    return wave_total(v);
  } else {
    float total;
    block_exclusive_scan<float>(v, scratch, &total);
    return total;
  }
}

template <bool WAVE>
__device__ __forceinline__ float team_max(float v, float* scratch) {
  if constexpr (WAVE) return wave_max(v);
  else return block_max(v, scratch);
}

// Everything after top_k (sampler.go:88-129) over entries 0 .. Vn-1 with logits lgp and ids
// `ids` (null: entry j is id j), of which {key > t_k} and the first r_k ties at t_k belong:
// probabilities into qp, top_p, min_p, the draw.  Every member of the team owns a contiguous
// chunk of the entries; sums run chunk by chunk and then in a fixed tree.
template <bool WAVE>
__device__ __forceinline__ void draw_from_kept(const SampleParams& p, const MaxIdx top, int Vn,
                                               const float* lgp, float* qp, const int* ids, uint32_t t_k, int r_k,
                                               int* out_id, float* fscratch, int* iscratch, int* sh_choice) {
  constexpr int TEAM = WAVE ? 64 : THREADS;
  const int me = WAVE ? (threadIdx.x & 63) : threadIdx.x;
  auto id_of = [&](int j) { return ids != nullptr ? ids[j] : j; };
  const int chunk = (Vn + TEAM - 1) / TEAM;
  const int j0 = min(Vn, me * chunk), j1 = min(Vn, j0 + chunk);
  int my_ties = 0;
  for (int j = j0; j < j1; ++j) my_ties += order_key(lgp[j]) == t_k;
  int all_ties;
  int tie_rank = team_exclusive_scan<int, WAVE>(my_ties, iscratch, &all_ties);
  float my_mass = 0.f;
  for (int j = j0; j < j1; ++j) {
    const float v = lgp[j];
    const uint32_t key = order_key(v);
    bool in = key > t_k;
    if (key == t_k) in = tie_rank++ < r_k;
    const float e = in ? expf((v - top.v) / p.temperature) : 0.f;
    qp[j] = e;
    my_mass += e;
  }
  if (!WAVE) __threadfence_block();
  const float Z = team_total<WAVE>(my_mass, fscratch);

  // ---- top_p: threshold key and how many of its ties belong (sampler.go:98-108)
  uint32_t t_p = 0u;
  int r_p = 0x7fffffff;
  if (p.top_p > 0.f && p.top_p < 1.f) {
    const float target = p.top_p * Z;
    uint32_t t = 0u;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t cand = t | (1u << bit);
      float mass = 0.f;
      for (int j = j0; j < j1; ++j) mass += order_key(lgp[j]) >= cand ? qp[j] : 0.f;
      if (team_total<WAVE>(mass, fscratch) >= target) t = cand;
    }
    t_p = t;
    float above = 0.f, tie_p = 0.f;
    for (int j = j0; j < j1; ++j) {
      const uint32_t key = order_key(lgp[j]);
      if (key > t_p) above += qp[j];
      else if (key == t_p && qp[j] > 0.f) tie_p = qp[j];
    }
    const float mass_above = team_total<WAVE>(above, fscratch);
    tie_p = team_max<WAVE>(tie_p, fscratch);
    r_p = tie_p > 0.f ? max(1, (int)ceilf((target - mass_above) / tie_p)) : 1;
  }

  // ---- min_p and the kept set (sampler.go:109-116), then the draw (sampler.go:118-129)
  int my_pties = 0;
  for (int j = j0; j < j1; ++j) my_pties += (order_key(lgp[j]) == t_p && qp[j] > 0.f);
  int all_pties;
  int ptie_rank = team_exclusive_scan<int, WAVE>(my_pties, iscratch, &all_pties);
  float my_keep = 0.f;
  int my_last = -1;
  for (int j = j0; j < j1; ++j) {
    const uint32_t key = order_key(lgp[j]);
    float w = qp[j];
    if (w > 0.f) {
      bool in = key > t_p;
      if (key == t_p) in = ptie_rank++ < r_p;
      if (p.min_p > 0.f && w < p.min_p && id_of(j) != top.i) in = false;
      if (!in) w = 0.f;
    }
    qp[j] = w;
    if (w > 0.f) my_last = id_of(j);
    my_keep += w;
  }
  if (!WAVE) __threadfence_block();
  float total;
  const float before = team_exclusive_scan<float, WAVE>(my_keep, fscratch, &total);
  const uint64_t seed = ((uint64_t)p.seed_hi << 32) | p.seed_lo;
  const uint64_t draw = ((uint64_t)p.draw_hi << 32) | p.draw_lo;
  const float r = (float)(uniform_from(seed, draw) * (double)total);

  // every chunk that starts below r walks; the smallest id whose running sum reaches r
  // wins, whatever rounding does to the chunk sums
  int mine = 0x7fffffff;
  if (my_keep > 0.f && (before < r || r <= 0.f)) {
    float run = before;
    for (int j = j0; j < j1; ++j) {
      if (qp[j] <= 0.f) continue;
      run += qp[j];
      if (run >= r) { mine = id_of(j); break; }
    }
  }
  if constexpr (WAVE) {
    int choice = mine, last = my_last;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      choice = min(choice, __shfl_xor(choice, off, 64));
      last = max(last, __shfl_xor(last, off, 64));
    }
    // rounding left r above every running sum: the last kept id (sampler.go:129)
    if (choice == 0x7fffffff) choice = last < 0 ? top.i : last;
    if (me == 0) *out_id = choice;
  } else {
    if (me == 0) *sh_choice = 0x7fffffff;
    __syncthreads();
    if (mine != 0x7fffffff) atomicMin(sh_choice, mine);
    __syncthreads();
    if (*sh_choice == 0x7fffffff) {
      int last = my_last;
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) last = max(last, __shfl_xor(last, off, 64));
      if ((me & 63) == 0) iscratch[me >> 6] = last;
      __syncthreads();
      if (me == 0) {
        int l = -1;
        for (int w = 0; w < THREADS / 64; ++w) l = max(l, iscratch[w]);
        *sh_choice = l < 0 ? top.i : l;
      }
      __syncthreads();
    }
    if (me == 0) *out_id = *sh_choice;
  }
}

// ---- a row spread over workgroups ------------------------------------------------------
// With a top_k of at most SLICE_K (the default is 40) a row of a large vocabulary is cut into
// SLICES slices, a workgroup each: the slice comes into LDS once, gets its share of the
// repeat penalty, and leaves its maximum and its own top_k (value desc, id asc: the order in
// which the whole row's top_k is taken, so the row's top_k lies within the slices' top_ks)
// in the row's scratch.  The row's workgroup (sample_kernel) then selects among at most
// SLICES x top_k candidates instead of reading the vocabulary seven times.  Rows that are
// greedy, or whose top_k is off or larger, get the penalty and the maxima here and the rest
// in sample_kernel as before.
constexpr int SLICES = 32, SLICE_K = 64, SLICE_THREADS = 256, SPAN_MAX = 8192;
constexpr int SLICE_HEAD = 128;                                   // words: SLICES maxima (value, id), SLICES counts
constexpr int SLICE_WORDS = SLICE_HEAD + SLICES * 2 * SLICE_K;    // of a row's scratch
constexpr int SLICED_MIN_V = 8192;

__device__ __forceinline__ MaxIdx* slice_tops(float* q) { return reinterpret_cast<MaxIdx*>(q); }
__device__ __forceinline__ int* slice_counts(float* q) { return reinterpret_cast<int*>(q) + 2 * SLICES; }
__device__ __forceinline__ float* slice_vals(float* q, int s) { return q + SLICE_HEAD + s * 2 * SLICE_K; }
__device__ __forceinline__ int* slice_ids(float* q, int s) {
  return reinterpret_cast<int*>(q) + SLICE_HEAD + s * 2 * SLICE_K + SLICE_K;
}
__device__ __forceinline__ bool sliced_top_k(const SampleParams& p) {
  return p.temperature > 0.f && p.top_k > 0 && p.top_k <= SLICE_K;
}

template <int KPT>       // keys a thread: the slice has at most KPT * SLICE_THREADS ids
__global__ __launch_bounds__(SLICE_THREADS) void sample_slices_kernel(float* __restrict__ logits, int64_t ld, int V,
                                                                      int span, const SampleParams* __restrict__ params,
                                                                      const int* __restrict__ history, const int* latest,
                                                                      float* __restrict__ scratch, int64_t ld_scratch) {
  constexpr int WAVES_HERE = SLICE_THREADS / 64;
  __shared__ __align__(16) float vals[SPAN_MAX];
  __shared__ uint32_t seen[SPAN_MAX / 32];
  __shared__ MaxIdx mscratch[WAVES_HERE];
  __shared__ int counts[2][WAVES_HERE];
  __shared__ int wave_above[WAVES_HERE], wave_ties[WAVES_HERE];
  const int s = blockIdx.x, row = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const SampleParams p = params[row];
  float* lg = logits + (int64_t)p.logits_row * ld;
  float* q = scratch + (int64_t)row * ld_scratch;
  const int lo = min(V, s * span), n = min(V, lo + span) - lo;

  if ((((uintptr_t)(lg + lo)) & 15) == 0) {
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    const f32x4* src = reinterpret_cast<const f32x4*>(lg + lo);
    for (int i = tid; i < (n >> 2); i += SLICE_THREADS) *reinterpret_cast<f32x4*>(&vals[4 * i]) = src[i];
    for (int j = (n & ~3) + tid; j < n; j += SLICE_THREADS) vals[j] = lg[lo + j];
  } else {
    for (int j = tid; j < n; j += SLICE_THREADS) vals[j] = lg[lo + j];
  }
  for (int w = tid; w < (n + 31) / 32; w += SLICE_THREADS) seen[w] = 0u;
  __syncthreads();

  // ---- repeat penalty on the ids of this slice (see sample_kernel)
  if (p.repeat_penalty != 1.0f && (p.history_length > 0 || latest != nullptr)) {
    const int count = p.history_length + (latest != nullptr ? 1 : 0);
    for (int i = tid; i < count; i += SLICE_THREADS) {
      const int id = i < p.history_length ? history[p.history_offset + i] : latest[row];
      if (id >= lo && id < lo + n) {
        const int k = id - lo;
        const uint32_t bit = 1u << (k & 31);
        if (!(atomicOr(&seen[k >> 5], bit) & bit)) {
          const float v = vals[k];
          const float w = v > 0.f ? v / p.repeat_penalty : v * p.repeat_penalty;
          vals[k] = w;
          lg[id] = w;
        }
      }
    }
    __syncthreads();
  }

  // ---- the slice's first maximum
  MaxIdx best{-INFINITY, 0x7fffffff};
  for (int j = tid; j < n; j += SLICE_THREADS) {
    const float v = vals[j];
    if (v > best.v) best = MaxIdx{v, lo + j};
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    MaxIdx o{__shfl_xor(best.v, off, 64), __shfl_xor(best.i, off, 64)};
    best = better(best, o);
  }
  if (lane == 0) mscratch[wave] = best;
  __syncthreads();
  if (tid == 0) {
    MaxIdx r = mscratch[0];
    for (int w = 1; w < WAVES_HERE; ++w) r = better(r, mscratch[w]);
    slice_tops(q)[s] = r;
  }
  if (!sliced_top_k(p)) return;

  // ---- the key of the slice's kk-th largest logit, bit by bit: the largest t with
  // at least kk keys >= t
  const int kk = min(p.top_k, n);
  if (kk == 0) {
    if (tid == 0) slice_counts(q)[s] = 0;
    return;
  }
  // (a thread's keys in registers: a count is a few dozen instructions and one barrier, where
  // a loop over LDS waited for every read in turn: 55 us a slice instead of 10)
  uint32_t key[KPT];
#pragma unroll
  for (int i = 0; i < KPT; ++i) {
    const int j = tid + i * SLICE_THREADS;
    key[i] = j < n ? order_key(vals[j]) : 0u;              // (no count asks for keys >= 0)
  }
  int turn = 0;
  auto count_from = [&](uint32_t t) {                      // keys >= t in the slice, t > 0
    int c = 0;                                             // (by ballots: the wave's count is a scalar; a count
#pragma unroll                                             //  a lane and one sum over the wave measured 2 us slower)
    for (int i = 0; i < KPT; ++i) c += __popcll(__ballot(key[i] >= t));
    if (lane == 0) counts[turn][wave] = c;
    __syncthreads();                                       // (two sets in turn: one barrier a count)
    int all = 0;
#pragma unroll
    for (int w = 0; w < WAVES_HERE; ++w) all += counts[turn][w];
    turn ^= 1;
    return all;
  };
  uint32_t t_k = 0u;
  for (int bit = 31; bit >= 0; --bit) {
    const uint32_t cand = t_k | (1u << bit);
    if (count_from(cand) >= kk) t_k = cand;
  }
  const int r_k = kk - (t_k == 0xffffffffu ? 0 : count_from(t_k + 1u));      // ties at t_k that belong

  // ---- {key > t_k} and the first r_k ties, ids ascending: wave w takes the w-th quarter
  // of the slice, 64 consecutive ids at a time; it counts, then places
  const int wspan = ((n + WAVES_HERE - 1) / WAVES_HERE + 63) / 64 * 64;
  const int first = min(n, wave * wspan), last = min(n, first + wspan);
  int above = 0, ties = 0;
  for (int j = first + lane; j - lane < last; j += 64) {
    const uint32_t key = j < last ? order_key(vals[j]) : 0u;
    above += __popcll(__ballot(j < last && key > t_k));
    ties += __popcll(__ballot(j < last && key == t_k));
  }
  if (lane == 0) { wave_above[wave] = above; wave_ties[wave] = ties; }
  __syncthreads();
  int above_before = 0, ties_before = 0;
  for (int w = 0; w < wave; ++w) { above_before += wave_above[w]; ties_before += wave_ties[w]; }
  int at = above_before + min(ties_before, r_k);
  int ties_seen = ties_before;
  const uint64_t below = (1ull << lane) - 1ull;
  float* out_v = slice_vals(q, s);
  int* out_i = slice_ids(q, s);
  for (int j = first + lane; j - lane < last; j += 64) {
    const float v = j < last ? vals[j] : 0.f;
    const uint32_t key = order_key(v);
    const bool tie = j < last && key == t_k;
    const uint64_t tie_mask = __ballot(tie);
    const bool in = j < last && (key > t_k || (tie && ties_seen + __popcll(tie_mask & below) < r_k));
    const uint64_t in_mask = __ballot(in);
    if (in) {
      const int slot = at + __popcll(in_mask & below);
      if (slot < SLICE_K) { out_v[slot] = v; out_i[slot] = lo + j; }
    }
    at += __popcll(in_mask);
    ties_seen += __popcll(tie_mask);
  }
  if (tid == 0) slice_counts(q)[s] = kk;
}

// The largest top_k whose kept set is gathered into LDS (ids ascending): every rule after
// top_k then runs over at most this many entries instead of the whole vocabulary.
constexpr int GATHER_MAX = 1024;
constexpr int HIST_COPIES = 32, HIST_PITCH = 257;   // counters of a radix pass: one set per lane % 32, a bank apart

__global__ __launch_bounds__(THREADS) void sample_kernel(int* __restrict__ out, float* __restrict__ logits,
                                                         int64_t ld, int V, const SampleParams* __restrict__ params,
                                                         const int* __restrict__ history,
                                                         const int* latest,
                                                         float* __restrict__ scratch, int64_t ld_scratch,
                                                         bool sliced) {
  extern __shared__ uint32_t bits[];            // (V + 31) / 32 words, used by the repeat penalty
  __shared__ MaxIdx mscratch[16];
  __shared__ float fscratch[16];
  __shared__ int iscratch[16];
  __shared__ int hist[HIST_COPIES * HIST_PITCH];
  __shared__ int bins[256];
  __shared__ uint32_t sh_prefix;
  __shared__ int sh_need;
  __shared__ float kept_logit[GATHER_MAX];
  __shared__ float kept_q[GATHER_MAX];
  __shared__ int kept_id[GATHER_MAX];
  __shared__ int wave_above[THREADS / 64], wave_ties[THREADS / 64];

  const int row = blockIdx.x, tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const SampleParams p = params[row];
  float* lg = logits + (int64_t)p.logits_row * ld;
  float* q = scratch + (int64_t)row * ld_scratch;

  // ---- repeat penalty (sampler.go:57-74): each distinct recent id once; the bit set says
  // which ids have had theirs
  // (latest: one more id a row that counts as the newest of its history: the token of the
  // step before, which lies on the device and which the host has not seen yet when this
  // sampling is launched.  It may be the very place that `out` names: it is read here,
  // before anything is written there.)
  // (sliced: sample_slices_kernel has run over this row; the penalty is done, and the
  // slices' maxima lie at the head of the row's scratch)
  if (!sliced && p.repeat_penalty != 1.0f && (p.history_length > 0 || latest != nullptr)) {
    const int words = (V + 31) / 32;
    for (int w = tid; w < words; w += THREADS) bits[w] = 0u;
    __syncthreads();
    const int count = p.history_length + (latest != nullptr ? 1 : 0);
    for (int i = tid; i < count; i += THREADS) {
      const int id = i < p.history_length ? history[p.history_offset + i] : latest[row];
      if (id >= 0 && id < V) {
        const uint32_t bit = 1u << (id & 31);
        if (!(atomicOr(&bits[id >> 5], bit) & bit)) {
          const float v = lg[id];
          lg[id] = v > 0.f ? v / p.repeat_penalty : v * p.repeat_penalty;
        }
      }
    }
    __threadfence_block();
    __syncthreads();
  }

  // ---- greedy (sampler.go:76-84)
  MaxIdx top;
  if (sliced) {
    if (wave == 0) {
      MaxIdx best = lane < SLICES ? slice_tops(q)[lane] : MaxIdx{-INFINITY, 0x7fffffff};
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        MaxIdx o{__shfl_xor(best.v, off, 64), __shfl_xor(best.i, off, 64)};
        best = better(best, o);
      }
      if (lane == 0) mscratch[0] = best;
    }
    __syncthreads();
    top = mscratch[0];
    if (top.i == 0x7fffffff) top.i = 0;
  } else {
    top = block_argmax(lg, V, mscratch);
  }
  if (p.temperature <= 0.f) {
    if (tid == 0) out[row] = top.i;
    return;
  }
  __shared__ int sh_choice;

  // ---- a small top_k over a row in slices: the slices' candidates (ids ascending: slice by
  // slice, and ascending within each) come into LDS in their order; the key of the top_k-th
  // largest among them bit by bit, then {key > t_k} and the first ties as below
  if (sliced && sliced_top_k(p)) {
    __shared__ int cand_before[SLICES + 1];
    float* cand_val = reinterpret_cast<float*>(hist);              // (the radix counters are not used on this path)
    constexpr int CAND_WORDS = SLICES * SLICE_K + SLICES * SLICE_K / 32;
    int* cand_id = hist + CAND_WORDS;
    static_assert(2 * CAND_WORDS <= HIST_COPIES * HIST_PITCH && SLICES * SLICE_K % 64 == 0 && SLICES * SLICE_K / 64 <= 64 &&
                  SLICES <= 64 && SLICE_K <= GATHER_MAX, "the candidates of a row: within the counters' LDS, 32 a lane");
    if (wave == 0) {
      const int c = lane < SLICES ? slice_counts(q)[lane] : 0;
      int incl = c;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const int up = __shfl_up(incl, off, 64);
        if (lane >= off) incl += up;
      }
      if (lane < SLICES) cand_before[lane] = incl - c;
      if (lane == SLICES - 1) cand_before[SLICES] = incl;
    }
    __syncthreads();
    for (int e = tid; e < SLICES * SLICE_K; e += THREADS) {
      const int sl = e / SLICE_K, k = e % SLICE_K;
      if (k < cand_before[sl + 1] - cand_before[sl]) {
        const int at = cand_before[sl] + k;
        cand_val[at + at / 32] = slice_vals(q, sl)[k];             // (a word of padding every 32: lane l reads 33 l + i)
        cand_id[at + at / 32] = slice_ids(q, sl)[k];
      }
    }
    __syncthreads();
    // wave 0 alone from here: lane l holds candidates 32 l .. 32 l + 31 as keys in registers,
    // counts meet by shuffles, no barrier
    if (wave != 0) return;
    constexpr int PER = SLICES * SLICE_K / 64;
    const int N = cand_before[SLICES], kk = min(p.top_k, N);
    uint32_t key[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int e = lane * PER + i;
      key[i] = e < N ? order_key(cand_val[e + e / 32]) : 0u;       // (no count asks for keys >= 0)
    }
    auto wave_before = [&](int c) {                  // of the lanes before this one
      int incl = c;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const int up = __shfl_up(incl, off, 64);
        if (lane >= off) incl += up;
      }
      return incl - c;
    };
    uint32_t t = 0u;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t cand = t | (1u << bit);
      int c[4] = {0, 0, 0, 0};                       // (a lane's own count in four chains, then one sum over the
#pragma unroll                                       //  wave: 1,024 ballots in a row took 17 us)
      for (int i = 0; i < PER; ++i) c[i & 3] += key[i] >= cand;
      if (wave_total((c[0] + c[1]) + (c[2] + c[3])) >= kk) t = cand;
    }
    int above = 0, ties = 0;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      above += key[i] > t;
      ties += lane * PER + i < N && key[i] == t;
    }
    const int r = kk - wave_total(above);
    int tie_rank = wave_before(ties);
    uint64_t in = 0ull;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const bool have = lane * PER + i < N;
      bool take = have && key[i] > t;
      if (have && key[i] == t) take = tie_rank++ < r;
      in |= (uint64_t)take << i;
    }
    int slot = wave_before(__popcll(in));
#pragma unroll
    for (int i = 0; i < PER; ++i)
      if ((in >> i) & 1ull) {
        const int e = lane * PER + i;
        kept_logit[slot] = cand_val[e + e / 32];
        kept_id[slot] = cand_id[e + e / 32];
        ++slot;
      }
    draw_from_kept<true>(p, top, kk, kept_logit, kept_q, kept_id, 0u, 0x7fffffff, out + row, fscratch, iscratch,
                         &sh_choice);
    return;
  }

  // ---- top_k: key of the k-th largest and how many of its ties belong (sampler.go:132-151).
  // A radix select, eight bits a pass.  Logits crowd into a few values of the leading bits, and
  // 128,000 atomic increments of a handful of LDS words would take milliseconds: every lane % 32
  // counts in a set of its own, laid out so that equal digits of different lanes fall into
  // different banks, and the sets are added up after the pass.
  uint32_t t_k = 0u;
  int r_k = 0x7fffffff;
  if (p.top_k > 0 && p.top_k < V) {
    if (tid == 0) { sh_prefix = 0u; sh_need = p.top_k; }
    uint32_t mask = 0u;
    int* mine = hist + (lane & (HIST_COPIES - 1)) * HIST_PITCH;
    for (int shift = 24; shift >= 0; shift -= 8) {
      for (int b = tid; b < HIST_COPIES * HIST_PITCH; b += THREADS) hist[b] = 0;
      __syncthreads();
      const uint32_t prefix = sh_prefix;
      scan_logits(lg, V, [&](int, float v) {
        const uint32_t key = order_key(v);
        if ((key & mask) == prefix) atomicAdd(&mine[(key >> shift) & 255u], 1);
      });
      __syncthreads();
      if (tid < 256) {
        int sum = 0;
#pragma unroll 8
        for (int c = 0; c < HIST_COPIES; ++c) sum += hist[c * HIST_PITCH + tid];
        bins[tid] = sum;
      }
      __syncthreads();
      // the digit whose count, with the counts of all larger digits, first reaches what is
      // still needed: thread t looks at digit 255 - t
      const int need = sh_need;
      const int count = tid < 256 ? bins[255 - tid] : 0;
      int all;
      const int larger = block_exclusive_scan<int>(count, iscratch, &all);
      __syncthreads();                                       // (everyone has read sh_need)
      if (tid < 256 && larger < need && (need <= larger + count || tid == 255)) {
        sh_need = need - larger;
        sh_prefix = prefix | ((uint32_t)(255 - tid) << shift);
      }
      mask |= 255u << shift;
      __syncthreads();
    }
    t_k = sh_prefix;
    r_k = sh_need;
  }

  // ---- a small top_k: its set goes to LDS, ids ascending ({key > t_k} and the first r_k
  // ties), and everything below runs over these few entries.  Wave w takes the w-th
  // sixteenth of the ids, 64 consecutive ids at a time: first it counts, then, knowing what
  // the waves before it hold, it places.
  const bool gathered = p.top_k > 0 && p.top_k < V && p.top_k <= GATHER_MAX;
  int Vn = V;                                   // entries that the rules below run over
  const float* lgp = lg;                        // their logits
  float* qp = q;                                // their unnormalised probabilities
  if (gathered) {
    const int span = ((V + THREADS / 64 - 1) / (THREADS / 64) + 63) / 64 * 64;     // ids of a wave, whole groups of 64
    const int first = min(V, wave * span), last = min(V, first + span);
    int above = 0, ties = 0;
    for (int j0 = first + lane; j0 - lane < last; j0 += 8 * 64) {     // eight loads in flight
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = j0 + 64 * u < last ? lg[j0 + 64 * u] : 0.f;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int j = j0 + 64 * u;
        const uint32_t key = order_key(v[u]);
        above += __popcll(__ballot(j < last && key > t_k));
        ties += __popcll(__ballot(j < last && key == t_k));
      }
    }
    if (lane == 0) { wave_above[wave] = above; wave_ties[wave] = ties; }
    __syncthreads();
    int above_before = 0, ties_before = 0;
    for (int w = 0; w < wave; ++w) { above_before += wave_above[w]; ties_before += wave_ties[w]; }
    int at = above_before + min(ties_before, r_k);         // kept entries of the waves before
    int ties_seen = ties_before;
    const uint64_t below = (1ull << lane) - 1ull;          // the lanes before this one
    for (int j0 = first + lane; j0 - lane < last; j0 += 8 * 64) {
      float vs[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) vs[u] = j0 + 64 * u < last ? lg[j0 + 64 * u] : 0.f;
#pragma unroll
      for (int u = 0; u < 8; ++u) {                         // in ascending id
        const int j = j0 + 64 * u;
        const float v = vs[u];
        const uint32_t key = order_key(v);
        const bool tie = j < last && key == t_k;
        const uint64_t tie_mask = __ballot(tie);
        const bool in = j < last && (key > t_k || (tie && ties_seen + __popcll(tie_mask & below) < r_k));
        const uint64_t in_mask = __ballot(in);
        if (in) {
          const int slot = at + __popcll(in_mask & below);
          if (slot < GATHER_MAX) { kept_logit[slot] = v; kept_id[slot] = j; }
        }
        at += __popcll(in_mask);
        ties_seen += __popcll(tie_mask);
      }
    }
    if (wave == THREADS / 64 - 1 && lane == 0) sh_need = min(at, GATHER_MAX);       // (the last wave has counted them all)
    __syncthreads();
    Vn = sh_need;
    lgp = kept_logit;
    qp = kept_q;
    t_k = 0u;                                   // top_k is done: every gathered entry belongs
    r_k = 0x7fffffff;
  }
  if (gathered) {
    if (wave == 0)
      draw_from_kept<true>(p, top, Vn, lgp, qp, kept_id, t_k, r_k, out + row, fscratch, iscratch, &sh_choice);
  } else {
    draw_from_kept<false>(p, top, Vn, lgp, qp, nullptr, t_k, r_k, out + row, fscratch, iscratch, &sh_choice);
  }
}

}  // namespace

// partial (rows x 64 pairs of 32-bit words) and counters (rows int32 that are zero, and are
// zero again afterwards) let a row be spread over up to 64 workgroups; without them one
// workgroup takes a row.
HFEE_API int hfee_argmax(int* out, const float* logits, int64_t ld, int rows, int V, void* partial,
                         int64_t partial_pairs, int* counters, int num_counters, hipStream_t stream) {
  HFEE_REQUIRE(rows >= 0 && V > 0 && ld >= V, "argmax: bad sizes rows=%d V=%d", rows, V);
  if (rows == 0) return 0;
  // as many workgroups as fill the chip once, each with at least 2,048 logits
  int parts = 256 / rows;
  if (parts > V / 2048) parts = V / 2048;
  if (parts > 64) parts = 64;
  if (parts > 1 && partial != nullptr && counters != nullptr && partial_pairs >= (int64_t)rows * parts &&
      num_counters >= rows) {
    argmax_parts_kernel<<<rows * parts, ARGMAX_THREADS, 0, stream>>>(out, logits, ld, V, parts, (MaxIdx*)partial, counters);
  } else {
    argmax_kernel<<<rows, THREADS, 0, stream>>>(out, logits, ld, V);
  }
  HFEE_CHECK_LAUNCH("argmax");
  return 0;
}

// ---- the same without a buffer from the caller (see no_alloc_entry.h) ----------------
// The partial results and the counters live in this array.  In host code its name is only a
// handle for hipGetSymbolAddress: every GPU has its own copy at its own address, looked up
// once per device (with that device current) and kept in argmax_static_address; host code
// hands that address on, never the name.
static __device__ __align__(256) unsigned char argmax_static_scratch[HFEE_ARGMAX_STATIC_BYTES];

namespace {

constexpr int MAX_DEVICES = 64;
std::atomic<void*> argmax_static_address[MAX_DEVICES];

// (a fill kernel and not hipMemsetAsync: a caller may be capturing a graph)
__global__ void clear_counters_kernel(int* __restrict__ counters, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) counters[i] = 0;
}

}  // namespace

HFEE_API int hfee_argmax_static(int* out, const float* logits, int64_t ld, int rows, int V, hipStream_t stream) {
  HFEE_REQUIRE(rows >= 0 && V > 0 && ld >= V, "argmax_static: bad sizes rows=%d V=%d", rows, V);
  HFEE_REQUIRE(rows <= HFEE_ARGMAX_STATIC_MAX_ROWS, "argmax_static: %d rows in one call, the library's buffer holds %d",
               rows, HFEE_ARGMAX_STATIC_MAX_ROWS);
  HFEE_REQUIRE(out != nullptr && logits != nullptr, "argmax_static: null pointer");
  if (rows == 0) return 0;
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  HFEE_REQUIRE(e == hipSuccess && device >= 0 && device < MAX_DEVICES, "argmax_static: no current device (%s)",
               hipGetErrorString(e));
  void* base = argmax_static_address[device].load(std::memory_order_acquire);
  if (base == nullptr) {        // first call on this device (two threads at once find the same address)
    e = hipGetSymbolAddress(&base, HIP_SYMBOL(argmax_static_scratch));
    HFEE_REQUIRE(e == hipSuccess && base != nullptr, "argmax_static: cannot find the library's buffer on device %d: %s",
                 device, hipGetErrorString(e));
    argmax_static_address[device].store(base, std::memory_order_release);
  }
  MaxIdx* partial = (MaxIdx*)base;
  int* counters = (int*)((unsigned char*)base + (size_t)HFEE_ARGMAX_STATIC_MAX_ROWS * HFEE_ARGMAX_STATIC_PARTS * sizeof(MaxIdx));
  int parts = 256 / rows;                                   // as hfee_argmax chooses
  if (parts > V / 2048) parts = V / 2048;
  if (parts > HFEE_ARGMAX_STATIC_PARTS) parts = HFEE_ARGMAX_STATIC_PARTS;
  if (parts > 1) {
    // the counters must be zero; a call that was cut short may have left them otherwise
    clear_counters_kernel<<<(rows + 255) / 256, 256, 0, stream>>>(counters, rows);
    argmax_parts_kernel<<<rows * parts, ARGMAX_THREADS, 0, stream>>>(out, logits, ld, V, parts, partial, counters);
  } else {
    argmax_kernel<<<rows, THREADS, 0, stream>>>(out, logits, ld, V);
  }
  HFEE_CHECK_LAUNCH("argmax_static");
  return 0;
}

// params: rows x 12 32-bit words (SampleParams).  logits may be changed in place by
// the repeat penalty, as the reference changes them.  scratch: rows x ld_scratch floats.
// latest: null, or one id a row that the repeat penalty counts as the newest of the row's
// history (a row with a window of n ids then brings n - 1 in `history`).
HFEE_API int hfee_sample(int* out, float* logits, int64_t ld, int rows, int V, const void* params,
                         const int* history, const int* latest, float* scratch, int64_t ld_scratch,
                         hipStream_t stream) {
  HFEE_REQUIRE(rows >= 0 && V > 0 && ld >= V && ld_scratch >= V, "sample: bad sizes rows=%d V=%d", rows, V);
  if (rows == 0) return 0;
  // a large vocabulary goes through the slices first (the penalty's bit set is then theirs)
  const bool sliced = V >= SLICED_MIN_V && V <= SLICES * SPAN_MAX && ld_scratch >= SLICE_WORDS && rows <= 65535;
  if (sliced) {
    const int span = ((V + SLICES - 1) / SLICES + 3) & ~3;
    const dim3 grid(SLICES, rows);
    const SampleParams* sp = (const SampleParams*)params;
    if (span <= 8 * SLICE_THREADS)
      sample_slices_kernel<8><<<grid, SLICE_THREADS, 0, stream>>>(logits, ld, V, span, sp, history, latest, scratch, ld_scratch);
    else if (span <= 16 * SLICE_THREADS)
      sample_slices_kernel<16><<<grid, SLICE_THREADS, 0, stream>>>(logits, ld, V, span, sp, history, latest, scratch, ld_scratch);
    else
      sample_slices_kernel<SPAN_MAX / SLICE_THREADS><<<grid, SLICE_THREADS, 0, stream>>>(logits, ld, V, span, sp, history, latest,
                                                                                       scratch, ld_scratch);
    HFEE_CHECK_LAUNCH("sample slices");
  }
  const size_t lds = sliced ? 0 : (size_t)((V + 31) / 32) * 4;
  HFEE_REQUIRE(lds <= 96 * 1024, "sample: a vocabulary of %d ids does not fit the penalty's bit set", V);
  static bool raised = false;
  if (lds > 32 * 1024 && !raised) {
    hipError_t e = hipFuncSetAttribute((const void*)sample_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       96 * 1024);
    HFEE_REQUIRE(e == hipSuccess, "sample: cannot raise the LDS limit: %s", hipGetErrorString(e));
    raised = true;
  }
  sample_kernel<<<rows, THREADS, lds, stream>>>(out, logits, ld, V, (const SampleParams*)params, history, latest,
                                                scratch, ld_scratch, sliced);
  HFEE_CHECK_LAUNCH("sample");
  return 0;
}
