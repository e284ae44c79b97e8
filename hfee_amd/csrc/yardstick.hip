// What the chip gives to the simplest possible kernels, as yardsticks beside the published
// peaks: a read-only stream over device memory, and a loop of nothing but matrix
// instructions.  The read-only stream doubles as a prefetch: reading a tensor that a later
// kernel will stream brings it into the memory-side cache while a kernel that is bound by
// latency, not by memory, runs beside it.
#include "common.h"

using namespace hfee;

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int READ_THREADS = 256;
constexpr int READ_AHEAD = 8;        // 16-byte loads a thread keeps in flight

// Every workgroup walks its own contiguous stretch of the buffer; nothing is stored unless the
// words read add up to a value that they never do (which keeps the loads alive).
template <bool KEEP_OUT_OF_L2>
__global__ __launch_bounds__(READ_THREADS) void read_stream_kernel(const u32x4* __restrict__ p, int64_t count,
                                                                   uint32_t* __restrict__ sink) {
  const int64_t per = (count + gridDim.x - 1) / gridDim.x;
  const int64_t begin = (int64_t)blockIdx.x * per, end = min(count, begin + per);
  uint32_t acc = 0;
  int64_t i = begin + threadIdx.x;
  for (; i + (int64_t)(READ_AHEAD - 1) * READ_THREADS < end; i += (int64_t)READ_AHEAD * READ_THREADS) {
    u32x4 v[READ_AHEAD];
#pragma unroll
    for (int u = 0; u < READ_AHEAD; ++u) {
      if constexpr (KEEP_OUT_OF_L2) v[u] = __builtin_nontemporal_load(p + i + (int64_t)u * READ_THREADS);
      else v[u] = p[i + (int64_t)u * READ_THREADS];
    }
#pragma unroll
    for (int u = 0; u < READ_AHEAD; ++u) acc += v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
  }
  for (; i < end; i += READ_THREADS) {
    const u32x4 v = p[i];
    acc += v[0] ^ v[1] ^ v[2] ^ v[3];
  }
  if (acc == 0x9E3779B9u && sink != nullptr) sink[0] = acc;      // (never, for all practical data)
}

// Each wave issues `iterations` rounds of 64 independent matrix instructions on registers: a
// wave tile of 128 x 128 as the product kernels have it, eight operands a side.  The
// instruction is the 16 x 16 x 32 one: with operands as real ones are the GPU sustains about
// 2.1 PFLOP/s of it and 1.76 of the 32 x 32 x 16 one (both 2.5 on zeros).
__global__ __launch_bounds__(256) void mfma_loop_kernel(float* __restrict__ sink, int iterations) {
  f32x4 acc[8][8];
  bf16x8 a[8], b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) {     // operands with every bit in use, as real ones have: the power they draw sets the clock
      const uint32_t h = ((threadIdx.x + 977u * i) * 8u + e + 1u) * 2654435761u;
      a[i][e] = (__bf16)((float)(int)((h >> 8) & 0xffff) * (1.0f / 65536.0f) - 0.5f);
      b[i][e] = (__bf16)((float)(int)((h >> 12) & 0xffff) * (1.0f / 65536.0f) - 0.5f);
    }
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iterations; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
  }
  float total = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) total += acc[i][j][r];
  if (total == 12345.678f && sink != nullptr) sink[0] = total;   // (never, for all practical purposes)
}

}  // namespace

// Reads `bytes` (a multiple of 16, from a 16-byte aligned address) once, with `workgroups`
// workgroups.  keep_out_of_l2: the loads carry the non-temporal hint (a prefetch for another
// kernel should not push that kernel's own lines out of the L2).
HFEE_API int hfee_read_stream(const void* p, int64_t bytes, void* sink, int workgroups, int keep_out_of_l2,
                              hipStream_t stream) {
  HFEE_REQUIRE(bytes >= 0 && bytes % 16 == 0 && (uintptr_t)p % 16 == 0, "read_stream: 16-byte alignment expected");
  HFEE_REQUIRE(workgroups >= 1 && workgroups <= 65536, "read_stream: bad number of workgroups %d", workgroups);
  if (bytes == 0) return 0;
  if (keep_out_of_l2)
    read_stream_kernel<true><<<workgroups, READ_THREADS, 0, stream>>>((const u32x4*)p, bytes / 16, (uint32_t*)sink);
  else
    read_stream_kernel<false><<<workgroups, READ_THREADS, 0, stream>>>((const u32x4*)p, bytes / 16, (uint32_t*)sink);
  HFEE_CHECK_LAUNCH("read_stream");
  return 0;
}

// workgroups x 4 waves x iterations x 64 matrix instructions of 2 * 16 * 16 * 32 flops each.
HFEE_API int hfee_mfma_loop(void* sink, int iterations, int workgroups, hipStream_t stream) {
  HFEE_REQUIRE(iterations >= 1 && workgroups >= 1 && workgroups <= 65536, "mfma_loop: bad sizes");
  mfma_loop_kernel<<<workgroups, 256, 0, stream>>>((float*)sink, iterations);
  HFEE_CHECK_LAUNCH("mfma_loop");
  return 0;
}
