// Seeded random tensors on the device: element i of a tensor is a function of
// (key, i) alone, where the key comes from the seed and the tensor's name, and the
// host twin in weights/random_stream.py gives the same bits.  The reference has no
// random-weights mode (a model there is always a file: /root/reference/internal/llm/model.go:58-70).
//
// Normal numbers: one 64-bit hash per pair of elements, Box-Muller in float64.  Both
// sides must round alike, so nothing comes from a math library: the logarithm, sine and
// cosine in random_stream.h are fixed sequences of float64 additions, multiplications,
// divisions and one square root, which IEEE 754 rounds correctly on either side; products
// are not contracted into fused multiply-adds (numpy has none).
#include "common.h"
#include "random_stream.h"

namespace {

// kind 0: std * z; 1: 1 + std * z (float64, rounded once to float32, then to the type);
// out_type 0: float32, 1: bfloat16.  A thread makes the pair (2j, 2j + 1).
__global__ void __launch_bounds__(256) random_normal_kernel(void* __restrict__ out, int out_type, int64_t count,
                                                            uint64_t key, int kind, double std) {
  const int64_t pairs = (count + 1) / 2;
  for (int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; j < pairs; j += (int64_t)gridDim.x * blockDim.x) {
    float f0, f1;
    hfee_random::normal_pair(key, (uint64_t)j, kind == 1, std, f0, f1);
    const int64_t i = 2 * j;
    if (out_type == 0) {
      ((float*)out)[i] = f0;
      if (i + 1 < count) ((float*)out)[i + 1] = f1;
    } else {
      ((bf16_t*)out)[i] = hfee::float_to_bf16(f0);
      if (i + 1 < count) ((bf16_t*)out)[i + 1] = hfee::float_to_bf16(f1);
    }
  }
}

// out[i] = (hash(key, i) >> 11) mod bound, int32.
__global__ void __launch_bounds__(256) random_int_kernel(int32_t* __restrict__ out, int64_t count, uint64_t key,
                                                         uint32_t bound) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (int64_t)gridDim.x * blockDim.x)
    out[i] = hfee_random::integer(key, (uint64_t)i, bound);
}

}  // namespace

// kind 0 / 1: normal numbers (see random_normal_kernel; out_type 0 float32, 1 bfloat16);
// kind 2: integers in [0, bound) as int32 (out_type ignored).
HFEE_API int hfee_random_fill(void* out, int out_type, int64_t count, uint64_t key, int kind, double std, int64_t bound,
                              hipStream_t stream) {
  HFEE_REQUIRE(out != nullptr && count >= 0, "random_fill: no output");
  HFEE_REQUIRE(kind >= 0 && kind <= 2, "random_fill: kind %d is not 0 (normal), 1 (one plus normal) or 2 (integers)", kind);
  if (count == 0) return 0;
  if (kind == 2) {
    HFEE_REQUIRE(bound >= 1 && bound <= 0x7FFFFFFF, "random_fill: integers need a bound in 1..2^31-1, got %lld", (long long)bound);
    const int64_t blocks = (count + 255) / 256;
    random_int_kernel<<<(unsigned)(blocks < 65536 ? blocks : 65536), 256, 0, stream>>>((int32_t*)out, count, key, (uint32_t)bound);
  } else {
    HFEE_REQUIRE(out_type == 0 || out_type == 1, "random_fill: output type %d is not float32 (0) or bfloat16 (1)", out_type);
    const int64_t blocks = ((count + 1) / 2 + 255) / 256;
    random_normal_kernel<<<(unsigned)(blocks < 65536 ? blocks : 65536), 256, 0, stream>>>(out, out_type, count, key, kind, std);
  }
  HFEE_CHECK_LAUNCH("random_fill");
  return 0;
}
