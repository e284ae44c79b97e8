// True 32-bit matrix product for the check path: C[M,N] (+)= A[M,K] * W[N,K]^T.
//
// The role of /root/reference/internal/ggml/ops.go:54-71 (out[t,r] = W[r,:] . x[t,:]).
// Each output element is one chain of fused multiply-adds over k = 0 .. K-1 in
// ascending order, carried by a single thread; its value therefore does not
// depend on M, on where the row sits in the batch, or on the tile it falls in.
// No matrix-core instruction and no reduced-precision mode is used.
#include "common.h"

using namespace hfee;

namespace {

constexpr int BM = 64, BN = 64, BK = 16, TM = 4, TN = 4;

template <bool ACCUMULATE>
__global__ __launch_bounds__(256) void gemm_f32_kernel(float* __restrict__ C, int64_t ldc,
                                                       const float* __restrict__ A, int64_t lda,
                                                       const float* __restrict__ W, int64_t ldw,
                                                       int M, int N, int K) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int tm = (tid / 16) * TM, tn = (tid % 16) * TN;

  float acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = 0.f;

  // each thread loads 4 elements of the A tile and 4 of the W tile per step
  const int lrow = tid / 4;          // 0..63
  const int lk = (tid % 4) * 4;      // 0,4,8,12

  for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int k = k0 + lk + u;
      const int am = m0 + lrow, wn = n0 + lrow;
      As[lk + u][lrow] = (am < M && k < K) ? A[(int64_t)am * lda + k] : 0.f;
      Ws[lk + u][lrow] = (wn < N && k < K) ? W[(int64_t)wn * ldw + k] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = As[kk][tm + i];
#pragma unroll
      for (int j = 0; j < TN; ++j) b[j] = Ws[kk][tn + j];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + tm + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + tn + j;
      if (n >= N) continue;
      float* c = C + (int64_t)m * ldc + n;
      *c = ACCUMULATE ? (*c + acc[i][j]) : acc[i][j];
    }
  }
}

}  // namespace

// accumulate != 0: C += A W^T (the residual add of forward.go:106-107, 113-114).
HFEE_API int hfee_gemm_f32(float* C, int64_t ldc, const float* A, int64_t lda, const float* W, int64_t ldw,
                           int M, int N, int K, int accumulate, hipStream_t stream) {
  HFEE_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_f32: bad sizes M=%d N=%d K=%d", M, N, K);
  HFEE_REQUIRE(ldc >= N && lda >= K && ldw >= K, "gemm_f32: a leading dimension is shorter than its row");
  if (M == 0) return 0;
  dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  HFEE_REQUIRE(grid.y <= 65535, "gemm_f32: too many rows (%d)", M);
  if (accumulate)
    gemm_f32_kernel<true><<<grid, 256, 0, stream>>>(C, ldc, A, lda, W, ldw, M, N, K);
  else
    gemm_f32_kernel<false><<<grid, 256, 0, stream>>>(C, ldc, A, lda, W, ldw, M, N, K);
  HFEE_CHECK_LAUNCH("gemm_f32");
  return 0;
}
