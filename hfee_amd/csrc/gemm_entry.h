// The entry points that the two files of bfloat16 products call in each other
// (gemm_skinny.hip: at most 64 rows; gemm_bf16.hip: the tiled kernels).  Both include
// this, so that a declaration cannot drift from its definition.
#pragma once
#include "common.h"
#include "qkv_epilogue.h"

HFEE_API int hfee_gemm_skinny(void* C, int64_t ldc, const void* A, int a_is_f32, int64_t lda, const void* W,
                              int64_t w_stride, int M, int N, int K, int epi,
                              const void* norm_weight, int norm_weight_is_f32, float eps, const int* rows,
                              const int* positions, const int* token_segment, const int* block_tables,
                              int bt_stride, const float* cos_table, const float* sin_table, int half,
                              int table_positions, void* cache, int num_heads, int kv_heads, int head_dim,
                              int page_size, const void* emit_weight, int emit_weight_is_f32, void* emit_out,
                              int64_t ld_emit, float* emit_ss, const float* scale_ss, int scale_blocks,
                              float scale_eps, float* scratch, int64_t scratch_floats, int force_mid,
                              hipStream_t stream);

HFEE_API int hfee_gemm_bf16_qkv(void* C, int64_t ldc, const void* A, int64_t lda, const void* W, int64_t ldw, int M,
                                int N, int K, const hfee::QkvArgs* qkv, int force_kernel, hipStream_t stream);

// (elementwise.hip: the norm as a kernel of its own, for the product that is followed by one)
enum { DT_F32 = 0, DT_BF16 = 1 };      // how the elementwise entry points name a tensor's type
HFEE_API int hfee_rmsnorm(void* out, int out_dtype, const float* x, const void* w, int w_dtype, const int* rows,
                          float eps, int n, int d, hipStream_t stream);
