// Row-block variants of the fused aggregation kernels (see spmm_fast.hip).
#pragma once
#include "common.hpp"

namespace f2cgt {

// True when the row-block SQ kernel covers this shape (otherwise use the per-row skeleton).
bool sq_block_eligible(const void* codes, const float* out, int64_t N, int64_t src_dim, int feat_dim,
                       int target_bits, int64_t lut_entries);

// affine: table = params [2, param_stride]; log domain: table = codebooks [num_codebooks, 5].
int sq_block_run(bool affine, const uint8_t* codes, const float* table, int64_t param_stride,
                 int64_t column_slice, int num_codebooks, const void* indptr, const void* indices,
                 int idx_dtype, float* out, int64_t R, int64_t E, int64_t N, int64_t src_dim, int feat_dim,
                 int target_bits, hipStream_t st, const char* what);

// Integer-accumulating row-block kernel for per-column affine codes of 4 or 8 bits.
bool sq_affine_acc_eligible(const void* codes, const float* out, int64_t N, int64_t src_dim, int feat_dim,
                            int target_bits);
int sq_affine_acc_run(const uint8_t* codes, const float* params, int64_t param_stride, const void* indptr,
                      const void* indices, int idx_dtype, float* out, int64_t R, int64_t E, int64_t N,
                      int64_t src_dim, int feat_dim, int target_bits, hipStream_t st, const char* what);

// Row-block two-table hybrid kernel (8-bit affine SQ rows + VQ rows).
bool hybrid_acc_eligible(const void* sq_codes, const float* vq_codebooks, const float* out, int64_t N,
                         int64_t n_sq, int64_t n_vq, int feat_dim, int w);
int hybrid_acc_run(const int32_t* row_map, const uint8_t* sq_codes, const float* sq_params, int64_t param_stride,
                   const uint8_t* vq_codes, const float* vq_codebooks, const void* indptr, const void* indices,
                   int idx_dtype, float* out, int64_t R, int64_t E, int64_t N, int64_t n_sq, int64_t n_vq,
                   int feat_dim, int n_cb, int K, int w, hipStream_t st, const char* what);

// Persistent software-pipelined VQ kernel (uint8 codes, K <= 256, width 8/16/32), vq_fast.hip.
bool vq_pipe_eligible(const void* codes, const float* codebooks, const float* out, int64_t R, int64_t E,
                      int64_t N, int feat_dim, int n_cb, int K, int w);
int vq_pipe_run(const uint8_t* codes, const float* codebooks, const void* indptr, const void* indices,
                int idx_dtype, float* out, int64_t R, int64_t E, int64_t N, int feat_dim, int n_cb, int K, int w,
                hipStream_t st, const char* what);

}  // namespace f2cgt
