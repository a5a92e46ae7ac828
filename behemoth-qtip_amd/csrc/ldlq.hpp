#pragma once
#include "qtip_internal.hpp"
namespace qtipmi {
// P[128][N] = sum_{k < K} A[k][i] * (B1 - B2)[k][j] (fp64 MFMA, K split over workgroups, partial tiles summed in a
// fixed order); partials: gemm_splitk_splits(K) x 128 x N doubles of scratch
int gemm_splitk_splits(long K);
void launch_gemm_tn_f64_gather(int N, long K, const float* A, long lda, const float* B1, const float* B2, long ldb,
                               double* P, double* partials, hipStream_t s);
// the same product with fp32 C and every operand split into bf16 hi + lo (three MFMA terms, fp32 accumulate); K = 128
void launch_gemm_tn_bf16x3_acc(int M, int N, int K, const float* A, long lda, const float* B1, const float* B2, long ldb,
                               float* C, long ldc, hipStream_t s);
}  // namespace qtipmi
