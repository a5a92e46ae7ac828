#pragma once
#include "qtip_internal.hpp"
namespace qtipmi {
void launch_ldlq_prep_f64(const float* WT, const float* hatWT, const double* prod, const float* L, long n, long m,
                          int col0, int bufend, float* X, hipStream_t s);
void launch_ldlq_prep_f32(const float* WT, const float* hatWT, const float* prod, const float* L, long n, long m,
                          int col0, int bufend, float* X, hipStream_t s);
// C[M][N] += sum_k A[k][i] * (B1 - B2)[k][j]; A fp32 [K][lda], B fp32 [K][ldb] (B2 may be null), C fp64
void launch_gemm_tn_f64_acc(int M, int N, int K, const float* A, long lda, const float* B1, const float* B2, long ldb,
                            double* C, long ldc, hipStream_t s);
// the same product with fp32 C and every operand split into bf16 hi + lo (three MFMA terms, fp32 accumulate); K = 128
void launch_gemm_tn_bf16x3_acc(int M, int N, int K, const float* A, long lda, const float* B1, const float* B2, long ldb,
                               float* C, long ldc, hipStream_t s);
// sum over the N columns x of X = B1 - B2 (n x N, stride ldb) of x^T H x, H n x n fp32; synchronises the stream
double quad_trace_f64(int n, int N, const float* H, const float* B1, const float* B2, long ldb, DBuf<double>& scratch,
                      hipStream_t s);
}  // namespace qtipmi
