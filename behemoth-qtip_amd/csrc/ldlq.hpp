#pragma once
#include "qtip_internal.hpp"
namespace qtipmi {
// P[128][N] = sum_{k < K} A[k][i] * (B1 - B2)[k][j] (fp64 MFMA, K split over workgroups, partial tiles summed in a
// fixed order); partials: up to kMaxGatherSplits x 128 x N doubles of scratch.  slots: the workgroup slots the
// launch will find free (it picks the number of splits that fills whole rounds of them); K a multiple of 16
constexpr int kMaxGatherSplits = 16;
int gemm_splitk_splits(long K, int N, int slots);
void launch_gemm_tn_f64_gather(int N, long K, const float* A, long lda, const float* B1, const float* B2, long ldb,
                               double* P, double* partials, int slots, hipStream_t s);
// the gathered product with every operand split into bf16 hi + lo (three MFMA terms, fp32 accumulate), P and the
// partials (up to kMaxGatherSplits x 128 x N) in fp32
void launch_gemm_tn_bf16x3_gather(int N, long K, const float* A, long lda, const float* B1, const float* B2, long ldb,
                                  float* P, float* partials, int slots, hipStream_t s);
}  // namespace qtipmi
