#pragma once
#include "qtip_internal.hpp"
namespace qtipmi {
// P[128][N] = sum_{k < K} A[k][i] * (B1 - B2)[k][j] (fp64 MFMA, K split over workgroups, partial tiles summed in a
// fixed order); partials: up to kMaxGatherSplits x 128 x N doubles of scratch.  slots: the workgroup slots the
// launch will find free (it picks the number of splits that fills whole rounds of them); K a multiple of 16
constexpr int kMaxGatherSplits = 16;
int gemm_splitk_splits(long K, int N, int slots);
// Returns the number of splits S.  reduce = false leaves the sum to the reader: S == 1: the product is in P;
// otherwise the partial slabs are partials[y * 128 * N + ...], y < S, to be added in this order.
int launch_gemm_tn_f64_gather(int N, long K, const float* A, long lda, const float* B1, const float* B2, long ldb,
                              double* P, double* partials, int slots, hipStream_t s, bool reduce = true);
// The gathered product in the reference GPU path's arithmetic: operands as bf16 hi + lo images with k contiguous,
// three MFMA terms, fp32 accumulate; P and the partials (up to kMaxGatherSplits x 128 x N) in fp32.
//   a: Ah / Al[i * lda + k], i < 128   (launch_split_transpose_bf16 of L, offset to the buffer's columns and rows)
//   b: Bh / Bl[j * ldb + k], j < N     (written by the Viterbi kernel, TileJob::dimg_h / dimg_l)
int launch_gemm_img_gather(int N, long K, const uint16_t* Ah, const uint16_t* Al, long lda, const uint16_t* Bh,
                           const uint16_t* Bl, long ldb, float* P, float* partials, int slots, hipStream_t s,
                           bool reduce = true);
// Th / Tl[i * ldt + k] = bf16 hi / lo of X[k * ldx + i] (minus X2[k * ldx + i] when X2 is given), k < rows_k,
// i < cols_i, both multiples of 64; lower_only: the 64 x 64 tiles wholly above the diagonal are skipped
void launch_split_transpose_bf16(const float* X, const float* X2, long ldx, long rows_k, long cols_i, uint16_t* Th,
                                 uint16_t* Tl, long ldt, bool lower_only, hipStream_t s);
}  // namespace qtipmi
