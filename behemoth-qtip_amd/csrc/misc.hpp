#pragma once
#include "qtip_internal.hpp"
namespace qtipmi {
void launch_bf16_to_f32(const uint16_t* in, float* out, long count, hipStream_t s);
void launch_fp8_to_f32(const uint8_t* w, const uint16_t* scale_bf16, float* out, long rows, long cols, hipStream_t s);
void launch_scale_rc(float* X, long rows, long cols, long ld, const float* rs, const float* cs, hipStream_t s);
// states of one linear (m x n weights, tiles row-major) -> kernel-layout trellis words
void launch_pack_swizzle(const uint16_t* Q, long m, long n, uint16_t* out, hipStream_t s);
// kernel-layout trellis words of one linear -> hatWr (m x n fp32, row stride ld): lookup of every 16-bit window (decode.hip)
void launch_decode_trellis(const uint16_t* trellis, long m, long n, const float* entry_f, float* out, long ld,
                           hipStream_t s);
// H (n x n fp32) += X^T X for X = rows x n bf16, tiles on or below the diagonal only; then mirror + scale (hessian.hip)
void launch_hessian_accumulate(const uint16_t* X, long rows, long n, float* H, DBuf<uint16_t>& image, hipStream_t s);
void launch_hessian_finish(float* H, long n, float scale, hipStream_t s);
// tr(D H D^T) for D = A^T - B^T (m x n; A, B n x m fp32 with leading dimension ld, B may be null), H symmetric n x n
// fp32, from bf16 hi/lo products on the matrix cores; synchronises the stream
double quad_trace_bf16x3(long n, long m, const float* H, const float* A, const float* B, long ld, DBuf<uint16_t>& stack,
                         DBuf<double>& scratch, hipStream_t s);
// NVFP4 fallback quantizer (nvfp4.hip): one 16-column block of the transposed matrices, the feedback of its residual
// into the columns before it, and a byte transposer for the outputs
void launch_nvfp4_block(const float* WT, const float* FT, long m, long n, long c0, const float* L, const float* dw,
                        float global, bool calibrate, bool search, uint8_t* packedT, uint8_t* scalesT, float* E,
                        hipStream_t s);
void launch_nvfp4_feedback(float* FT, long m, long n, long c0, long col_lo, const float* E, const float* L,
                           hipStream_t s);
void launch_nvfp4_gather(float* FT, long m, long n, long cb, const float* ET, const float* L, hipStream_t s);
void launch_transpose_u8(const uint8_t* in, long rows, long cols, uint8_t* out, hipStream_t s);
}  // namespace qtipmi
