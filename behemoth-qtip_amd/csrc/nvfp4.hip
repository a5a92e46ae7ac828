// NVFP4 fallback quantizer on the device: scale search and Hessian-calibrated rounding (reference:
// nvfp4_quantize_group, nv_block_kernel and nv_feedback_kernel, src/nvfp4_gpu.hip:66-243; format src/nvfp4.hpp).
// Every fp32 operation is the reference kernel's, in its order.  The reference builds with hipcc's default
// floating-point contraction, which turns its three "sum += a * b" statements (block feedback, cost, column
// feedback) into fused multiply-adds; this file is built without contraction and writes those three as fmaf, so
// the bytes equal both the reference's gfx950 build and a CPU evaluation of the same formulas.
//
// Layout: the reference walks row-major W with one thread per matrix row, so neighbouring lanes are n floats apart.
// Here W, the feedback F and the outputs live transposed on the device ([column][row]): a wave's 64 rows are one
// 256-byte line for every column it touches.  Columns are processed in 16-wide blocks from the last to the first;
// the residual of a finished block goes to all remaining columns before the next block starts.
#include "misc.hpp"
#include "nvfp4_codec.hpp"
#include "qtip_internal.hpp"

namespace qtipmi {
namespace {

// The scalar codec is nvfp4_codec.hpp's: e4m3_value (code <= 126 -> value), e4m3_of_magnitude (finite x -> code of |x|),
// through_bf16, e2m1_value and e2m1_of_magnitude (a >= 0 -> code).
namespace nvc = nvcodec;

constexpr int kScaleTries = 11;  // scale candidates of the search: the plain one, 8 shrink factors, one code down, one up
constexpr int kBlockRows = 64;  // matrix rows per workgroup: one per lane

// Block scale candidate number `which` (uniform over a wave) of a row whose 16 targets have the largest magnitude
// amax; the list and its order are the reference's (src/nvfp4_gpu.hip:97-105).
__device__ __forceinline__ unsigned nv_candidate(int which, float amax, float global) {
  if (which >= 1 && which <= 8) {
    float shrink = 1.05f;
    switch (which) {
      case 1: shrink = 0.70f; break;
      case 2: shrink = 0.75f; break;
      case 3: shrink = 0.80f; break;
      case 4: shrink = 0.85f; break;
      case 5: shrink = 0.90f; break;
      case 6: shrink = 0.95f; break;
      case 7: shrink = 1.00f; break;
      default: break;
    }
    return nvc::e4m3_of_magnitude(amax * shrink / (6.f * global));
  }
  const unsigned plain = nvc::e4m3_of_magnitude(amax / (6.f * global));
  if (which == 9) return plain > 0 ? plain - 1 : 0;
  if (which == 10) return plain < 126 ? plain + 1 : 126;
  return plain;
}

// One 16-column block (columns c0 .. c0 + 15) per launch, 64 matrix rows per workgroup, and one wave per scale
// candidate: the reference's thread walks through its row's candidates one after the other and then rounds once more
// with the winner (src/nvfp4_gpu.hip:66-158); here the ncand waves of a workgroup round the same 64 rows at the same
// time, each under its own candidate, leave their costs in LDS, and the wave whose candidate wins a row (smallest cost,
// the earliest candidate among equals) writes that row's result.  With s the candidate's scale:
//   t_k  = W[k] + F[k] + sum_{j > k in block} d_j Ltile[j][k]   target after the feedback, j ascending
//   q_k  = bf16(level * dec(s) * global)                       what execution sees
//   d_k  = W[k] - q_k                                          error fed back
//   cost = sum_k dw[k] (t_k - q_k)^2                           proxy increment, k descending
// WT, FT: [n][m].  packedT: [n/2][m], scalesT: [n/16][m], E: [16][m].
__global__ __launch_bounds__(kBlockRows * kScaleTries) void nv_block_kernel(
    const float* __restrict__ WT, const float* __restrict__ FT, long m, long n, long c0, const float* __restrict__ L,
    const float* __restrict__ dw, float global, int calibrate, int ncand, uint8_t* __restrict__ packedT,
    uint8_t* __restrict__ scalesT, float* __restrict__ E) {
  __shared__ float Ltile[16][16];
  __shared__ float colw[16];
  __shared__ float costs[kScaleTries][kBlockRows];
  const int lane = threadIdx.x & 63;
  const int which = __builtin_amdgcn_readfirstlane(int(threadIdx.x >> 6));
  for (int idx = threadIdx.x; idx < 256; idx += blockDim.x)
    Ltile[idx >> 4][idx & 15] = calibrate ? L[(c0 + (idx >> 4)) * n + c0 + (idx & 15)] : 0.f;
  if (threadIdx.x < 16) colw[threadIdx.x] = dw ? dw[c0 + threadIdx.x] : 1.f;
  __syncthreads();
  const long r = long(blockIdx.x) * kBlockRows + lane;
  const bool live = r < m;
  float w[16], t0[16], err[16];
  float amax = 0.f;
#pragma unroll
  for (int k = 0; k < 16; ++k) {
    w[k] = live ? WT[(c0 + k) * m + r] : 0.f;
    t0[k] = w[k] + (calibrate && live ? FT[(c0 + k) * m + r] : 0.f);
    amax = fmaxf(amax, fabsf(calibrate ? t0[k] : w[k]));
  }
  const unsigned code8 = nv_candidate(which, amax, global);
  const float sd = nvc::e4m3_value(code8);
  const float step = sd * global;
  float cost = 0.f;
  uint32_t nib_lo = 0, nib_hi = 0;  // E2M1 codes of columns 0..7 and 8..15, 4 bits each
#pragma unroll
  for (int k = 15; k >= 0; --k) {
    float t = t0[k];
    if (calibrate) {
#pragma unroll
      for (int j = k + 1; j < 16; ++j) t = fmaf(err[j], Ltile[j][k], t);
    }
    const float x = step != 0.f ? t / step : 0.f;
    const unsigned mag = nvc::e2m1_of_magnitude(fabsf(x));
    const float q = nvc::through_bf16((x < 0 ? -1.f : 1.f) * nvc::e2m1_value(mag) * sd * global);
    cost = fmaf(colw[k] * (t - q), t - q, cost);
    err[k] = w[k] - q;
    const uint32_t nib = mag | ((__float_as_uint(x) >> 31) << 3);
    if (k < 8) nib_lo |= nib << (4 * k);
    else nib_hi |= nib << (4 * (k - 8));
  }
  costs[which][lane] = cost;
  __syncthreads();
  int winner = 0;
  float least = __builtin_inff();
  for (int i = 0; i < ncand; ++i)
    if (costs[i][lane] < least) least = costs[i][lane], winner = i;
  if (!live || winner != which) return;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    packedT[(c0 / 2 + k) * m + r] = uint8_t(nib_lo >> (8 * k));
    packedT[(c0 / 2 + 4 + k) * m + r] = uint8_t(nib_hi >> (8 * k));
  }
  scalesT[(c0 / 16) * m + r] = uint8_t(code8);
#pragma unroll
  for (int k = 0; k < 16; ++k) E[k * m + r] = err[k];
}

// FT[col][r] += sum_{j < 16} E[j][r] * L[c0 + j][col]  for col_lo <= col < c0 (the sum first, in j order, then one
// add).  A workgroup: 256 rows x 32 columns; the 16 x 32 piece of L sits in LDS.
__global__ __launch_bounds__(256) void nv_feedback_kernel(float* __restrict__ FT, long m, long n, long c0, long col_lo,
                                                          const float* __restrict__ E, const float* __restrict__ L) {
  __shared__ float Ls[16][32];
  const long col0 = col_lo + long(blockIdx.y) * 32;
  for (int idx = threadIdx.x; idx < 512; idx += 256) {
    const int j = idx >> 5, c = idx & 31;
    Ls[j][c] = col0 + c < c0 ? L[(c0 + j) * n + col0 + c] : 0.f;
  }
  __syncthreads();
  const long r = long(blockIdx.x) * 256 + threadIdx.x;
  if (r >= m) return;
  float e[16];
#pragma unroll
  for (int j = 0; j < 16; ++j) e[j] = E[j * m + r];
  const int ncol = int(c0 - col0 < 32 ? c0 - col0 : 32);
  for (int c = 0; c < ncol; ++c) {
    float acc = 0;
#pragma unroll
    for (int j = 0; j < 16; ++j) acc = fmaf(e[j], Ls[j][c], acc);
    FT[(col0 + c) * m + r] += acc;
  }
}

// The feedback a 128-column buffer [cb, cb + 128) receives from every block behind it, gathered in one pass:
//   FT[col][r] = ((0 + a_{n-16}) + a_{n-32}) + ... + a_{cb+128},   a_b = sum_{j < 16} E[b + j][r] * L[b + j][col]
// (each a_b a chain of fused multiply-adds in j order from zero): the values and the order of additions of the
// block-by-block form, which reads and writes every column left of a block once per block (n^2 m / 4 bytes in all);
// this form reads the error rows once per buffer (n^2 m / 64 bytes).  ET: the errors of all finished columns, [n][m].
// A wave: 64 rows x kGatherCols columns (narrow, so that a matrix of 12288 rows still gives every SIMD several waves);
// the four waves of a workgroup take four neighbouring column pieces of the same 64 rows, so three of them find the
// error values in the vector L1.  The piece of L of a block is the same for a whole wave and arrives through the
// scalar cache.
constexpr int kGatherCols = 8;
__global__ __launch_bounds__(256) void nv_gather_kernel(float* __restrict__ FT, long m, long n, long cb,
                                                        const float* __restrict__ ET, const float* __restrict__ L) {
  const long r = long(blockIdx.x) * 64 + (threadIdx.x & 63);
  const long col0 = cb + (long(blockIdx.y) * 4 + __builtin_amdgcn_readfirstlane(int(threadIdx.x >> 6))) * kGatherCols;
  if (r >= m) return;
  float f[kGatherCols];
#pragma unroll
  for (int c = 0; c < kGatherCols; ++c) f[c] = 0.f;
  for (long b = n - 16; b >= cb + 128; b -= 16) {
    float e[16], acc[kGatherCols];
#pragma unroll
    for (int j = 0; j < 16; ++j) e[j] = ET[(b + j) * m + r];
#pragma unroll
    for (int c = 0; c < kGatherCols; ++c) acc[c] = 0.f;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const float* __restrict__ lrow = L + (b + j) * n + col0;  // uniform over the workgroup
#pragma unroll
      for (int c = 0; c < kGatherCols; ++c) acc[c] = fmaf(e[j], lrow[c], acc[c]);
    }
#pragma unroll
    for (int c = 0; c < kGatherCols; ++c) f[c] += acc[c];
  }
#pragma unroll
  for (int c = 0; c < kGatherCols; ++c) FT[(col0 + c) * m + r] = f[c];
}

// bytes [rows][cols] -> [cols][rows], 32 x 32 patches through LDS
__global__ __launch_bounds__(256) void transpose_u8_kernel(const uint8_t* __restrict__ in, long rows, long cols,
                                                           uint8_t* __restrict__ out) {
  __shared__ uint8_t tile[32][33];
  const long r0 = long(blockIdx.y) * 32, c0 = long(blockIdx.x) * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const long r = r0 + ty + 8 * k, c = c0 + tx;
    tile[ty + 8 * k][tx] = r < rows && c < cols ? in[r * cols + c] : uint8_t(0);
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const long c = c0 + ty + 8 * k, r = r0 + tx;
    if (c < cols && r < rows) out[c * rows + r] = tile[tx][ty + 8 * k];
  }
}

}  // namespace

void launch_nvfp4_block(const float* WT, const float* FT, long m, long n, long c0, const float* L, const float* dw,
                        float global, bool calibrate, bool search, uint8_t* packedT, uint8_t* scalesT, float* E,
                        hipStream_t s) {
  const int ncand = search ? kScaleTries : 1;
  nv_block_kernel<<<dim3(unsigned((m + kBlockRows - 1) / kBlockRows)), dim3(unsigned(kBlockRows * ncand)), 0, s>>>(
      WT, FT, m, n, c0, L, dw, global, calibrate ? 1 : 0, ncand, packedT, scalesT, E);
  QTIP_HIP(hipGetLastError());
}
void launch_nvfp4_feedback(float* FT, long m, long n, long c0, long col_lo, const float* E, const float* L,
                           hipStream_t s) {
  if (c0 <= col_lo) return;
  QTIP_REQUIRE(col_lo >= 0 && c0 <= n, "nvfp4 feedback: column window [%ld, %ld) outside [0, %ld)", col_lo, c0, n);
  nv_feedback_kernel<<<dim3(unsigned((m + 255) / 256), unsigned((c0 - col_lo + 31) / 32)), dim3(256), 0, s>>>(
      FT, m, n, c0, col_lo, E, L);
  QTIP_HIP(hipGetLastError());
}
void launch_nvfp4_gather(float* FT, long m, long n, long cb, const float* ET, const float* L, hipStream_t s) {
  QTIP_REQUIRE(cb >= 0 && cb % 16 == 0 && cb + 128 <= n && n % 16 == 0, "nvfp4 gather: buffer [%ld, %ld) outside [0, %ld)",
               cb, cb + 128, n);
  nv_gather_kernel<<<dim3(unsigned((m + 63) / 64), 128 / kGatherCols / 4), dim3(256), 0, s>>>(FT, m, n, cb, ET, L);
  QTIP_HIP(hipGetLastError());
}
void launch_transpose_u8(const uint8_t* in, long rows, long cols, uint8_t* out, hipStream_t s) {
  if (rows <= 0 || cols <= 0) return;
  transpose_u8_kernel<<<dim3(unsigned((cols + 31) / 32), unsigned((rows + 31) / 32)), dim3(256), 0, s>>>(in, rows, cols, out);
  QTIP_HIP(hipGetLastError());
}

}  // namespace qtipmi
