// Cross-buffer feedback of LDLQ for gfx950 (reference: ldlq_gpu, src/quantizer.cpp:30-89; the CPU form of the
// algorithm, tests/test_gpu.cpp:180-225).  The in-buffer feedback of a 16-column block is formed inside the Viterbi
// kernel (viterbi.hip, tile_targets).
//
//  * gemm_tn: sum_k A[k][i] * (B1 - B2)[k][j] on the fp64 matrix cores (v_mfma_f64_16x16x4_f64), fp32 operands
//    widened while staging through LDS.  The cross-buffer feedback ("prod cache") of a 128-column buffer is gathered
//    from all rows quantized so far by a K-split kernel.
//  * gemm_tn_bf16x3_gather: the same gathered product in the arithmetic of the reference's GPU path: every fp32
//    operand split into bf16 hi + lo, three v_mfma_f32_32x32x16_bf16 terms, fp32 accumulation.
#include <algorithm>

#include "ldlq.hpp"
#include "qtip_internal.hpp"

namespace qtipmi {
namespace {

// ---------------------------------------------------------------- fp64 MFMA GEMM
typedef double double4_t __attribute__((ext_vector_type(4)));
constexpr int BM = 128, BN = 128, KC = 16;

// ---------------------------------------------------------------- fp64 MFMA GEMM, 128 output rows, K split
// out[y][i][j] = sum over the K slices of split y of A[k][i] * (B1 - B2)[k][j], i < 128: the cross-buffer feedback
// of one 128-column LDLQ buffer gathered from all rows already quantized ("left-looking": every product term is
// read once and nothing is read-modified-written).  K is long and the output small, so the K range is shared out
// over gridDim.y workgroups per column tile (boundaries at multiples of 16 rows) and the partial tiles are summed
// afterwards in a fixed order.
// The fp32 operand rows go from global memory straight into LDS (global_load_lds_dwordx4: a wave's 64 lanes fill
// two 128-float rows), 8 rows of K per stage, four stages of LDS (three in flight ahead of the one in use), one barrier per stage that orders LDS only; a
// lane widens its fragments to fp64 (and forms B1 - B2) as it reads them.  No staging registers: 168 registers and
// 48 KB of LDS, so that a workgroup fits beside two workgroups of the Viterbi kernel, which holds the other chain's
// share of the chip while this one runs.  Columns beyond N (last column tile) read the row's last four floats
// instead; they only feed outputs that are not stored.
constexpr int GVK = 8, GST = 4;
__global__ __launch_bounds__(256, 3) void gemm_tn_f64_splitk_kernel(int N, long K, const float* __restrict__ A, long lda,
                                                                    const float* __restrict__ B1,
                                                                    const float* __restrict__ B2, long ldb,
                                                                    double* __restrict__ out, long ldo) {
  __shared__ __attribute__((aligned(16))) float S[GST][3][GVK][BM];  // [stage][A | B1 | B2][k][column]
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const long j0 = long(blockIdx.x) * BN;
  const long slices = (K + KC - 1) / KC;  // K is a multiple of 16
  const long k0 = KC * (slices * blockIdx.y / gridDim.y), k1 = KC * (slices * (blockIdx.y + 1) / gridDim.y);
  const int stages = int((k1 - k0) / GVK);
  double4_t acc[4][4];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b) acc[a][b] = double4_t{0, 0, 0, 0};
  // wave w brings rows 2w (lanes 0..31) and 2w + 1 (lanes 32..63) of a stage, four floats per lane
  const long row = k0 + 2 * wave + (lane >> 5), colA = 4 * (lane & 31);
  long colB = j0 + colA;
  if (colB + 3 >= N) colB = N - 4;
  const float* ga = A + row * lda + colA;
  const float* gb = B1 + row * ldb + colB;
  const float* gc = B2 + row * ldb + colB;
  typedef __attribute__((address_space(3))) void* lds_ptr;
  auto issue = [&](int stage) {
    const int st = stage % GST;
    const long off = long(stage) * GVK;
    __builtin_amdgcn_global_load_lds(ga + off * lda, (lds_ptr)&S[st][0][2 * wave][0], 16, 0, 0);
    __builtin_amdgcn_global_load_lds(gb + off * ldb, (lds_ptr)&S[st][1][2 * wave][0], 16, 0, 0);
    __builtin_amdgcn_global_load_lds(gc + off * ldb, (lds_ptr)&S[st][2][2 * wave][0], 16, 0, 0);
  };
  for (int p = 0; p < GST - 1 && p < stages; ++p) issue(p);
  for (int sg = 0; sg < stages; ++sg) {
    // this wave's loads of stage sg have landed when only those of the stages issued after it are outstanding
    // (3 loads per stage; loads return in order)
    const int later = stages - 1 - sg < GST - 2 ? stages - 1 - sg : GST - 2;
    if (later >= 2) __builtin_amdgcn_s_waitcnt(0x0F76);       // vmcnt(6)
    else if (later == 1) __builtin_amdgcn_s_waitcnt(0x0F73);  // vmcnt(3)
    else __builtin_amdgcn_s_waitcnt(0x0F70);                  // vmcnt(0)
    // everyone's have, and everyone is done reading the stage that the next issue overwrites (a bare barrier:
    // __syncthreads() would also wait for the loads still in flight)
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (sg + GST - 1 < stages) issue(sg + GST - 1);
    const int st = sg % GST;
#pragma unroll
    for (int kk = 0; kk < GVK; kk += 4) {
      const int kr = kk + (lane >> 4), c = lane & 15;
      double a[4], b[4];
#pragma unroll
      for (int mi = 0; mi < 4; ++mi) a[mi] = double(S[st][0][kr][wm * 64 + mi * 16 + c]);
#pragma unroll
      for (int ni = 0; ni < 4; ++ni)
        b[ni] = double(S[st][1][kr][wn * 64 + ni * 16 + c]) - double(S[st][2][kr][wn * 64 + ni * 16 + c]);
#pragma unroll
      for (int mi = 0; mi < 4; ++mi)
#pragma unroll
        for (int ni = 0; ni < 4; ++ni)
          acc[mi][ni] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[mi], b[ni], acc[mi][ni], 0, 0, 0);
    }
  }
  double* o = out + long(blockIdx.y) * BM * ldo;
#pragma unroll
  for (int mi = 0; mi < 4; ++mi)
#pragma unroll
    for (int ni = 0; ni < 4; ++ni)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const long gi = wm * 64 + mi * 16 + (lane >> 4) + 4 * v;
        const long gj = j0 + wn * 64 + ni * 16 + (lane & 15);
        if (gj < N) o[gi * ldo + gj] = acc[mi][ni][v];
      }
}

// P[i] = part[0][i] + part[1][i] + ... (in this order), i < count
__global__ void sum_splits_kernel(const double* __restrict__ part, int splits, long count, double* __restrict__ P) {
  const long i = long(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= count) return;
  double s = part[i];
  for (int k = 1; k < splits; ++k) s += part[long(k) * count + i];
  P[i] = s;
}

// ---------------------------------------------------------------- bf16 hi/lo split operands
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
constexpr int SB = 128;  // rows and columns of a workgroup's output tile

__device__ __forceinline__ uint32_t bf16_rne_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}

// ---------------------------------------------------------------- bf16 hi/lo split MFMA GEMM, gathered (fp32 accumulate)
// out[y][i][j] = sum over the K slices of split y of A[k][i] * (B1 - B2)[k][j], i < 128, in the arithmetic of the
// reference's prod-cache update (src/quantizer.cpp:66-76: x = hi + lo in bf16, product = hi*hi + hi*lo + lo*hi, fp32
// accumulate) but gathered like the fp64 kernel above: K is everything quantized so far, nothing is
// read-modified-written.  128 x 128 outputs per workgroup, 4 waves of 64 x 64 (2 x 2 tiles of 32 x 32); K goes
// through LDS 32 rows at a time, split on the way ([row][k] with k contiguous: a lane's 8 consecutive k are one
// 16-byte read; the row stride of 80 bytes keeps those reads free of bank conflicts); a thread stages 4 rows x 8 k of
// one operand per slice and fetches the next slice's while the matrix cores work.  Bound by HBM, not by the matrix
// cores: a row k of the operands is (128 + 2 N) fp32 for 768 N flop.
constexpr int GK = 32, GLD = GK + 8;
__global__ __launch_bounds__(256, 2) void gemm_tn_bf16x3_gather_kernel(int N, long K, const float* __restrict__ A,
                                                                       long lda, const float* __restrict__ B1,
                                                                       const float* __restrict__ B2, long ldb,
                                                                       float* __restrict__ out, long ldo) {
  __shared__ __attribute__((aligned(16))) uint16_t Ah[SB][GLD], Al[SB][GLD], Bh[SB][GLD], Bl[SB][GLD];
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6, wm = wave >> 1, wn = wave & 1;
  const long j0 = long(blockIdx.x) * SB;
  const long slices = (K + GK - 1) / GK;
  const long s0 = slices * blockIdx.y / gridDim.y, s1 = slices * (blockIdx.y + 1) / gridDim.y;
  // staging task of this thread: operand, 4 rows at rg * 4, 8 k at kg * 8 of the slice
  const bool isB = t >= 128;
  const int rg = t & 31, kg = (t >> 5) & 3;
  const long r0 = (isB ? j0 : 0) + rg * 4;
  const bool in_range = isB ? r0 + 3 < N : true;
  float4 g1[8], g2[8];
  auto fetch = [&](long slice) {
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) {
      const long k = slice * GK + kg * 8 + kk;
      g1[kk] = g2[kk] = float4{0.f, 0.f, 0.f, 0.f};
      if (k < K && in_range) {
        if (!isB) {
          g1[kk] = *reinterpret_cast<const float4*>(A + k * lda + r0);
        } else {
          g1[kk] = *reinterpret_cast<const float4*>(B1 + k * ldb + r0);
          g2[kk] = *reinterpret_cast<const float4*>(B2 + k * ldb + r0);
        }
      }
    }
  };
  floatx16 acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;
  const int kq = 8 * (lane >> 5), rl = lane & 31;
  if (s0 < s1) fetch(s0);
  for (long sl = s0; sl < s1; ++sl) {
#pragma unroll
    for (int ii = 0; ii < 4; ++ii) {
      uint32_t hi[4], lo[4];
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const float a = (&g1[2 * p].x)[ii] - (&g2[2 * p].x)[ii], b = (&g1[2 * p + 1].x)[ii] - (&g2[2 * p + 1].x)[ii];
        const uint32_t ha = bf16_rne_bits(a), hb = bf16_rne_bits(b);
        const uint32_t la = bf16_rne_bits(a - __uint_as_float(ha << 16)), lb = bf16_rne_bits(b - __uint_as_float(hb << 16));
        hi[p] = ha | (hb << 16);
        lo[p] = la | (lb << 16);
      }
      uint16_t* dh = isB ? &Bh[rg * 4 + ii][kg * 8] : &Ah[rg * 4 + ii][kg * 8];
      uint16_t* dl = isB ? &Bl[rg * 4 + ii][kg * 8] : &Al[rg * 4 + ii][kg * 8];
      *reinterpret_cast<uint4*>(dh) = uint4{hi[0], hi[1], hi[2], hi[3]};
      *reinterpret_cast<uint4*>(dl) = uint4{lo[0], lo[1], lo[2], lo[3]};
    }
    __syncthreads();
    if (sl + 1 < s1) fetch(sl + 1);
#pragma unroll
    for (int ks = 0; ks < GK / 16; ++ks) {
      bf16x8 ah[2], al[2], bh[2], bl[2];
#pragma unroll
      for (int mi = 0; mi < 2; ++mi) {
        const int r = wm * 64 + mi * 32 + rl;
        ah[mi] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(&Ah[r][ks * 16 + kq]));
        al[mi] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(&Al[r][ks * 16 + kq]));
      }
#pragma unroll
      for (int ni = 0; ni < 2; ++ni) {
        const int r = wn * 64 + ni * 32 + rl;
        bh[ni] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(&Bh[r][ks * 16 + kq]));
        bl[ni] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(&Bl[r][ks * 16 + kq]));
      }
#pragma unroll
      for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) {
          acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al[mi], bh[ni], acc[mi][ni], 0, 0, 0);
          acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah[mi], bl[ni], acc[mi][ni], 0, 0, 0);
          acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah[mi], bh[ni], acc[mi][ni], 0, 0, 0);
        }
    }
    __syncthreads();
  }
  // accumulator element v of a lane: row (v % 4) + 8 (v / 4) + 4 (lane / 32), column lane % 32 of the 32x32 tile
  float* o = out + long(blockIdx.y) * SB * ldo;
#pragma unroll
  for (int mi = 0; mi < 2; ++mi)
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const long gi = wm * 64 + mi * 32 + (v & 3) + 8 * (v >> 2) + 4 * (lane >> 5);
        const long gj = j0 + wn * 64 + ni * 32 + rl;
        if (gj < N) o[gi * ldo + gj] = acc[mi][ni][v];
      }
}

__global__ void sum_splits_f32_kernel(const float* __restrict__ part, int splits, long count, float* __restrict__ P) {
  const long i = long(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= count) return;
  float s = part[i];
  for (int k = 1; k < splits; ++k) s += part[long(k) * count + i];
  P[i] = s;
}

}  // namespace

int gemm_splitk_splits(long K, int N, int slots) {
  // The workgroups of a gather take the workgroup slots that the chain's last Viterbi launch has just left (`slots`
  // of them, half of the chip with two chains), so the number of splits is chosen to fill whole rounds of those
  // slots: the smallest count that fills at least 95 % of the rounds it needs, else the best there is; a split has
  // at least 512 rows of K.  m = 12288 in two chains: 48 column tiles x 8 splits = 384 workgroups on 384 slots.
  const long tiles = (N + BN - 1) / BN, most = std::min<long>(kMaxGatherSplits, std::max<long>(1, K / 512));
  long best = 1;
  double best_fill = 0;
  for (long s = 1; s <= most; ++s) {
    const long wgs = tiles * s, rounds = (wgs + slots - 1) / slots;
    const double fill = double(wgs) / double(rounds * slots);
    if (fill > best_fill + 1e-9) best = s, best_fill = fill;
    if (fill >= 0.95) return int(s);
  }
  return int(best);
}

void launch_gemm_tn_f64_gather(int N, long K, const float* A, long lda, const float* B1, const float* B2, long ldb,
                               double* P, double* partials, int slots, hipStream_t s) {
  QTIP_REQUIRE(N >= 4 && K > 0 && K % KC == 0 && N % 4 == 0 && lda % 4 == 0 && ldb % 4 == 0 && B2 != nullptr,
               "fp64 gather GEMM needs 16-byte aligned fp32 rows and K %% 16 == 0");
  const int S = gemm_splitk_splits(K, N, slots);
  dim3 grid(unsigned((N + BN - 1) / BN), unsigned(S));
  gemm_tn_f64_splitk_kernel<<<grid, dim3(256), 0, s>>>(N, K, A, lda, B1, B2, ldb, S == 1 ? P : partials, N);
  QTIP_HIP(hipGetLastError());
  if (S > 1) {
    const long count = long(BM) * N;
    sum_splits_kernel<<<dim3(unsigned((count + 255) / 256)), dim3(256), 0, s>>>(partials, S, count, P);
    QTIP_HIP(hipGetLastError());
  }
}

void launch_gemm_tn_bf16x3_gather(int N, long K, const float* A, long lda, const float* B1, const float* B2, long ldb,
                                  float* P, float* partials, int slots, hipStream_t s) {
  QTIP_REQUIRE(N > 0 && K > 0 && N % 4 == 0 && lda % 4 == 0 && ldb % 4 == 0 && B2 != nullptr,
               "split-bf16 gather GEMM needs 16-byte aligned fp32 rows");
  const int S = gemm_splitk_splits(K, N, slots);
  dim3 grid(unsigned((N + SB - 1) / SB), unsigned(S));
  gemm_tn_bf16x3_gather_kernel<<<grid, dim3(256), 0, s>>>(N, K, A, lda, B1, B2, ldb, S == 1 ? P : partials, N);
  QTIP_HIP(hipGetLastError());
  if (S > 1) {
    const long count = long(SB) * N;
    sum_splits_f32_kernel<<<dim3(unsigned((count + 255) / 256)), dim3(256), 0, s>>>(partials, S, count, P);
    QTIP_HIP(hipGetLastError());
  }
}

}  // namespace qtipmi
