// Cross-buffer feedback of LDLQ for gfx950 (reference: ldlq_gpu, src/quantizer.cpp:30-89; the CPU form of the
// algorithm, tests/test_gpu.cpp:180-225).  The in-buffer feedback of a 16-column block is formed inside the Viterbi
// kernel (viterbi.hip, tile_targets).
//
//  * gemm_tn: sum_k A[k][i] * (B1 - B2)[k][j] on the fp64 matrix cores (v_mfma_f64_16x16x4_f64), fp32 operands
//    widened while staging through LDS.  The cross-buffer feedback ("prod cache") of a 128-column buffer is gathered
//    from all rows quantized so far by a K-split kernel.
//  * gather_img: the same gathered product in the arithmetic of the reference's GPU path: every fp32 operand held
//    as bf16 hi + lo images (L's made once per group, the residual's written by the Viterbi kernel as it decodes),
//    three v_mfma_f32_32x32x16_bf16 terms, fp32 accumulation.
#include <algorithm>

#include "bf16_split.hpp"
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

// Th[i][k], Tl[i][k] = the bf16 hi and lo parts of x = X[k][i] (or X[k][i] - X2[k][i]): x = hi + lo + O(2^-16 x),
// hi = bf16(x), lo = bf16(x - hi), in tiles of 64 x 64 through LDS: the transposed images that the gathered product
// reads with k contiguous.  lower_only: tiles wholly above the diagonal (k + 63 < i) are left alone; nothing reads
// them when X is L.
__global__ __launch_bounds__(256) void split_transpose_bf16_kernel(const float* __restrict__ X,
                                                                   const float* __restrict__ X2, long ldx,
                                                                   uint16_t* __restrict__ Th,
                                                                   uint16_t* __restrict__ Tl, long ldt,
                                                                   int lower_only) {
  __shared__ float T[64][65];
  const long k0 = long(blockIdx.y) * 64, i0 = long(blockIdx.x) * 64;
  if (lower_only && k0 + 64 <= i0) return;
  const int t = threadIdx.x;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int row = (t >> 4) + 16 * p, col = 4 * (t & 15);
    float4 v = *reinterpret_cast<const float4*>(X + (k0 + row) * ldx + i0 + col);
    if (X2) {
      const float4 w = *reinterpret_cast<const float4*>(X2 + (k0 + row) * ldx + i0 + col);
      v.x -= w.x, v.y -= w.y, v.z -= w.z, v.w -= w.w;
    }
    T[row][col] = v.x, T[row][col + 1] = v.y, T[row][col + 2] = v.z, T[row][col + 3] = v.w;
  }
  __syncthreads();
  const int i = t >> 2, kc = 16 * (t & 3);
  uint32_t hi[8], lo[8];
#pragma unroll
  for (int p = 0; p < 8; ++p) {
    uint32_t ha, la, hb, lb;
    bf16_split_bits(T[kc + 2 * p][i], ha, la);
    bf16_split_bits(T[kc + 2 * p + 1][i], hb, lb);
    hi[p] = ha | (hb << 16);
    lo[p] = la | (lb << 16);
  }
  uint4* dh = reinterpret_cast<uint4*>(Th + (i0 + i) * ldt + k0 + kc);
  uint4* dl = reinterpret_cast<uint4*>(Tl + (i0 + i) * ldt + k0 + kc);
  dh[0] = uint4{hi[0], hi[1], hi[2], hi[3]}, dh[1] = uint4{hi[4], hi[5], hi[6], hi[7]};
  dl[0] = uint4{lo[0], lo[1], lo[2], lo[3]}, dl[1] = uint4{lo[4], lo[5], lo[6], lo[7]};
}

// ---------------------------------------------------------------- bf16 hi/lo split MFMA GEMM, gathered (fp32 accumulate)
// out[y][i][j] = sum over the K slices of split y of a[i][k] * b[j][k], i < 128, where a and b are fp32 values held
// as bf16 hi + lo images with k contiguous (a: the transposed image of L above; b: the image of WT - hatWT that the
// Viterbi kernel writes with every tile it decodes), in the arithmetic of the reference's prod-cache update
// (src/quantizer.cpp:66-76: product = lo*hi + hi*lo + hi*hi on the bf16 matrix cores, fp32 accumulate) but gathered
// like the fp64 kernel above: K is everything quantized so far, nothing is read-modified-written.
// 128 x 128 outputs per workgroup, 4 waves of 64 x 64 (2 x 2 tiles of 32 x 32 of v_mfma_f32_32x32x16_bf16).  A stage
// is 16 k of the four images: 128 rows x 32 bytes each, brought by global_load_lds_dwordx4 (wave w brings image w,
// four instructions of 32 rows) into one of three LDS stages, two in flight ahead of the one in use, one barrier per
// stage.  A lane's operand fragment (row lane % 32, the 8 k at 8 (lane / 32)) is one 16-byte LDS read; the two
// 16-byte halves of a row sit swapped in rows 8..15 of every 16, which spreads the 16 rows that are read together
// over all banks (the swap is made by the lane that fetches the half choosing which half it fetches).  No staging
// registers, no conversion in the loop: 48 KB of LDS and under 128 registers, so that a workgroup fits in the slot
// that a Viterbi workgroup of the same chain has just left.
constexpr int IK = 16, IST = 3;
__global__ __launch_bounds__(256, 3) void gather_img_kernel(int N, long K, const uint16_t* __restrict__ Ah,
                                                            const uint16_t* __restrict__ Al, long lda,
                                                            const uint16_t* __restrict__ Bh,
                                                            const uint16_t* __restrict__ Bl, long ldb,
                                                            float* __restrict__ out, long ldo) {
  __shared__ __attribute__((aligned(16))) uint16_t S[IST][4][SB][IK];  // [stage][Ah | Al | Bh | Bl][row][k]
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6, wm = wave >> 1, wn = wave & 1;
  const long j0 = long(blockIdx.x) * SB;
  const long all = K / IK;  // K is a multiple of 16
  const long sg0 = all * blockIdx.y / gridDim.y, sg1 = all * (blockIdx.y + 1) / gridDim.y;
  const int stages = int(sg1 - sg0);
  // loads of this lane: image `wave`, rows 32 q + lane / 2 (q < 4), the half that belongs at position lane % 2
  const uint16_t* g[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int r = 32 * q + (lane >> 1), half = (lane & 1) ^ ((r >> 3) & 1);
    long row = r;
    if (wave >= 2) row = j0 + r < N ? j0 + r : N - 1;  // rows beyond N only feed outputs that are not stored
    const uint16_t* base = wave == 0 ? Ah : wave == 1 ? Al : wave == 2 ? Bh : Bl;
    g[q] = base + row * (wave < 2 ? lda : ldb) + sg0 * IK + 8 * half;
  }
  typedef __attribute__((address_space(3))) void* lds_ptr;
  auto issue = [&](int stage) {
    const int st = stage % IST;
#pragma unroll
    for (int q = 0; q < 4; ++q)
      __builtin_amdgcn_global_load_lds(g[q] + long(stage) * IK, (lds_ptr)&S[st][wave][32 * q][0], 16, 0, 0);
  };
  floatx16 acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;
  const int rl = lane & 31;
  // fragment positions: row, and the position of the half 8 (lane / 32) in that row
  int fa[2], fb[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int ra = wm * 64 + i * 32 + rl, rb = wn * 64 + i * 32 + rl;
    fa[i] = ra * IK + 8 * ((lane >> 5) ^ ((ra >> 3) & 1));
    fb[i] = rb * IK + 8 * ((lane >> 5) ^ ((rb >> 3) & 1));
  }
  for (int p = 0; p < IST - 1 && p < stages; ++p) issue(p);
  for (int sg = 0; sg < stages; ++sg) {
    // this wave's loads of stage sg have landed when only those of the stage issued after it are outstanding
    // (4 loads per stage; loads return in order)
    if (sg + 1 < stages) __builtin_amdgcn_s_waitcnt(0x0F74);  // vmcnt(4)
    else __builtin_amdgcn_s_waitcnt(0x0F70);                   // vmcnt(0)
    // everyone's have, and everyone is done reading the stage that the next issue overwrites
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (sg + IST - 1 < stages) issue(sg + IST - 1);
    const uint16_t* base = &S[sg % IST][0][0][0];
    bf16x8 ah[2], al[2], bh[2], bl[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      ah[i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(base + fa[i]));
      al[i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(base + SB * IK + fa[i]));
      bh[i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(base + 2 * SB * IK + fb[i]));
      bl[i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(base + 3 * SB * IK + fb[i]));
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

int launch_gemm_tn_f64_gather(int N, long K, const float* A, long lda, const float* B1, const float* B2, long ldb,
                              double* P, double* partials, int slots, hipStream_t s, bool reduce) {
  QTIP_REQUIRE(N >= 4 && K > 0 && K % KC == 0 && N % 4 == 0 && lda % 4 == 0 && ldb % 4 == 0 && B2 != nullptr,
               "fp64 gather GEMM needs 16-byte aligned fp32 rows and K %% 16 == 0");
  const int S = gemm_splitk_splits(K, N, slots);
  dim3 grid(unsigned((N + BN - 1) / BN), unsigned(S));
  gemm_tn_f64_splitk_kernel<<<grid, dim3(256), 0, s>>>(N, K, A, lda, B1, B2, ldb, S == 1 ? P : partials, N);
  QTIP_HIP(hipGetLastError());
  if (S > 1 && reduce) {
    const long count = long(BM) * N;
    sum_splits_kernel<<<dim3(unsigned((count + 255) / 256)), dim3(256), 0, s>>>(partials, S, count, P);
    QTIP_HIP(hipGetLastError());
  }
  return S;
}

void launch_split_transpose_bf16(const float* X, const float* X2, long ldx, long rows_k, long cols_i, uint16_t* Th,
                                 uint16_t* Tl, long ldt, bool lower_only, hipStream_t s) {
  QTIP_REQUIRE(rows_k > 0 && cols_i > 0 && rows_k % 64 == 0 && cols_i % 64 == 0 && ldx % 4 == 0 && ldt % 8 == 0,
               "bf16 images are made in tiles of 64 x 64 from 16-byte aligned rows");
  split_transpose_bf16_kernel<<<dim3(unsigned(cols_i / 64), unsigned(rows_k / 64)), dim3(256), 0, s>>>(
      X, X2, ldx, Th, Tl, ldt, lower_only ? 1 : 0);
  QTIP_HIP(hipGetLastError());
}

int launch_gemm_img_gather(int N, long K, const uint16_t* Ah, const uint16_t* Al, long lda, const uint16_t* Bh,
                           const uint16_t* Bl, long ldb, float* P, float* partials, int slots, hipStream_t s,
                           bool reduce) {
  QTIP_REQUIRE(N > 0 && K > 0 && K % IK == 0 && lda % 8 == 0 && ldb % 8 == 0 && Ah && Al && Bh && Bl,
               "split-bf16 gather GEMM needs K %% 16 == 0 and 16-byte aligned image rows");
  const int S = gemm_splitk_splits(K, N, slots);
  dim3 grid(unsigned((N + SB - 1) / SB), unsigned(S));
  gather_img_kernel<<<grid, dim3(256), 0, s>>>(N, K, Ah, Al, lda, Bh, Bl, ldb, S == 1 ? P : partials, N);
  QTIP_HIP(hipGetLastError());
  if (S > 1 && reduce) {
    const long count = long(SB) * N;
    sum_splits_f32_kernel<<<dim3(unsigned((count + 255) / 256)), dim3(256), 0, s>>>(partials, S, count, P);
    QTIP_HIP(hipGetLastError());
  }
  return S;
}

}  // namespace qtipmi
