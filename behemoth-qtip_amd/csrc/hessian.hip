// Hessian accumulation, the step that feeds the group quantizer: H (n x n fp32) += X^T X for a batch X of `rows`
// activation vectors (rows x n bf16, row-major).  Reference: the hess() lambda of LayerRunner::forward_batch,
// src/model.cpp:352-363 (a bf16 GEMM with fp32 accumulation over the 10 blocks bi <= bj of a 4 x 4 partition),
// symmetrize_hess / k_symmetrize_blocks (src/model.cpp:260-264, src/kernels.hip:465-474) and the division by the
// token count (src/pipeline.cpp:160-166).
//
// A symmetric rank-`rows` update on the bf16 matrix cores (v_mfma_f32_32x32x16_bf16, fp32 accumulate).  Only the
// 256 x 256 tiles on or below the diagonal are computed (50.4 % of the square at n = 28672, against 62.5 % for the
// 4 x 4 block schedule); hessian_finish mirrors them into the other triangle and scales.
//
// One 256-thread workgroup per tile, one workgroup per CU: a wave owns 128 x 128 outputs (4 x 4 MFMA tiles, 256
// accumulator registers).  Both operands are column slices of X and the contraction runs over the rows of X, so the
// matrix cores want, per lane, 8 consecutive rows of one column, while memory has the columns contiguous.  The batch
// is therefore first rewritten (batch_image_kernel, one pass over it) as the LDS images of the update kernel's stages,
// and the update kernel (syrk_img_kernel, which the proxy's quadratic forms use as well) moves them from global memory
// straight into LDS.  Workgroups are numbered so that the 32 that share an XCD (and its L2) at a time form an 8 x 4
// patch of tiles, which needs 12 operand slices instead of 33.
#include <mutex>
#include <type_traits>
#include <vector>

#include "misc.hpp"
#include "qtip_internal.hpp"

namespace qtipmi {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kTile = 256;    // output tile edge
constexpr int kPatchRows = 8, kPatchCols = 4;             // tiles per XCD patch

// The operands of the update kernel are written (batch_image_kernel for a Hessian batch, split_image_kernel for the
// proxy's quadratic forms) as the LDS images of its stages: [stage of 32 rows of K][column tile of 256][column][32 k], the four 16-byte
// pieces of a column at position p ^ ((column >> 2) & 3) (free of bank conflicts for the 16-byte fragment reads: the
// 16 lanes the LDS serves together then touch 16 different 16-byte bank groups).  A stage of an operand is 16 KB of
// contiguous global memory and goes straight into LDS (global_load_lds_dwordx4, 1 KB per wave and instruction): no
// staging registers, no transposes, no LDS writes by the waves.  Four stages of LDS; the loads run three stages ahead
// of the matrix cores, and a wave fetches the fragments of the next 16 k while the 16 MFMAs of the present ones run,
// every fragment read and every load in the shadow of an MFMA of its own.
constexpr int IK = 32, ISTAGES = 4;
constexpr int kImgSliceU16 = kTile * IK;                                  // one operand slice of a stage, 16 KB
constexpr size_t kImgLdsBytes = size_t(ISTAGES) * 2 * kImgSliceU16 * 2;   // 128 KB

__host__ __device__ inline size_t img_index(long k, long c, long tiles) {
  const long st = k / IK, p = (k % IK) >> 3, T = c / kTile, col = c % kTile;
  return (size_t(st * tiles + T) * kTile + size_t(col)) * IK + size_t((p ^ ((col >> 2) & 3)) * 8 + (k & 7));
}

template <bool DOT>
__global__ __launch_bounds__(256, 1) void syrk_img_kernel(const uint16_t* __restrict__ IA, const uint16_t* __restrict__ IB,
                                                         int stages, long n, float* __restrict__ H,
                                                         double* __restrict__ partial, int tiles, int patch_cols) {
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
  const long b = blockIdx.x;
  const long xcd = b & 7, local = b >> 3;
  const long patch = (local / (kPatchRows * kPatchCols)) * 8 + xcd, within = local % (kPatchRows * kPatchCols);
  const long ti = (patch / patch_cols) * kPatchRows + within / kPatchCols;
  const long tj = (patch % patch_cols) * kPatchCols + within % kPatchCols;
  if (ti >= tiles || tj > ti) return;  // outside the matrix or above the diagonal
  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);  // uniform: the LDS addresses of the loads stay scalar
  const int wm = wave >> 1, wn = wave & 1;
  const int rl = lane & 31;

  floatx16 acc[4][4];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][c][v] = 0.f;
  {
    // the accumulators enter the loop as results of a matrix instruction: they live in the accumulation registers
    bf16x8 z;
#pragma unroll
    for (int e = 0; e < 8; ++e) z[e] = __bf16(0.f);
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[a][c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(z, z, acc[a][c], 0, 0, 0);
  }

  // wave w brings the 1 KB chunks 4 w .. 4 w + 3 of both operand slices of a stage, 16 bytes per lane.  pa / pb: this
  // lane's piece of operand A's / B's slice of stage sa / sb, the stage whose loads are requested next (a quarter of a
  // slice per instruction: one address and one LDS base per operand and stage, the quarter in the immediate offset)
  const size_t stage_stride = size_t(tiles) * kImgSliceU16;
  const uint16_t* pa = IA + size_t(ti) * kImgSliceU16 + (wave * 4) * 512 + lane * 8;
  const uint16_t* pb = IB + size_t(tj) * kImgSliceU16 + (wave * 4) * 512 + lane * 8;
  int sa = 0, sb = 0;
  typedef __attribute__((address_space(3))) void* lds_ptr;
#define QTIP_LOAD_A(q) \
  __builtin_amdgcn_global_load_lds(pa, (lds_ptr)(lds + (sa % ISTAGES) * 2 * kImgSliceU16 + (wave * 4) * 512), 16, (q) * 1024, 0)
#define QTIP_LOAD_B(q)                                                                                                  \
  __builtin_amdgcn_global_load_lds(pb, (lds_ptr)(lds + (sb % ISTAGES) * 2 * kImgSliceU16 + kImgSliceU16 + (wave * 4) * 512), \
                                   16, (q) * 1024, 0)
  auto request_a = [&] { QTIP_LOAD_A(0); QTIP_LOAD_A(1); QTIP_LOAD_A(2); QTIP_LOAD_A(3); pa += stage_stride; ++sa; };
  auto request_b = [&] { QTIP_LOAD_B(0); QTIP_LOAD_B(1); QTIP_LOAD_B(2); QTIP_LOAD_B(3); pb += stage_stride; ++sb; };
  // fragment of 8 k (piece 2 ks + lane / 32) of column wX * 128 + 32 i + rl.  read1 fetches fragment j of a step in the
  // order its MFMAs first use them: a0 b0 b1 b2 b3 a1 a2 a3
  const int offA = (wm * 128 + rl) * IK, offB = (wn * 128 + rl) * IK, sw = (rl >> 2) & 3, hi = lane >> 5;
  bf16x8 fa[2][4], fb[2][4];
  auto read1 = [&](int st, int ks, int set, int j) {
    const uint16_t* As = lds + (st % ISTAGES) * 2 * kImgSliceU16;
    const int piece = ((2 * ks + hi) ^ sw) << 3;
    if (j == 0 || j >= 5) {
      const int i = j == 0 ? 0 : j - 4;
      fa[set][i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(As + offA + i * 32 * IK + piece));
    } else {
      const int i = j - 1;
      fb[set][i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(As + kImgSliceU16 + offB + i * 32 * IK + piece));
    }
  };
  auto mfma = [&](int set, int j) {  // MFMA j of a step: row tile j / 4, column tile j % 4
    const int mi = j >> 2, ni = j & 3;
    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[set][mi], fb[set][ni], acc[mi][ni], 0, 0, 0);
  };

  // Stages 0..2 requested, stage 0 landed (this wave's loads, then everyone's: a bare barrier, which does not wait
  // for the loads still in flight), operand A of stage 3 requested, the fragments of stage 0's first 16 k read.
  const int pre = stages < ISTAGES - 1 ? stages : ISTAGES - 1;
  for (int p = 0; p < pre; ++p) request_a(), request_b();
  if (pre >= 3) __builtin_amdgcn_s_waitcnt(0x4F70);       // vmcnt(16)
  else if (pre == 2) __builtin_amdgcn_s_waitcnt(0x0F78);  // vmcnt(8)
  else __builtin_amdgcn_s_waitcnt(0x0F70);                // vmcnt(0)
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  if (sa < stages) request_a();
#pragma unroll
  for (int j = 0; j < 8; ++j) read1(0, 0, 0, j);

  // One stage: 32 MFMAs, two steps of 16 k on fragment sets 0 and 1.  A wave has nothing to hide a wait behind but
  // its own MFMAs (one wave per SIMD), and an MFMA keeps the matrix core busy for 32 cycles while the wave may issue
  // other work: so no two memory instructions follow each other.  Under every other MFMA of a step the wave reads one
  // fragment of the next step, and under MFMAs 1, 5, 9, 13 it requests a quarter of an operand slice three stages
  // ahead: operand B of stage st + 3 during step 0, then - after the barrier that says stage st + 1 has landed
  // everywhere and every wave has asked for its last fragments of stage st, whose buffer is therefore free - operand
  // A of stage st + 4 during step 1.  (The same instructions in bursts - 8 fragment reads, then 8 MFMAs, 8 loads
  // after the barrier - left the matrix cores idle for a quarter of the loop.)  The scheduling barriers pin the order.
  // kSteady: every stage asked for exists and two stages beyond st + 1 are on their way, so vmcnt(16) = "stage
  // st + 1 is here"; the last stages run the same code with the conditions and a full wait.
#define QTIP_SB __builtin_amdgcn_sched_barrier(0)
  auto stage = [&](auto steady, int st) {
    constexpr bool kSteady = decltype(steady)::value;
    const bool next = kSteady || st + 1 < stages;
    {
      const bool go = kSteady || sb < stages;
#define QTIP_M0(j) { mfma(0, j); QTIP_SB; }
#define QTIP_R0(j) { mfma(0, j); QTIP_SB; read1(st, 1, 1, (j) / 2); QTIP_SB; }
#define QTIP_L0(j) { mfma(0, j); QTIP_SB; if (go) QTIP_LOAD_B(((j) - 1) / 4); QTIP_SB; }
      QTIP_SB;
      QTIP_R0(0) QTIP_L0(1) QTIP_R0(2) QTIP_M0(3) QTIP_R0(4) QTIP_L0(5) QTIP_R0(6) QTIP_M0(7)
      QTIP_R0(8) QTIP_L0(9) QTIP_R0(10) QTIP_M0(11) QTIP_R0(12) QTIP_L0(13) QTIP_R0(14) QTIP_M0(15)
      if (go) pb += stage_stride, ++sb;
    }
    if (next) {
      if (kSteady) __builtin_amdgcn_s_waitcnt(0x4F70);  // vmcnt(16)
      else __builtin_amdgcn_s_waitcnt(0x0F70);          // vmcnt(0)
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
    }
    {
      const bool go = kSteady || sa < stages;
#define QTIP_M1(j) { mfma(1, j); QTIP_SB; }
#define QTIP_R1(j) { mfma(1, j); QTIP_SB; if (next) read1(st + 1, 0, 0, (j) / 2); QTIP_SB; }
#define QTIP_L1(j) { mfma(1, j); QTIP_SB; if (go) QTIP_LOAD_A(((j) - 1) / 4); QTIP_SB; }
      QTIP_SB;
      QTIP_R1(0) QTIP_L1(1) QTIP_R1(2) QTIP_M1(3) QTIP_R1(4) QTIP_L1(5) QTIP_R1(6) QTIP_M1(7)
      QTIP_R1(8) QTIP_L1(9) QTIP_R1(10) QTIP_M1(11) QTIP_R1(12) QTIP_L1(13) QTIP_R1(14) QTIP_M1(15)
      if (go) pa += stage_stride, ++sa;
    }
  };
  int st = 0;
  for (; st + 4 < stages; ++st) stage(std::true_type{}, st);
  for (; st < stages; ++st) stage(std::false_type{}, st);
#undef QTIP_M0
#undef QTIP_R0
#undef QTIP_L0
#undef QTIP_M1
#undef QTIP_R1
#undef QTIP_L1
#undef QTIP_SB
#undef QTIP_LOAD_A
#undef QTIP_LOAD_B
  __syncthreads();

  // accumulator element v of a lane: row (v % 4) + 8 (v / 4) + 4 (lane / 32), column lane % 32 of the 32 x 32 tile
  double dot = 0.0;
  if ((ti + 1) * kTile <= n && (tj + 1) * kTile <= n) {
    // (the lane number is taken anew: nothing of the addresses below then has to live through the loop above)
    const int ln = int(__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)));
    float* hb = H + (ti * kTile + wm * 128 + 4 * (ln >> 5)) * n + tj * kTile + wn * 128 + (ln & 31);
    // The 16 values of H that go with a 32 x 32 accumulator are fetched together (one predicated load at a time
    // would be 256 dependent round trips to HBM per tile), and in the accumulating form one accumulator ahead of the
    // one being added to: a lone wave per SIMD has nothing else to cover the 16 round trips with, and a batch of 8192
    // rows is only 256 stages of work per tile.  (The proxy's form has 4.5 times the stages and 64-bit sums to hold.
    // Larger batches - a row of four accumulators, or two accumulators ahead - do not fit the registers.)
    constexpr int kAheadH = DOT ? 0 : 1;
    float h[kAheadH + 1][16];
    auto fetch_h = [&](int blk) {
      const int mi = blk >> 2, ni = blk & 3;
#pragma unroll
      for (int v = 0; v < 16; ++v) h[blk % (kAheadH + 1)][v] = hb[long(mi * 32 + (v & 3) + 8 * (v >> 2)) * n + ni * 32];
    };
    if (kAheadH) fetch_h(0);
#pragma unroll
    for (int blk = 0; blk < 16; ++blk) {
      const int mi = blk >> 2, ni = blk & 3;
      __builtin_amdgcn_sched_barrier(0);
      if (blk + kAheadH < 16) fetch_h(blk + kAheadH);
      __builtin_amdgcn_sched_barrier(0);  // all 16 loads are issued before a value (of this or an earlier fetch) is used
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        if (DOT) dot += double(acc[mi][ni][v]) * double(h[blk % (kAheadH + 1)][v]);
        else hb[long(mi * 32 + (v & 3) + 8 * (v >> 2)) * n + ni * 32] = h[blk % (kAheadH + 1)][v] + acc[mi][ni][v];
      }
    }
  } else {
#pragma unroll
    for (int mi = 0; mi < 4; ++mi)
#pragma unroll
      for (int ni = 0; ni < 4; ++ni)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const long gi = ti * kTile + wm * 128 + mi * 32 + (v & 3) + 8 * (v >> 2) + 4 * (lane >> 5);
          const long gj = tj * kTile + wn * 128 + ni * 32 + rl;
          if (gi < n && gj < n) {
            if (DOT) dot += double(acc[mi][ni][v]) * double(H[gi * n + gj]);
            else H[gi * n + gj] += acc[mi][ni][v];
          }
        }
  }
  if (DOT) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) dot += __shfl_xor(dot, off, 64);
    double* red = reinterpret_cast<double*>(lds);
    if (lane == 0) red[wave] = dot;
    __syncthreads();
    if (t == 0) partial[ti * tiles + tj] = (ti == tj ? 1.0 : 2.0) * (((red[0] + red[1]) + red[2]) + red[3]);
  }
}

// The batch of a Hessian accumulation (rows x n bf16, row-major) as the stage images of syrk_img_kernel: one workgroup
// per stage of 32 rows and tile of 256 columns brings the 32 x 256 block in with 16-byte loads (zeros beyond the
// matrix), turns it in LDS and writes each column's 32 values as the four swizzled 16-byte pieces of its image: 16 KB
// of contiguous global memory per workgroup.
__global__ __launch_bounds__(256) void batch_image_kernel(const uint16_t* __restrict__ X, long rows, long n, int tiles,
                                                          uint16_t* __restrict__ I) {
  __shared__ __attribute__((aligned(16))) uint16_t blk[IK][kTile + 8];
  const long st = blockIdx.y, T = blockIdx.x;
  const int t = threadIdx.x;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int idx = t + 256 * i, r = idx >> 5, c8 = idx & 31;
    const long gr = st * IK + r, gc = T * kTile + 8 * c8;
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    if (gr < rows && gc + 8 <= n) v = *reinterpret_cast<const uint4*>(X + gr * n + gc);
    *reinterpret_cast<uint4*>(&blk[r][8 * c8]) = v;
  }
  __syncthreads();
  uint16_t* out = I + (size_t(st) * tiles + size_t(T)) * kImgSliceU16 + size_t(t) * IK;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    uint32_t w[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) w[e] = uint32_t(blk[8 * p + 2 * e][t]) | (uint32_t(blk[8 * p + 2 * e + 1][t]) << 16);
    *reinterpret_cast<uint4*>(out + ((p ^ ((t >> 2) & 3)) << 3)) = make_uint4(w[0], w[1], w[2], w[3]);
  }
}

__device__ __forceinline__ uint16_t f32_to_bf16_dev(float f) {  // round to nearest even; the inputs here are finite
  uint32_t u = __float_as_uint(f);
  u += 0x7fffu + ((u >> 16) & 1u);
  return uint16_t(u >> 16);
}

// X[r][c] = A[c][r] - (B ? B[c][r] : 0) for r < m, c < n (A, B: n x m with leading dimension ld), split into bf16 hi + lo
// and written as the stage images (img_index) of the two operand stacks of the three-product form, XA = [hi; hi; lo]
// and XB = [hi; lo; hi], so that XA^T XB = hi^T hi + hi^T lo + lo^T hi.  Every segment is padded with zero rows to mp
// (a multiple of 32) and the columns with zeros to tiles x 256.  A thread takes 8 consecutive r of one column: one
// 16-byte piece of each segment of each image; the rows of A run along r, so no transpose is needed.
__global__ __launch_bounds__(256) void split_image_kernel(const float* __restrict__ A, const float* __restrict__ B, long n,
                                                          long m, long ld, long mp, long tiles, uint16_t* __restrict__ IA,
                                                          uint16_t* __restrict__ IB) {
  const long pieces = mp / 8, idx = long(blockIdx.x) * 256 + threadIdx.x;
  const long c = idx / pieces, r0 = (idx % pieces) * 8;
  if (c >= tiles * kTile) return;
  uint32_t h[4], l[4];
#pragma unroll
  for (int e = 0; e < 8; e += 2) {
    uint16_t hh[2], ll[2];
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const long r = r0 + e + q;
      float v = 0.f;
      if (c < n && r < m) v = A[c * ld + r] - (B ? B[c * ld + r] : 0.f);
      hh[q] = f32_to_bf16_dev(v);
      ll[q] = f32_to_bf16_dev(v - __uint_as_float(uint32_t(hh[q]) << 16));
    }
    h[e >> 1] = uint32_t(hh[0]) | (uint32_t(hh[1]) << 16);
    l[e >> 1] = uint32_t(ll[0]) | (uint32_t(ll[1]) << 16);
  }
  const uint4 hi = {h[0], h[1], h[2], h[3]}, lo = {l[0], l[1], l[2], l[3]};
  *reinterpret_cast<uint4*>(IA + img_index(r0, c, tiles)) = hi;
  *reinterpret_cast<uint4*>(IA + img_index(mp + r0, c, tiles)) = hi;
  *reinterpret_cast<uint4*>(IA + img_index(2 * mp + r0, c, tiles)) = lo;
  *reinterpret_cast<uint4*>(IB + img_index(r0, c, tiles)) = hi;
  *reinterpret_cast<uint4*>(IB + img_index(mp + r0, c, tiles)) = lo;
  *reinterpret_cast<uint4*>(IB + img_index(2 * mp + r0, c, tiles)) = hi;
}

__global__ __launch_bounds__(256) void sum_doubles_kernel(const double* __restrict__ p, long count, double* __restrict__ out) {
  __shared__ double red[256];
  double a = 0.0;
  for (long i = threadIdx.x; i < count; i += 256) a += p[i];
  red[threadIdx.x] = a;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if (int(threadIdx.x) < w) red[threadIdx.x] += red[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) *out = red[0];
}

// H[i][j] for j > i takes H[j][i] (computed tiles hold the lower triangle and the whole diagonal tiles); everything
// is scaled.  32 x 32 patches through LDS so both the read and the write are row segments.
__global__ __launch_bounds__(256) void hessian_finish_kernel(float* __restrict__ H, long n, float scale) {
  __shared__ float tile[32][33];
  const long bi = blockIdx.y, bj = blockIdx.x;
  if (bj > bi) return;  // the patch pair (bi, bj), (bj, bi) is handled by the lower one
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const long i = bi * 32 + ty + 8 * k, j = bj * 32 + tx;
    float v = 0.f;
    if (i < n && j < n) {
      v = H[i * n + j] * scale;
      if (bi != bj || j <= i) H[i * n + j] = v;
    }
    tile[ty + 8 * k][tx] = v;
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const long i = bj * 32 + ty + 8 * k, j = bi * 32 + tx;  // element (i, j) of the mirrored patch = lower (j, i)
    if (i < n && j < n && (bi != bj || j > i)) H[i * n + j] = tile[tx][ty + 8 * k];
  }
}

}  // namespace

namespace {
// launch geometry shared by the two forms of the kernel; also raises the kernels' dynamic LDS limit, once for every
// device the library is used on (the attribute is kept per device) and safe against concurrent first calls
struct SyrkGrid {
  int tiles, patch_cols;
  unsigned grid;
  explicit SyrkGrid(long n) {
    static std::mutex mu;
    static std::vector<bool> configured;
    int dev = 0;
    QTIP_HIP(hipGetDevice(&dev));
    {
      std::lock_guard<std::mutex> lk(mu);
      if (configured.size() <= size_t(dev)) configured.resize(size_t(dev) + 1, false);
      if (!configured[size_t(dev)]) {
        QTIP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(syrk_img_kernel<true>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, int(kImgLdsBytes)));
        QTIP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(syrk_img_kernel<false>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, int(kImgLdsBytes)));
        configured[size_t(dev)] = true;
      }
    }
    tiles = int((n + kTile - 1) / kTile);
    const int patch_rows = (tiles + kPatchRows - 1) / kPatchRows;
    patch_cols = (tiles + kPatchCols - 1) / kPatchCols;
    const long patches = long(patch_rows) * patch_cols;
    const long padded = (patches + 7) / 8 * 8;  // whole rounds over the 8 XCDs
    const long g = padded * kPatchRows * kPatchCols;
    QTIP_REQUIRE(g < (1l << 31), "symmetric update: n too large (%ld)", n);
    grid = unsigned(g);
  }
};
}  // namespace

void launch_hessian_accumulate(const uint16_t* X, long rows, long n, float* H, DBuf<uint16_t>& image, hipStream_t s) {
  QTIP_REQUIRE(X != nullptr && H != nullptr && rows >= 0 && n > 0, "hessian_accumulate: bad arguments");
  QTIP_REQUIRE(n % 8 == 0 && (reinterpret_cast<uintptr_t>(X) & 15) == 0, "hessian_accumulate: rows of X must be 16-byte aligned (n = %ld)", n);
  if (rows == 0) return;
  SyrkGrid g(n);
  // the batch is first written as the LDS images of the update kernel's stages (a pass over the batch, 4 % of the
  // update's time), which then feeds its matrix cores with direct global-to-LDS loads; both operands are the batch
  const long stages = (rows + IK - 1) / IK;
  QTIP_REQUIRE(stages <= 65535, "hessian_accumulate: at most %d rows per call (rows = %ld)", 65535 * IK, rows);
  image.ensure(size_t(stages) * size_t(g.tiles) * kImgSliceU16);
  batch_image_kernel<<<dim3(unsigned(g.tiles), unsigned(stages)), dim3(256), 0, s>>>(X, rows, n, g.tiles, image.p);
  QTIP_HIP(hipGetLastError());
  syrk_img_kernel<false><<<dim3(g.grid), dim3(256), kImgLdsBytes, s>>>(image.p, image.p, int(stages), n, H, nullptr,
                                                                      g.tiles, g.patch_cols);
  QTIP_HIP(hipGetLastError());
}

// sum_ij H_ij (D^T D)_ij = tr(D H D^T) for D = A^T - B^T (m x n), H symmetric n x n fp32: the quadratic forms of the
// proxy (src/quantizer.cpp:268-303, which also takes them from bf16 hi/lo products with fp32 accumulation).
// A, B: n x m fp32 with leading dimension ld (B may be null).  Synchronises the stream.
double quad_trace_bf16x3(long n, long m, const float* H, const float* A, const float* B, long ld, DBuf<uint16_t>& stack,
                         DBuf<double>& scratch, hipStream_t s) {
  if (n <= 0 || m <= 0) return 0.0;
  QTIP_REQUIRE(n % 8 == 0, "proxy: n must be a multiple of 8 (n = %ld)", n);
  SyrkGrid g(n);
  const long mp = (m + IK - 1) / IK * IK, tiles = g.tiles;
  const size_t img = size_t(3 * mp) * size_t(tiles) * kTile;  // one operand stack as stage images
  stack.ensure(2 * img);
  uint16_t* IA = stack.p;
  uint16_t* IB = stack.p + img;
  const long threads = tiles * kTile * (mp / 8);
  split_image_kernel<<<dim3(unsigned((threads + 255) / 256)), dim3(256), 0, s>>>(A, B, n, m, ld, mp, tiles, IA, IB);
  QTIP_HIP(hipGetLastError());
  const size_t np = size_t(g.tiles) * g.tiles;
  scratch.ensure(np + 1);
  QTIP_HIP(hipMemsetAsync(scratch.p, 0, np * sizeof(double), s));
  syrk_img_kernel<true><<<dim3(g.grid), dim3(256), kImgLdsBytes, s>>>(IA, IB, int(3 * mp / IK), n, const_cast<float*>(H),
                                                                     scratch.p, g.tiles, g.patch_cols);
  QTIP_HIP(hipGetLastError());
  sum_doubles_kernel<<<dim3(1), dim3(256), 0, s>>>(scratch.p, long(np), scratch.p + np);
  QTIP_HIP(hipGetLastError());
  double h = 0;
  QTIP_HIP(hipMemcpyAsync(&h, scratch.p + np, sizeof(double), hipMemcpyDeviceToHost, s));
  QTIP_HIP(hipStreamSynchronize(s));
  return h;
}

void launch_hessian_finish(float* H, long n, float scale, hipStream_t s) {
  QTIP_REQUIRE(H != nullptr && n > 0, "hessian_finish: bad arguments");
  const unsigned nb = unsigned((n + 31) / 32);
  hessian_finish_kernel<<<dim3(nb, nb), dim3(256), 0, s>>>(H, n, scale);
  QTIP_HIP(hipGetLastError());
}

}  // namespace qtipmi
