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
// matrix cores want, per lane, 8 consecutive rows of one column, while memory has the columns contiguous: every
// thread loads an 8 row x 8 column block (eight 16-byte loads, whole 128-byte lines per wave), transposes it in
// registers (v_perm_b32) and writes eight 16-byte column pieces to LDS ([column][row], 128-byte pitch with the pieces
// XOR-swizzled: conflict-free for the writes and for the lanes' 16-byte fragment reads).  Two LDS stages of 64 rows: the next stage is fetched
// and written while the matrix cores work on the current one.  Workgroups are numbered so that the 32 that share an
// XCD (and its L2) at a time form an 8 x 4 patch of tiles, which needs 12 operand slices instead of 33.
#include <mutex>
#include <vector>

#include "misc.hpp"
#include "qtip_internal.hpp"

namespace qtipmi {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kTile = 256;    // output tile edge
constexpr int kStage = 64;    // rows of X per LDS stage
constexpr int kPitch = 64;    // u16 per LDS row: the 64 rows of X of one stage (128 bytes), 16-byte pieces XOR-swizzled
constexpr int kSliceU16 = kTile * kPitch;                 // one operand slice in LDS
constexpr size_t kLdsBytes = size_t(4) * kSliceU16 * 2;   // 2 stages x (A, B)
constexpr int kPatchRows = 8, kPatchCols = 4;             // tiles per XCD patch

struct Block8x8 {
  uint4 r[8];  // r[q]: 8 consecutive columns of row q
};

// Rows beyond `rows` read as zero (they would add to every output); columns beyond n only feed outputs that are
// never stored, so their address is clamped instead.  FULL: the caller knows that all 8 rows exist.
template <bool FULL>
__device__ __forceinline__ void fetch_block(Block8x8& b, const uint16_t* __restrict__ X, long rows, long n, long row0,
                                            long col0) {
  const long c = col0 + 7 < n ? col0 : 0;
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    if (FULL) {
      b.r[q] = *reinterpret_cast<const uint4*>(X + (row0 + q) * n + c);
    } else {
      const bool ok = row0 + q < rows;
      const uint4 v = *reinterpret_cast<const uint4*>(X + (ok ? row0 + q : 0) * n + c);
      b.r[q] = ok ? v : uint4{0u, 0u, 0u, 0u};
    }
  }
}

// LDS layout of an operand slice: column `col` of X occupies 128 bytes; its 16-byte piece holding rows 8 p .. 8 p + 7 of
// the stage sits at piece position p ^ (col & 7) ^ ((col >> 3) & 7).  The writers of one instruction are 8 lanes with
// the same column offset in 8 neighbouring column groups, the readers 8 lanes on 8 neighbouring columns: both then
// touch 8 different 16-byte bank groups.
//
// column c of the block as 8 consecutive rows (4 dwords), written to piece (sw ^ c) of row c of dst; sw = p ^ (group & 7)
template <int D>
__device__ __forceinline__ void store_chunk_transposed(const Block8x8& b, uint16_t* dst, int sw) {
  const uint32_t w[8] = {D == 0 ? b.r[0].x : D == 1 ? b.r[0].y : D == 2 ? b.r[0].z : b.r[0].w,
                         D == 0 ? b.r[1].x : D == 1 ? b.r[1].y : D == 2 ? b.r[1].z : b.r[1].w,
                         D == 0 ? b.r[2].x : D == 1 ? b.r[2].y : D == 2 ? b.r[2].z : b.r[2].w,
                         D == 0 ? b.r[3].x : D == 1 ? b.r[3].y : D == 2 ? b.r[3].z : b.r[3].w,
                         D == 0 ? b.r[4].x : D == 1 ? b.r[4].y : D == 2 ? b.r[4].z : b.r[4].w,
                         D == 0 ? b.r[5].x : D == 1 ? b.r[5].y : D == 2 ? b.r[5].z : b.r[5].w,
                         D == 0 ? b.r[6].x : D == 1 ? b.r[6].y : D == 2 ? b.r[6].z : b.r[6].w,
                         D == 0 ? b.r[7].x : D == 1 ? b.r[7].y : D == 2 ? b.r[7].z : b.r[7].w};
  uint4 even, odd;  // columns 2 D and 2 D + 1: (row 0, row 1), (2, 3), (4, 5), (6, 7)
  even.x = __builtin_amdgcn_perm(w[1], w[0], 0x05040100u);
  even.y = __builtin_amdgcn_perm(w[3], w[2], 0x05040100u);
  even.z = __builtin_amdgcn_perm(w[5], w[4], 0x05040100u);
  even.w = __builtin_amdgcn_perm(w[7], w[6], 0x05040100u);
  odd.x = __builtin_amdgcn_perm(w[1], w[0], 0x07060302u);
  odd.y = __builtin_amdgcn_perm(w[3], w[2], 0x07060302u);
  odd.z = __builtin_amdgcn_perm(w[5], w[4], 0x07060302u);
  odd.w = __builtin_amdgcn_perm(w[7], w[6], 0x07060302u);
  *reinterpret_cast<uint4*>(dst + (2 * D) * kPitch + ((sw ^ (2 * D)) << 3)) = even;
  *reinterpret_cast<uint4*>(dst + (2 * D + 1) * kPitch + ((sw ^ (2 * D + 1)) << 3)) = odd;
}
__device__ __forceinline__ void store_block_transposed(const Block8x8& b, uint16_t* dst, int sw) {
  store_chunk_transposed<0>(b, dst, sw);
  store_chunk_transposed<1>(b, dst, sw);
  store_chunk_transposed<2>(b, dst, sw);
  store_chunk_transposed<3>(b, dst, sw);
}

// One 64-row stage of a workgroup: 64 MFMAs per wave on the LDS buffers As / Bs while (FETCH != 0) the next stage
// travels global memory -> registers -> transpose -> the other LDS buffer.  FETCH: 0 nothing follows, 1 the next
// stage is complete, 2 it is the ragged last one.  The function is one basic block; the group barriers at its end
// give the order the instruction scheduler is asked for: loads first, then fragment reads of k-slice ks + 1 between
// the MFMAs of slice ks, and the transposes and LDS writes of the next stage between the MFMAs of the last slice.
template <bool DIAG, int FETCH>
__device__ __forceinline__ void syrk_stage(floatx16 (&acc)[4][4], const uint16_t* As, const uint16_t* Bs, uint16_t* nxt,
                                           Block8x8& ga, Block8x8& gb, const uint16_t* __restrict__ X,
                                           const uint16_t* __restrict__ XB, long rows, long n, long r0, long ci, long cj,
                                           int offA, int offB, int swr, int sww) {
  if (FETCH) {
    fetch_block<FETCH == 1>(ga, X, rows, n, r0, ci);
    if (!DIAG) fetch_block<FETCH == 1>(gb, XB, rows, n, r0, cj);
  }
  bf16x8 fa[2][4], fb[2][4];
#pragma unroll
  for (int mi = 0; mi < 4; ++mi) {
    const int piece = (swr ^ (4 * (mi & 1))) << 3;
    fa[0][mi] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(As + offA + mi * 32 * kPitch + piece));
    fb[0][mi] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(Bs + offB + mi * 32 * kPitch + piece));
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int ks = 0; ks < kStage / 16; ++ks) {
    if (ks + 1 < kStage / 16) {
      // the fragments of the next k-slice are requested before the 16 MFMAs of this one are queued
#pragma unroll
      for (int mi = 0; mi < 4; ++mi) {
        const int piece = (swr ^ (2 * (ks + 1)) ^ (4 * (mi & 1))) << 3;
        fa[(ks + 1) & 1][mi] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(As + offA + mi * 32 * kPitch + piece));
        fb[(ks + 1) & 1][mi] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(Bs + offB + mi * 32 * kPitch + piece));
      }
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int mi = 0; mi < 4; ++mi)
#pragma unroll
      for (int ni = 0; ni < 4; ++ni) {
        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[ks & 1][mi], fb[ks & 1][ni], acc[mi][ni], 0, 0, 0);
        if (FETCH && ks == kStage / 16 - 1) {
          // last k-slice: the next stage's blocks are transposed and written to the other LDS buffer in the shadow of
          // the matrix instructions, one quarter block (8 permutes, 2 writes) after every second (fourth) MFMA
          const int i = mi * 4 + ni;
          if (!DIAG) {
            if (i == 0) store_chunk_transposed<0>(ga, nxt, sww);
            if (i == 2) store_chunk_transposed<1>(ga, nxt, sww);
            if (i == 4) store_chunk_transposed<2>(ga, nxt, sww);
            if (i == 6) store_chunk_transposed<3>(ga, nxt, sww);
            if (i == 8) store_chunk_transposed<0>(gb, nxt + kSliceU16, sww);
            if (i == 10) store_chunk_transposed<1>(gb, nxt + kSliceU16, sww);
            if (i == 12) store_chunk_transposed<2>(gb, nxt + kSliceU16, sww);
            if (i == 14) store_chunk_transposed<3>(gb, nxt + kSliceU16, sww);
          } else {
            if (i == 0) store_chunk_transposed<0>(ga, nxt, sww);
            if (i == 4) store_chunk_transposed<1>(ga, nxt, sww);
            if (i == 8) store_chunk_transposed<2>(ga, nxt, sww);
            if (i == 12) store_chunk_transposed<3>(ga, nxt, sww);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    __builtin_amdgcn_sched_barrier(0);
  }
  __syncthreads();
}

template <bool DIAG>
__device__ __forceinline__ void syrk_tile(floatx16 (&acc)[4][4], uint16_t* lds, const uint16_t* __restrict__ X,
                                          const uint16_t* __restrict__ XB, long rows, long n, long ci, long cj, int ro,
                                          int cg, int offA, int offB, int swr) {
  const long stages = (rows + kStage - 1) / kStage;
  Block8x8 ga, gb;
  uint16_t* const wr = lds + (8 * cg) * kPitch;  // row of this thread's first column within a slice
  const int sww = ro ^ (cg & 7);
  fetch_block<false>(ga, X, rows, n, 8 * ro, ci);
  if (!DIAG) fetch_block<false>(gb, XB, rows, n, 8 * ro, cj);
  store_block_transposed(ga, wr, sww);
  if (!DIAG) store_block_transposed(gb, wr + kSliceU16, sww);
  __syncthreads();
  // stages whose successor is complete run in one loop body; the ragged successor and the last stage follow
  long st = 0;
#define QTIP_SYRK_STAGE(F)                                                                                   \
  syrk_stage<DIAG, F>(acc, lds + (st & 1) * 2 * kSliceU16, lds + (st & 1) * 2 * kSliceU16 + (DIAG ? 0 : kSliceU16), \
                      wr + ((st + 1) & 1) * 2 * kSliceU16, ga, gb, X, XB, rows, n, (st + 1) * kStage + 8 * ro, ci, cj, offA, offB, swr, sww)
  for (; (st + 2) * kStage <= rows; ++st) QTIP_SYRK_STAGE(1);
  if (st + 1 < stages) {
    QTIP_SYRK_STAGE(2);
    ++st;
  }
  QTIP_SYRK_STAGE(0);
#undef QTIP_SYRK_STAGE
}

// DOT = false: H += X^T X on the tiles on or below the diagonal (XB == X).
// DOT = true:  nothing is stored; partial[ti * tiles + tj] = w * sum_ij (X^T XB)_ij H_ij over the tile, w = 2 below the
//              diagonal and 1 on it: with X^T XB symmetric the partials add up to sum_ij (X^T XB)_ij H_ij of a symmetric
//              H.  The tiles above the diagonal keep the zero the caller wrote.
template <bool DOT>
__global__ __launch_bounds__(256, 1) void syrk_bf16_kernel(const uint16_t* __restrict__ X, const uint16_t* __restrict__ XB,
                                                          long rows, long n, float* __restrict__ H,
                                                          double* __restrict__ partial, int tiles, int patch_cols) {
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
  // workgroup -> tile: ids that differ by 8 run on different XCDs; the 32 ids an XCD holds at a time are one patch
  const long b = blockIdx.x;
  const long xcd = b & 7, local = b >> 3;
  const long patch = (local / (kPatchRows * kPatchCols)) * 8 + xcd, within = local % (kPatchRows * kPatchCols);
  const long ti = (patch / patch_cols) * kPatchRows + within / kPatchCols;
  const long tj = (patch % patch_cols) * kPatchCols + within % kPatchCols;
  if (ti >= tiles || tj > ti) return;  // outside the matrix or above the diagonal
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  // this thread stages rows 8 ro .. 8 ro + 7, columns 8 cg .. 8 cg + 7 of a slice; 8 neighbouring lanes read one
  // 128-byte line of a row of X
  const int ro = (t >> 3) & 7, cg = (t & 7) + 8 * (t >> 6);
  const long ci = ti * kTile + 8 * cg, cj = tj * kTile + 8 * cg;
  const int rl = lane & 31;
  const int offA = (wm * 128 + rl) * kPitch, offB = (wn * 128 + rl) * kPitch;
  const int swr = (lane >> 5) ^ (rl & 7) ^ (rl >> 3);  // piece of k-slice 0, row tile 0; the others differ by constants

  floatx16 acc[4][4];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][c][v] = 0.f;
  {
    // The accumulators enter the stage loop as results of a matrix instruction (of zero operands): they then live in
    // the accumulation registers from the start.  Entering as plain zeros, the compiler keeps them in ordinary
    // registers at the loop head and copies all 256 of them to the accumulation registers and back in every stage.
    bf16x8 z;
#pragma unroll
    for (int e = 0; e < 8; ++e) z[e] = __bf16(0.f);
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[a][c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(z, z, acc[a][c], 0, 0, 0);
  }
  if (!DOT && ti == tj) syrk_tile<true>(acc, lds, X, XB, rows, n, ci, cj, ro, cg, offA, offB, swr);
  else syrk_tile<false>(acc, lds, X, XB, rows, n, ci, cj, ro, cg, offA, offB, swr);

  // accumulator element v of a lane: row (v % 4) + 8 (v / 4) + 4 (lane / 32), column lane % 32 of the 32 x 32 tile
  double dot = 0.0;
  if ((ti + 1) * kTile <= n && (tj + 1) * kTile <= n) {
    // a tile inside the matrix (all of them when n is a multiple of 256): the 16 values of H that go with one
    // 32 x 32 accumulator are fetched together - one round trip to memory per accumulator, not one per value
    float* hb = H + (ti * kTile + wm * 128 + 4 * (lane >> 5)) * n + tj * kTile + wn * 128 + rl;
#pragma unroll
    for (int mi = 0; mi < 4; ++mi)
#pragma unroll
      for (int ni = 0; ni < 4; ++ni) {
        float h[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) h[v] = hb[long(mi * 32 + (v & 3) + 8 * (v >> 2)) * n + ni * 32];
        __builtin_amdgcn_sched_barrier(0);  // all 16 loads are issued before the first value is used
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          if (DOT) dot += double(acc[mi][ni][v]) * double(h[v]);
          else hb[long(mi * 32 + (v & 3) + 8 * (v >> 2)) * n + ni * 32] = h[v] + acc[mi][ni][v];
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
    // lanes, then waves, in a fixed order (the stage loop ended with a barrier: the staging buffers are free)
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) dot += __shfl_xor(dot, off, 64);
    double* red = reinterpret_cast<double*>(lds);
    if (lane == 0) red[wave] = dot;
    __syncthreads();
    if (t == 0) partial[ti * tiles + tj] = (ti == tj ? 1.0 : 2.0) * (((red[0] + red[1]) + red[2]) + red[3]);
  }
}

// ---------------------------------------------------------------- the same update from operands stored as LDS images
// The quadratic forms of the proxy build their operands themselves (split_image_kernel), so they are written as the
// LDS images of the kernel's stages: [stage of 32 rows of K][column tile of 256][column][32 k], the four 16-byte
// pieces of a column at position p ^ ((column >> 2) & 3) (free of bank conflicts for the 16-byte fragment reads: the
// 16 lanes the LDS serves together then touch 16 different 16-byte bank groups).  A stage of an operand is 16 KB of
// contiguous global memory and goes straight into LDS (global_load_lds_dwordx4, 1 KB per wave and instruction): no
// staging registers, no transposes, no LDS writes by the waves.  Four stages of LDS; the loads run two stages ahead
// of the matrix cores, and a wave fetches the fragments of the next 16 k while the 16 MFMAs of the present ones run.
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
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
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

  // wave w brings the 1 KB chunks 4 w .. 4 w + 3 of both operand slices of a stage, 16 bytes per lane
  const size_t stage_stride = size_t(tiles) * kImgSliceU16;
  const uint16_t* ga = IA + size_t(ti) * kImgSliceU16 + (wave * 4) * 512 + lane * 8;
  const uint16_t* gb = IB + size_t(tj) * kImgSliceU16 + (wave * 4) * 512 + lane * 8;
  typedef __attribute__((address_space(3))) void* lds_ptr;
  auto issue = [&](int st) {
    uint16_t* la = lds + (st % ISTAGES) * 2 * kImgSliceU16 + (wave * 4) * 512;
    const size_t off = size_t(st) * stage_stride;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      __builtin_amdgcn_global_load_lds(ga + off + q * 512, (lds_ptr)(la + q * 512), 16, 0, 0);
      __builtin_amdgcn_global_load_lds(gb + off + q * 512, (lds_ptr)(la + kImgSliceU16 + q * 512), 16, 0, 0);
    }
  };
  // fragment of 8 k (piece 2 ks + lane / 32) of column wX * 128 + 32 i + rl
  const int offA = (wm * 128 + rl) * IK, offB = (wn * 128 + rl) * IK, sw = (rl >> 2) & 3, hi = lane >> 5;
  bf16x8 fa[2][4], fb[2][4];
  auto fetch = [&](int st, int ks, int set) {
    const uint16_t* As = lds + (st % ISTAGES) * 2 * kImgSliceU16;
    const int piece = ((2 * ks + hi) ^ sw) << 3;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      fa[set][i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(As + offA + i * 32 * IK + piece));
      fb[set][i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(As + kImgSliceU16 + offB + i * 32 * IK + piece));
    }
  };
  auto mfmas = [&](int set, int half) {  // the 8 MFMAs of row tiles 2 half, 2 half + 1
#pragma unroll
    for (int mi = 2 * half; mi < 2 * half + 2; ++mi)
#pragma unroll
      for (int ni = 0; ni < 4; ++ni)
        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[set][mi], fb[set][ni], acc[mi][ni], 0, 0, 0);
  };
  auto landed = [&](int later_stages) {  // this wave's loads of a stage have landed (8 per stage, in order) ...
    if (later_stages >= 1) __builtin_amdgcn_s_waitcnt(0x0F78);  // vmcnt(8)
    else __builtin_amdgcn_s_waitcnt(0x0F70);                    // vmcnt(0)
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();  // ... and so have everyone's (a bare barrier: no wait for the loads in flight)
    asm volatile("" ::: "memory");
  };
  for (int p = 0; p < 2 && p < stages; ++p) issue(p);
  landed(stages > 1 ? 1 : 0);
  if (stages > 2) issue(2);
  fetch(0, 0, 0);
  // A wave has nothing to hide a wait behind but its own MFMAs, so the fragments of the next 16 k are requested
  // between the two halves of the 16 MFMAs of the present ones: the wait the compiler puts in front of their first
  // use then finds them there.
  for (int st = 0; st < stages; ++st) {
    mfmas(0, 0);
    __builtin_amdgcn_sched_barrier(0);
    fetch(st, 1, 1);
    __builtin_amdgcn_sched_barrier(0);
    mfmas(0, 1);
    __builtin_amdgcn_sched_barrier(0);
    if (st + 1 < stages) {
      // stage st + 1 is needed next; stage st + 2 may still be on its way; the buffer of stage st - 1, which every
      // wave has read before this barrier, takes stage st + 3
      landed(st + 2 < stages ? 1 : 0);
      if (st + 3 < stages) issue(st + 3);
    }
    mfmas(1, 0);
    __builtin_amdgcn_sched_barrier(0);
    if (st + 1 < stages) fetch(st + 1, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    mfmas(1, 1);
    __builtin_amdgcn_sched_barrier(0);
  }
  __syncthreads();

  // accumulator element v of a lane: row (v % 4) + 8 (v / 4) + 4 (lane / 32), column lane % 32 of the 32 x 32 tile
  double dot = 0.0;
  if ((ti + 1) * kTile <= n && (tj + 1) * kTile <= n) {
    float* hb = H + (ti * kTile + wm * 128 + 4 * (lane >> 5)) * n + tj * kTile + wn * 128 + rl;
#pragma unroll
    for (int mi = 0; mi < 4; ++mi)
#pragma unroll
      for (int ni = 0; ni < 4; ++ni) {
        float h[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) h[v] = hb[long(mi * 32 + (v & 3) + 8 * (v >> 2)) * n + ni * 32];
        __builtin_amdgcn_sched_barrier(0);  // all 16 loads are issued before the first value is used
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          if (DOT) dot += double(acc[mi][ni][v]) * double(h[v]);
          else hb[long(mi * 32 + (v & 3) + 8 * (v >> 2)) * n + ni * 32] = h[v] + acc[mi][ni][v];
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
        QTIP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(syrk_bf16_kernel<false>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, int(kLdsBytes)));
        QTIP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(syrk_img_kernel<true>),
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

void launch_hessian_accumulate(const uint16_t* X, long rows, long n, float* H, hipStream_t s) {
  QTIP_REQUIRE(X != nullptr && H != nullptr && rows >= 0 && n > 0, "hessian_accumulate: bad arguments");
  QTIP_REQUIRE(n % 8 == 0 && (reinterpret_cast<uintptr_t>(X) & 15) == 0, "hessian_accumulate: rows of X must be 16-byte aligned (n = %ld)", n);
  if (rows == 0) return;
  SyrkGrid g(n);
  syrk_bf16_kernel<false><<<dim3(g.grid), dim3(256), kLdsBytes, s>>>(X, X, rows, n, H, nullptr, g.tiles, g.patch_cols);
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
