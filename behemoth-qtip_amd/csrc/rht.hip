// Randomised Hadamard transform pieces for gfx950: sign scaling + natural-order FWHT per power-of-two chunk + the
// K-point Hadamard-factor mix in one kernel, tiled transpose, and fixed-order fp64 reductions.
//
// The fp32 operation order is the one of the reference's GPU path (src/kernels.hip:214-254, 293-313: butterflies
// (a+b, a-b) for h = 1, 2, 4, ...; mix as a signed sum over k ascending from 0; one multiply by 1/sqrt(n) at the
// end), so results match it bit for bit.  The schedule is built for 64-wide waves and 160 KB of LDS:
//   * a lane holds up to 16 consecutive values: the butterfly stages below that width run in registers, the next six
//     stages exchange values between the lanes of the wave (a lane whose index bit is set adds its negated value to
//     the partner's: a - b as a + (-b)), so a wave finishes a 1024-point transform without LDS or barriers;
//   * the stages above 1024 (chunks of 2048..8192) run in registers again after one trip through LDS, on values
//     1024 apart;
//   * a row of up to 40000 values stays in LDS after its chunks are transformed and the K-point mix reads it from
//     there, so the row is read from HBM once and written once; the Hadamard factor is a table of sign bits that
//     flips the sign bit of a value before a plain add.  Longer rows take a second kernel for the mix.
#include <mutex>

#include "data/qtip_tables.h"
#include "qtip_internal.hpp"
#include "rht.hpp"

namespace qtipmi {
namespace {

constexpr int kRowThreads = 1024;     // 16 waves per row segment
constexpr int kRowLdsFloats = 40000;  // 160 000 of the 163 840 bytes of LDS
constexpr int kMixLanes = 64;

__device__ __forceinline__ float flip(float v, uint32_t sign_bit) { return __uint_as_float(__float_as_uint(v) ^ sign_bit); }

template <int N>
__device__ __forceinline__ void fwht_registers(float (&r)[N]) {
#pragma unroll
  for (int h = 1; h < N; h <<= 1)
#pragma unroll
    for (int i = 0; i < N; i += 2 * h)
#pragma unroll
      for (int j = i; j < i + h; ++j) {
        const float a = r[j], b = r[j + h];
        r[j] = a + b;
        r[j + h] = a - b;
      }
}

// One wave transforms spans of 64 * EPT consecutive values of the segment (stages h < min(P, 64 * EPT)) and leaves
// them in v.  seg_len values at x, column sign factors at cs (or null), row factor rsv.
template <int EPT>
__device__ __forceinline__ void fwht_spans(const float* __restrict__ x, const float* __restrict__ cs, float rsv,
                                           bool scaled, bool vec, int seg_len, int P, float* __restrict__ v) {
  constexpr int S = 64 * EPT;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int hend = P < S ? P : S;
  for (int base = wave * S + lane * EPT; base - lane * EPT < seg_len; base += (kRowThreads / 64) * S) {
    float r[EPT];
    if (EPT >= 4 && vec && base + EPT <= seg_len) {
#pragma unroll
      for (int e = 0; e < EPT; e += 4) {
        const float4 q = *reinterpret_cast<const float4*>(x + base + e);
        r[e] = q.x, r[e + 1] = q.y, r[e + 2] = q.z, r[e + 3] = q.w;
      }
    } else {
#pragma unroll
      for (int e = 0; e < EPT; ++e) r[e] = base + e < seg_len ? x[base + e] : 0.0f;
    }
    if (scaled) {
#pragma unroll
      for (int e = 0; e < EPT; ++e) {
        r[e] *= rsv;
        if (cs && base + e < seg_len) r[e] *= cs[base + e];
      }
    }
    fwht_registers<EPT>(r);
    for (int h = EPT; h < hend; h <<= 1) {
      const int mask = h / EPT;
      const uint32_t neg = (lane & mask) ? 0x80000000u : 0u;
#pragma unroll
      for (int e = 0; e < EPT; ++e) r[e] = __shfl_xor(r[e], mask, 64) + flip(r[e], neg);
    }
#pragma unroll
    for (int e = 0; e < EPT; ++e)
      if (base + e < seg_len) v[base + e] = r[e];
  }
}

// Stages h = 1024 .. P/2 of every chunk in v: a thread takes the J = P / 1024 values that lie 1024 apart.
template <int J>
__device__ __forceinline__ void fwht_high(float* __restrict__ v, int seg_len) {
  for (int q = threadIdx.x; q < seg_len / J; q += kRowThreads) {
    float* p = v + (q >> 10) * (J * 1024) + (q & 1023);
    float r[J];
#pragma unroll
    for (int j = 0; j < J; ++j) r[j] = p[j * 1024];
    fwht_registers<J>(r);
#pragma unroll
    for (int j = 0; j < J; ++j) p[j * 1024] = r[j];
  }
}

// bit k of row k2 of the table: entry (k2, k) of the mixing matrix is -1
__device__ __forceinline__ uint32_t neg_bit(const uint32_t* __restrict__ row_bits, int k) {
  return (row_bits[k >> 5] >> (k & 31)) << 31;
}

// One workgroup per segment of a row.  mix != 0 (the segment is the whole row, K > 1): out[k2 P + i] =
// (sum_k +-v[k P + i]) * scale.  Otherwise the transformed values times scale go back in place.
// KT: the factor size when it is one of the common ones (values in registers), 0 for any K (values re-read from LDS).
template <int KT>
__global__ __launch_bounds__(kRowThreads) void rht_rows_kernel(float* __restrict__ X, long ld, int n, int P, int K,
                                                              int seg, int nseg, float scale,
                                                              const float* __restrict__ rs,
                                                              const float* __restrict__ cs,
                                                              const uint32_t* __restrict__ neg, int mix) {
  extern __shared__ float v[];
  const long row = blockIdx.x / nseg;
  const int col0 = int(blockIdx.x % nseg) * seg;
  const int seg_len = n - col0 < seg ? n - col0 : seg;
  float* x = X + row * ld + col0;
  const bool vec = ((reinterpret_cast<uintptr_t>(x) & 15u) == 0);
  const bool scaled = rs != nullptr || cs != nullptr;
  const float rsv = rs ? rs[row] : 1.0f;
  const float* c = cs ? cs + col0 : nullptr;
  if (P >= 1024) fwht_spans<16>(x, c, rsv, scaled, vec, seg_len, P, v);
  else if (P == 512) fwht_spans<8>(x, c, rsv, scaled, vec, seg_len, P, v);
  else if (P == 256) fwht_spans<4>(x, c, rsv, scaled, vec, seg_len, P, v);
  else if (P == 128) fwht_spans<2>(x, c, rsv, scaled, false, seg_len, P, v);
  else fwht_spans<1>(x, c, rsv, scaled, false, seg_len, P, v);
  __syncthreads();
  if (P > 1024) {
    if (P == 2048) fwht_high<2>(v, seg_len);
    else if (P == 4096) fwht_high<4>(v, seg_len);
    else fwht_high<8>(v, seg_len);
    __syncthreads();
  }
  if (!mix) {
    for (int i = threadIdx.x; i < seg_len; i += kRowThreads) x[i] = v[i] * scale;
    return;
  }
  // P <= 1024 here would leave threads idle: the outputs k2 of one i are shared out over kRowThreads / P threads
  const int W = (K + 31) >> 5;
  const int per = P < kRowThreads ? kRowThreads / P : 1;
  for (int i = int(threadIdx.x) % (P < kRowThreads ? P : kRowThreads); i < P; i += kRowThreads) {
    const int first = P < kRowThreads ? int(threadIdx.x) / P : 0;
    if constexpr (KT > 0) {
      float y[KT];
#pragma unroll
      for (int k = 0; k < KT; ++k) y[k] = v[k * P + i];
      for (int k2 = first; k2 < KT; k2 += per) {
        const uint32_t* bits = neg + k2 * W;
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < KT; ++k) s += flip(y[k], neg_bit(bits, k));
        x[long(k2) * P + i] = s * scale;
      }
    } else {
      for (int k2 = first; k2 < K; k2 += per) {
        const uint32_t* bits = neg + k2 * W;
        float s = 0.0f;
        for (int k = 0; k < K; ++k) s += flip(v[k * P + i], neg_bit(bits, k));
        x[long(k2) * P + i] = s * scale;
      }
    }
  }
}

// ---- rows of K chunks of 1024 values (every large layer here: 12288 = 12 x 1024, 28672 = 28 x 1024): one resident
// workgroup per compute unit walks its share of the rows and has the next row on its way from HBM while it mixes
// the present one.  The form above gives a row to a workgroup that loads, transforms, mixes and stores it, one phase
// after the other, with nothing else resident beside it (a row fills most of the LDS): each phase leaves the other
// pipes idle.  Here
//   * a wave holds a 1024-point chunk in 16 registers per lane; the loads of the next row's chunks are issued before
//     the present row's mix and land while its 784 (K = 28) signed adds per thread run;
//   * the exchanges between lanes 1, 2, 4 and 8 apart are DPP moves in the vector pipe, only those 16 and 32 apart go
//     through the LDS crossbar;
//   * the signs of the mixing matrix are compile-time constants: a term of the mix is one add or one subtract
//     (s - y and s + (-y) are the same sum), with no sign table read and no sign-bit arithmetic.
// Same sums in the same order as the form above, so the same bits.
template <int K>
struct HadRows {
  uint64_t minus[K];  // bit k of minus[k2]: entry (k2, k) of the mixing matrix is -1
};
template <int K, bool kTranspose>
constexpr HadRows<K> had_rows() {
  HadRows<K> r{};
  const uint32_t* bits = K == 12 ? qtip_had12_bits : K == 20 ? qtip_had20_bits : K == 28 ? qtip_had28_bits : qtip_had36_bits;
  constexpr int wpr = (K + 31) / 32;
  for (int k2 = 0; k2 < K; ++k2)
    for (int k = 0; k < K; ++k) {
      const int row = kTranspose ? k : k2, col = kTranspose ? k2 : k;
      const bool plus = (bits[row * wpr + (col >> 5)] >> (col & 31)) & 1u;
      if (!plus) r.minus[k2] |= uint64_t(1) << k;
    }
  return r;
}
template <int K, bool kTranspose>
inline constexpr HadRows<K> kHadRows = had_rows<K, kTranspose>();

// the value of the lane whose index differs in bit log2(MASK), MASK <= 8: within a row of 16 lanes, by DPP
template <int MASK>
__device__ __forceinline__ float row_partner(float v) {
  const int x = __builtin_bit_cast(int, v);
  int y;
  if constexpr (MASK == 1) y = __builtin_amdgcn_update_dpp(0, x, 0xB1, 0xf, 0xf, false);        // quad_perm [1, 0, 3, 2]
  else if constexpr (MASK == 2) y = __builtin_amdgcn_update_dpp(0, x, 0x4E, 0xf, 0xf, false);   // quad_perm [2, 3, 0, 1]
  else if constexpr (MASK == 4)                                                                 // i ^ 3, then i ^ 7
    y = __builtin_amdgcn_update_dpp(0, __builtin_amdgcn_update_dpp(0, x, 0x1B, 0xf, 0xf, false), 0x141, 0xf, 0xf, false);
  else y = __builtin_amdgcn_update_dpp(0, x, 0x128, 0xf, 0xf, false);                           // row_ror:8
  return __builtin_bit_cast(float, y);
}

// natural-order 1024-point transform of the 16 consecutive values per lane of one wave
__device__ __forceinline__ void fwht_wave1024(float (&r)[16], int lane) {
  fwht_registers<16>(r);
#define QTIP_ROW_STAGE(MASK)                                                    \
  {                                                                             \
    const uint32_t neg = (lane & MASK) ? 0x80000000u : 0u;                      \
    _Pragma("unroll") for (int e = 0; e < 16; ++e) r[e] = row_partner<MASK>(r[e]) + flip(r[e], neg); \
  }
  QTIP_ROW_STAGE(1)
  QTIP_ROW_STAGE(2)
  QTIP_ROW_STAGE(4)
  QTIP_ROW_STAGE(8)
#undef QTIP_ROW_STAGE
#pragma unroll
  for (int mask = 16; mask <= 32; mask <<= 1) {
    const uint32_t neg = (lane & mask) ? 0x80000000u : 0u;
#pragma unroll
    for (int e = 0; e < 16; ++e) r[e] = __shfl_xor(r[e], mask, 64) + flip(r[e], neg);
  }
}

// X: rows of KT * 1024 values, 16-byte aligned (ld % 4 == 0).  gridDim.x workgroups share the rows out in turn.
template <int KT, bool kTranspose>
__global__ __launch_bounds__(kRowThreads) void rht_rows_p1024_kernel(float* __restrict__ X, long ld, long rows,
                                                                    float scale, const float* __restrict__ rs,
                                                                    const float* __restrict__ cs) {
  extern __shared__ float v[];
  constexpr int kWaves = kRowThreads / 64;
  constexpr int kTurns = (KT + kWaves - 1) / kWaves;  // chunks a wave takes at most
  constexpr HadRows<KT> kHad = kHadRows<KT, kTranspose>;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // A lane's 16 values leave as four 16-byte writes, 64 bytes from the neighbouring lane's: the four pieces of lane l
  // change places by (l / 4 % 4) ^ (l & 2), so that 8 neighbouring lanes write 8 different 16-byte columns of 128
  // bytes of banks and 16 lanes 16 of 256; the mix reads value i of a chunk at i with bits 2..3 changed accordingly
  // (64 neighbouring i: 64 neighbouring words).
  const int swz = ((lane >> 2) & 3) ^ (lane & 2);
  float4 in[kTurns][4];
  auto fetch = [&](long row) {
    const float* x = X + row * ld + lane * 16;
#pragma unroll
    for (int j = 0; j < kTurns; ++j) {
      const int chunk = wave + kWaves * j;
      if (chunk < KT) {
#pragma unroll
        for (int q = 0; q < 4; ++q) in[j][q] = *reinterpret_cast<const float4*>(x + chunk * 1024 + 4 * q);
      }
    }
  };
  long row = blockIdx.x;
  if (row < rows) fetch(row);
  for (; row < rows; row += gridDim.x) {
    const float rsv = rs ? rs[row] : 1.0f;
#pragma unroll
    for (int j = 0; j < kTurns; ++j) {
      const int chunk = wave + kWaves * j;
      if (chunk < KT) {
        float r[16];
#pragma unroll
        for (int q = 0; q < 4; ++q) r[4 * q] = in[j][q].x, r[4 * q + 1] = in[j][q].y, r[4 * q + 2] = in[j][q].z, r[4 * q + 3] = in[j][q].w;
        if (rs || cs) {
#pragma unroll
          for (int e = 0; e < 16; ++e) r[e] *= rsv;
          if (cs) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const float4 c = *reinterpret_cast<const float4*>(cs + chunk * 1024 + lane * 16 + 4 * q);
              r[4 * q] *= c.x, r[4 * q + 1] *= c.y, r[4 * q + 2] *= c.z, r[4 * q + 3] *= c.w;
            }
          }
        }
        fwht_wave1024(r, lane);
#pragma unroll
        for (int q = 0; q < 4; ++q)
          *reinterpret_cast<float4*>(v + chunk * 1024 + lane * 16 + 4 * (q ^ swz)) = make_float4(r[4 * q], r[4 * q + 1], r[4 * q + 2], r[4 * q + 3]);
      }
    }
    __syncthreads();
    const int i = threadIdx.x;
    float y[KT];
#pragma unroll
    for (int k = 0; k < KT; ++k) y[k] = v[k * 1024 + (i ^ ((((i >> 6) & 3) ^ ((i >> 4) & 2)) << 2))];
    __syncthreads();  // the next row's chunks may now be written over this one
    const long next = row + gridDim.x;
    if (next < rows) fetch(next);
    float* x = X + row * ld + i;
#pragma unroll
    for (int k2 = 0; k2 < KT; ++k2) {
      float s = 0.0f;
#pragma unroll
      for (int k = 0; k < KT; ++k) {
        if ((kHad.minus[k2] >> k) & 1) s -= y[k];
        else s += y[k];
      }
      x[k2 * 1024] = s * scale;
    }
  }
}

// The mix for rows too long for LDS, in place on transformed chunks: one wave per 64 values of i, the K inputs of a
// lane parked in LDS (ys[k][lane]) because the outputs overwrite them.
__global__ __launch_bounds__(kMixLanes) void had_mix_long_rows_kernel(float* __restrict__ X, long ld, int P, int K,
                                                                     float scale, const uint32_t* __restrict__ neg) {
  extern __shared__ float ys[];
  const int per_row = (P + kMixLanes - 1) / kMixLanes;
  const long row = blockIdx.x / per_row;
  const int i = int(blockIdx.x % per_row) * kMixLanes + int(threadIdx.x);
  if (i >= P) return;  // the only wave of the workgroup: no barrier is skipped
  float* x = X + row * ld + i;
  float* mine = ys + threadIdx.x;
  for (int k = 0; k < K; ++k) mine[k * kMixLanes] = x[long(k) * P];
  const int W = (K + 31) >> 5;
  for (int k2 = 0; k2 < K; ++k2) {
    const uint32_t* bits = neg + k2 * W;
    float s = 0.0f;
    for (int k = 0; k < K; ++k) s += flip(mine[k * kMixLanes], neg_bit(bits, k));
    x[long(k2) * P] = s * scale;
  }
}

__global__ __launch_bounds__(256) void transpose_kernel(const float* __restrict__ in, long rows, long cols, long ld_in,
                                                        float* __restrict__ out, long ld_out) {
  __shared__ float tile[64][65];
  const long c0 = long(blockIdx.x) * 64, r0 = long(blockIdx.y) * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // 64 x 4
  for (int k = ty; k < 64; k += 4) {
    const long r = r0 + k, c = c0 + tx;
    if (r < rows && c < cols) tile[k][tx] = in[r * ld_in + c];
  }
  __syncthreads();
  for (int k = ty; k < 64; k += 4) {
    const long c = c0 + k, r = r0 + tx;
    if (r < rows && c < cols) out[c * ld_out + r] = tile[tx][k];
  }
}

// X[r][c] *= a: a block takes a row segment of 1024 columns, four floats per thread where the row allows it
__global__ __launch_bounds__(256) void scale_kernel(float* __restrict__ X, long rows, long cols, long ld, float a) {
  const long r = blockIdx.y;
  const long c = (long(blockIdx.x) * 256 + threadIdx.x) * 4;
  float* p = X + r * ld + c;
  if (c + 4 <= cols && (reinterpret_cast<uintptr_t>(p) & 15) == 0) {
    float4 v = *reinterpret_cast<float4*>(p);
    v.x *= a, v.y *= a, v.z *= a, v.w *= a;
    *reinterpret_cast<float4*>(p) = v;
  } else {
    for (int e = 0; e < 4 && c + e < cols; ++e) p[e] *= a;
  }
}

__global__ void add_diag_kernel(float* __restrict__ H, long n, float a) {
  const long i = long(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) H[i * n + i] += a;
}

// ---- fixed-order fp64 reductions: block b sums its contiguous slice in a fixed tree, partial[b] is written,
// a second single-block launch adds the partials in index order.
constexpr int kRedBlocks = 1024, kRedThreads = 256;

__device__ __forceinline__ double block_sum(double v) {
  __shared__ double red[kRedThreads];
  red[threadIdx.x] = v;
  __syncthreads();
  for (int s = kRedThreads / 2; s > 0; s >>= 1) {
    if (int(threadIdx.x) < s) red[threadIdx.x] += red[threadIdx.x + s];
    __syncthreads();
  }
  return red[0];
}
// mode 0: sum A^2 ; mode 1: sum A*B ; mode 2: sum (A-B)^2 ; mode 3: sum diag(A) (rows = n, cols ignored)
__global__ __launch_bounds__(kRedThreads) void reduce_partial_kernel(const float* __restrict__ A, long lda,
                                                                     const float* __restrict__ B, long ldb, long rows,
                                                                     long cols, int mode, double* __restrict__ partial) {
  const long total = mode == 3 ? rows : rows * cols;
  const long per = (total + gridDim.x - 1) / gridDim.x;
  const long lo = long(blockIdx.x) * per, hi = lo + per < total ? lo + per : total;
  double acc = 0;
  // (row, column) of the element i = r cols + c, carried along instead of divided out for every element
  long r = 0, c = 0;
  if (mode != 3 && lo + threadIdx.x < hi) r = (lo + threadIdx.x) / cols, c = (lo + threadIdx.x) % cols;
  for (long i = lo + threadIdx.x; i < hi; i += kRedThreads) {
    if (mode == 3) {
      acc += double(A[i * lda + i]);
    } else {
      const double a = A[r * lda + c];
      if (mode == 0) acc += a * a;
      else {
        const double b = B[r * ldb + c];
        if (mode == 1) acc += a * b;
        else acc += (a - b) * (a - b);
      }
      c += kRedThreads;
      while (c >= cols) c -= cols, ++r;
    }
  }
  acc = block_sum(acc);
  if (threadIdx.x == 0) partial[blockIdx.x] = acc;
}
__global__ __launch_bounds__(kRedThreads) void reduce_final_kernel(const double* __restrict__ partial, int count,
                                                                   double* __restrict__ out) {
  double acc = 0;
  for (int i = threadIdx.x; i < count; i += kRedThreads) acc += partial[i];
  acc = block_sum(acc);
  if (threadIdx.x == 0) *out = acc;
}

}  // namespace

// ---- launchers
void Rht::init(int device, hipStream_t stream) {
  dev_ = device;
  s_ = stream;
  partial_.alloc(kRedBlocks + 1);
  QTIP_HIP(hipDeviceGetAttribute(&cus_, hipDeviceAttributeMultiprocessorCount, device));
  if (cus_ <= 0) cus_ = 1;
}

// sign bits of the mixing matrix (hadK, or its transpose), row k2 in (K + 31) / 32 words: bit k set = entry -1
const uint32_t* Rht::device_had(int K, bool transpose) {
  const int key = K * 2 + (transpose ? 1 : 0);
  for (auto& e : had_) if (e.first == key) return e.second->p;
  const auto m = had_matrix(K, transpose);
  const int W = (K + 31) / 32;
  std::vector<uint32_t> bits(size_t(K) * W, 0u);
  for (int r = 0; r < K; ++r)
    for (int k = 0; k < K; ++k)
      if (m[size_t(r) * K + k] < 0) bits[size_t(r) * W + (k >> 5)] |= 1u << (k & 31);
  auto buf = std::make_unique<DBuf<uint32_t>>(bits.size());
  QTIP_HIP(hipMemcpyAsync(buf->p, bits.data(), bits.size() * sizeof(uint32_t), hipMemcpyHostToDevice, s_));
  QTIP_HIP(hipStreamSynchronize(s_));
  had_.emplace_back(key, std::move(buf));
  return had_.back().second->p;
}

namespace {
using RowKernel = void (*)(float*, long, int, int, int, int, int, float, const float*, const float*, const uint32_t*,
                           int);
RowKernel row_kernel(int K) {
  switch (K) {
    case 12: return rht_rows_kernel<12>;
    case 20: return rht_rows_kernel<20>;
    case 28: return rht_rows_kernel<28>;
    case 36: return rht_rows_kernel<36>;
    default: return rht_rows_kernel<0>;
  }
}
using PipeKernel = void (*)(float*, long, long, float, const float*, const float*);
PipeKernel pipe_kernel(int K, bool transpose) {
  switch (K) {
    case 12: return transpose ? rht_rows_p1024_kernel<12, true> : rht_rows_p1024_kernel<12, false>;
    case 20: return transpose ? rht_rows_p1024_kernel<20, true> : rht_rows_p1024_kernel<20, false>;
    case 28: return transpose ? rht_rows_p1024_kernel<28, true> : rht_rows_p1024_kernel<28, false>;
    case 36: return transpose ? rht_rows_p1024_kernel<36, true> : rht_rows_p1024_kernel<36, false>;
    default: return nullptr;
  }
}
// the row kernels may use all of the LDS; told to the runtime once per device
void allow_full_lds() {
  static std::mutex mu;
  static std::vector<bool> configured;
  int dev = 0;
  QTIP_HIP(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lk(mu);
  if (configured.size() <= size_t(dev)) configured.resize(size_t(dev) + 1, false);
  if (configured[size_t(dev)]) return;
  for (int K : {0, 12, 20, 28, 36})
    QTIP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(row_kernel(K)),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, kRowLdsFloats * int(sizeof(float))));
  for (int K : {12, 20, 28, 36})
    for (bool t : {false, true})
      QTIP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(pipe_kernel(K, t)),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, kRowLdsFloats * int(sizeof(float))));
  configured[size_t(dev)] = true;
}
}  // namespace

void Rht::hadamard_rows(float* X, long rows, int n, long ld, bool transpose, const float* rs, const float* cs) {
  const int K = had_K(n);
  QTIP_REQUIRE(K > 0, "unsupported hadamard dim %d", n);
  const int P = n / K;
  QTIP_REQUIRE(P <= 8192, "hadamard pow2 part %d > 8192 unsupported", P);
  QTIP_REQUIRE(ld >= n, "hadamard: ld %ld < n %d", ld, n);
  if (rows <= 0) return;
  allow_full_lds();
  const float sc = 1.0f / std::sqrt(float(n));
  // rows of K x 1024 values that are 16-byte aligned: the form that keeps the next row in flight
  const auto aligned16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  if (P == 1024 && pipe_kernel(K, transpose) && n <= kRowLdsFloats && ld % 4 == 0 && aligned16(X) && aligned16(cs)) {
    // as many workgroups as are resident at once (a K = 12 row leaves room for two per compute unit)
    int per_cu = 1;
    QTIP_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(pipe_kernel(K, transpose)),
                                                          kRowThreads, size_t(n) * sizeof(float)));
    const unsigned grid = unsigned(std::min<long>(rows, long(cus_) * std::max(per_cu, 1)));
    pipe_kernel(K, transpose)<<<dim3(grid), dim3(kRowThreads), size_t(n) * sizeof(float), s_>>>(X, ld, rows, sc, rs, cs);
    QTIP_HIP(hipGetLastError());
    return;
  }
  const uint32_t* neg = K > 1 ? device_had(K, transpose) : nullptr;
  // a row that fits in LDS is transformed and mixed in one pass; a longer one goes chunk group by chunk group and is
  // mixed by a second kernel
  const bool whole = n <= kRowLdsFloats;
  const int seg = whole ? n : kRowLdsFloats / P * P;
  const int nseg = (n + seg - 1) / seg;
  QTIP_REQUIRE(rows * nseg < (1L << 31), "hadamard: too many rows");
  const int mix = whole && K > 1;
  const float first_scale = (K == 1) ? sc : (mix ? sc : 1.0f);
  row_kernel(K)<<<dim3(unsigned(rows * nseg)), dim3(kRowThreads), size_t(seg) * sizeof(float), s_>>>(
      X, ld, n, P, K, seg, nseg, first_scale, rs, cs, neg, mix);
  QTIP_HIP(hipGetLastError());
  if (K > 1 && !mix) {
    const long per_row = (P + kMixLanes - 1) / kMixLanes;
    QTIP_REQUIRE(rows * per_row < (1L << 31), "hadamard: too many rows");
    had_mix_long_rows_kernel<<<dim3(unsigned(rows * per_row)), dim3(kMixLanes), size_t(K) * kMixLanes * sizeof(float),
                               s_>>>(X, ld, P, K, sc, neg);
    QTIP_HIP(hipGetLastError());
  }
}

void Rht::transpose(const float* in, long rows, long cols, long ld_in, float* out, long ld_out) {
  if (rows <= 0 || cols <= 0) return;
  dim3 grid(unsigned((cols + 63) / 64), unsigned((rows + 63) / 64));
  transpose_kernel<<<grid, dim3(256), 0, s_>>>(in, rows, cols, ld_in, out, ld_out);
  QTIP_HIP(hipGetLastError());
}

void Rht::scale(float* X, long rows, long cols, long ld, float a) {
  if (rows * cols <= 0) return;
  for (long r0 = 0; r0 < rows; r0 += 65535) {  // the grid's second dimension holds 65535 rows
    const long nr = std::min<long>(65535, rows - r0);
    scale_kernel<<<dim3(unsigned((cols + 1023) / 1024), unsigned(nr)), dim3(256), 0, s_>>>(X + r0 * ld, nr, cols, ld, a);
  }
  QTIP_HIP(hipGetLastError());
}

void Rht::add_diag(float* H, long n, float a) {
  add_diag_kernel<<<dim3(unsigned((n + 255) / 256)), dim3(256), 0, s_>>>(H, n, a);
  QTIP_HIP(hipGetLastError());
}

double Rht::reduce(const float* A, long lda, const float* B, long ldb, long rows, long cols, int mode) {
  const long total = mode == 3 ? rows : rows * cols;
  if (total <= 0) return 0.0;
  int blocks = int(std::min<long>(kRedBlocks, (total + kRedThreads - 1) / kRedThreads));
  reduce_partial_kernel<<<dim3(blocks), dim3(kRedThreads), 0, s_>>>(A, lda, B, ldb, rows, cols, mode, partial_);
  QTIP_HIP(hipGetLastError());
  reduce_final_kernel<<<dim3(1), dim3(kRedThreads), 0, s_>>>(partial_, blocks, partial_ + kRedBlocks);
  QTIP_HIP(hipGetLastError());
  double h = 0;
  QTIP_HIP(hipMemcpyAsync(&h, partial_ + kRedBlocks, sizeof(double), hipMemcpyDeviceToHost, s_));
  QTIP_HIP(hipStreamSynchronize(s_));
  return h;
}

}  // namespace qtipmi
