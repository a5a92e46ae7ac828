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
