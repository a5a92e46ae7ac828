// Randomised Hadamard transform pieces for gfx950: sign scaling + natural-order FWHT per power-of-two chunk,
// the K-point Hadamard-factor mix, tiled transpose, and fixed-order fp64 reductions.
//
// The fp32 operation order is the one of the reference's GPU path (src/kernels.hip:214-254, 293-313:
// butterflies (a+b, a-b) for h = 1, 2, 4, ...; mix as a signed sum over k ascending from 0; one multiply by
// 1/sqrt(n) at the end), so results match it bit for bit; only the scheduling differs: the sign scaling is
// fused into the load, the first three butterfly stages run in registers on 8 consecutive values per lane,
// and the remaining stages go through LDS.
#include "qtip_internal.hpp"
#include "rht.hpp"

namespace qtipmi {
namespace {

constexpr int kFwhtThreads = 256;

// In-place FWHT of one chunk of P values held in LDS buffer v (P <= 8192), all threads of the block.
// Stages h < 8 run in registers on 8 consecutive values; the rest through LDS.
template <int EPT>
__device__ __forceinline__ void fwht_registers(float (&r)[EPT]) {
#pragma unroll
  for (int h = 1; h < EPT; h <<= 1)
#pragma unroll
    for (int i = 0; i < EPT; i += 2 * h)
#pragma unroll
      for (int j = i; j < i + h; ++j) {
        const float a = r[j], b = r[j + h];
        r[j] = a + b;
        r[j + h] = a - b;
      }
}

// grid: rows * K blocks; block b handles chunk (b % K) of row (b / K)
__global__ __launch_bounds__(kFwhtThreads) void fwht_chunks_kernel(float* __restrict__ X, long ld, int P, int K,
                                                                   float scale, const float* __restrict__ rs,
                                                                   const float* __restrict__ cs, int vec) {
  __shared__ float v[8192];
  const long row = blockIdx.x / K;
  const int chunk = blockIdx.x % K;
  float* x = X + row * ld + long(chunk) * P;
  const float rsv = rs ? rs[row] : 1.0f;
  const int t = threadIdx.x;
  if (vec) {  // P >= 8 and every chunk start is 16-byte aligned
    // 8 consecutive values per thread and sweep; stages 1, 2, 4 in registers
    for (int base = 8 * t; base < P; base += 8 * kFwhtThreads) {
      float r[8];
      const float4 lo = *reinterpret_cast<const float4*>(x + base);
      const float4 hi = *reinterpret_cast<const float4*>(x + base + 4);
      r[0] = lo.x, r[1] = lo.y, r[2] = lo.z, r[3] = lo.w, r[4] = hi.x, r[5] = hi.y, r[6] = hi.z, r[7] = hi.w;
      if (rs) {
#pragma unroll
        for (int e = 0; e < 8; ++e) r[e] *= rsv;
      }
      if (cs) {
        const float* c = cs + long(chunk) * P + base;
#pragma unroll
        for (int e = 0; e < 8; ++e) r[e] *= c[e];
      }
      fwht_registers<8>(r);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[base + e] = r[e];
    }
    __syncthreads();
    for (int h = 8; h < P; h <<= 1) {
      for (int k = t; k < P / 2; k += kFwhtThreads) {
        const int i = (k / h) * 2 * h + (k % h);
        const float a = v[i], b = v[i + h];
        v[i] = a + b;
        v[i + h] = a - b;
      }
      __syncthreads();
    }
  } else {
    for (int i = t; i < P; i += kFwhtThreads) {
      float a = x[i];
      if (rs) a *= rsv;
      if (cs) a *= cs[long(chunk) * P + i];
      v[i] = a;
    }
    __syncthreads();
    for (int h = 1; h < P; h <<= 1) {
      for (int k = t; k < P / 2; k += kFwhtThreads) {
        const int i = (k / h) * 2 * h + (k % h);
        const float a = v[i], b = v[i + h];
        v[i] = a + b;
        v[i + h] = a - b;
      }
      __syncthreads();
    }
  }
  if (scale != 1.0f) {
    for (int i = t; i < P; i += kFwhtThreads) x[i] = v[i] * scale;
  } else {
    for (int i = t; i < P; i += kFwhtThreads) x[i] = v[i];
  }
}

// y[k2*P + i] = (sum_k sign[k2][k] * y[k*P + i]) * scale, one thread per (row, i)
template <int K>
__global__ __launch_bounds__(256) void had_mix_kernel(float* __restrict__ X, long rows, int P, long ld,
                                                      const int8_t* __restrict__ had, float scale) {
  __shared__ int8_t hs[K * K];
  for (int i = threadIdx.x; i < K * K; i += blockDim.x) hs[i] = had[i];
  __syncthreads();
  const long idx = long(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= rows * P) return;
  const long row = idx / P;
  const int i = int(idx % P);
  float* x = X + row * ld + i;
  float y[K];
#pragma unroll
  for (int k = 0; k < K; ++k) y[k] = x[long(k) * P];
#pragma unroll
  for (int k2 = 0; k2 < K; ++k2) {
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < K; ++k) s += hs[k2 * K + k] > 0 ? y[k] : -y[k];
    x[long(k2) * P] = s * scale;
  }
}

// any K: the K inputs of a thread are parked in a global scratch column
__global__ __launch_bounds__(256) void had_mix_generic_kernel(float* __restrict__ X, long rows, int P, int K, long ld,
                                                              const int8_t* __restrict__ had, float scale,
                                                              float* __restrict__ tmp) {
  const long idx = long(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= rows * P) return;
  const long row = idx / P;
  const int i = int(idx % P);
  float* x = X + row * ld + i;
  const long total = rows * P;
  for (int k = 0; k < K; ++k) tmp[long(k) * total + idx] = x[long(k) * P];
  for (int k2 = 0; k2 < K; ++k2) {
    float s = 0.0f;
    for (int k = 0; k < K; ++k) {
      const float t = tmp[long(k) * total + idx];
      s += had[k2 * K + k] > 0 ? t : -t;
    }
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

__global__ void scale_kernel(float* __restrict__ X, long rows, long cols, long ld, float a) {
  const long i = long(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= rows * cols) return;
  X[(i / cols) * ld + i % cols] *= a;
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
  for (long i = lo + threadIdx.x; i < hi; i += kRedThreads) {
    if (mode == 3) {
      acc += double(A[i * lda + i]);
    } else {
      const long r = i / cols, c = i % cols;
      const double a = A[r * lda + c];
      if (mode == 0) acc += a * a;
      else {
        const double b = B[r * ldb + c];
        if (mode == 1) acc += a * b;
        else acc += (a - b) * (a - b);
      }
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

const int8_t* Rht::device_had(int K, bool transpose) {
  const int key = K * 2 + (transpose ? 1 : 0);
  for (auto& e : had_) if (e.first == key) return e.second->p;
  auto m = had_matrix(K, transpose);
  auto buf = std::make_unique<DBuf<int8_t>>(m.size());
  QTIP_HIP(hipMemcpyAsync(buf->p, m.data(), m.size(), hipMemcpyHostToDevice, s_));
  QTIP_HIP(hipStreamSynchronize(s_));
  had_.emplace_back(key, std::move(buf));
  return had_.back().second->p;
}

void Rht::hadamard_rows(float* X, long rows, int n, long ld, bool transpose, const float* rs, const float* cs) {
  const int K = had_K(n);
  QTIP_REQUIRE(K > 0, "unsupported hadamard dim %d", n);
  const int P = n / K;
  QTIP_REQUIRE(P <= 8192, "hadamard pow2 part %d > 8192 unsupported", P);
  QTIP_REQUIRE(ld >= n, "hadamard: ld %ld < n %d", ld, n);
  if (rows <= 0) return;
  const float sc = 1.0f / std::sqrt(float(n));
  QTIP_REQUIRE(rows * K < (1L << 31), "hadamard: too many chunks");
  const int vec = (P >= 8 && ld % 4 == 0 && (reinterpret_cast<uintptr_t>(X) & 15u) == 0) ? 1 : 0;
  fwht_chunks_kernel<<<dim3(unsigned(rows * K)), dim3(kFwhtThreads), 0, s_>>>(X, ld, P, K, K == 1 ? sc : 1.0f, rs, cs,
                                                                               vec);
  QTIP_HIP(hipGetLastError());
  if (K == 1) return;
  const int8_t* had = device_had(K, transpose);
  const unsigned nb = unsigned((rows * P + 255) / 256);
  switch (K) {
    case 12: had_mix_kernel<12><<<nb, 256, 0, s_>>>(X, rows, P, ld, had, sc); break;
    case 20: had_mix_kernel<20><<<nb, 256, 0, s_>>>(X, rows, P, ld, had, sc); break;
    case 28: had_mix_kernel<28><<<nb, 256, 0, s_>>>(X, rows, P, ld, had, sc); break;
    case 36: had_mix_kernel<36><<<nb, 256, 0, s_>>>(X, rows, P, ld, had, sc); break;
    default: {
      DBuf<float> tmp(size_t(rows) * P * K);
      had_mix_generic_kernel<<<nb, 256, 0, s_>>>(X, rows, P, K, ld, had, sc, tmp);
      QTIP_HIP(hipGetLastError());
      QTIP_HIP(hipStreamSynchronize(s_));  // tmp is released on return
    }
  }
  QTIP_HIP(hipGetLastError());
}

void Rht::transpose(const float* in, long rows, long cols, long ld_in, float* out, long ld_out) {
  if (rows <= 0 || cols <= 0) return;
  dim3 grid(unsigned((cols + 63) / 64), unsigned((rows + 63) / 64));
  transpose_kernel<<<grid, dim3(256), 0, s_>>>(in, rows, cols, ld_in, out, ld_out);
  QTIP_HIP(hipGetLastError());
}

void Rht::scale(float* X, long rows, long cols, long ld, float a) {
  if (rows * cols <= 0) return;
  scale_kernel<<<dim3(unsigned((rows * cols + 255) / 256)), dim3(256), 0, s_>>>(X, rows, cols, ld, a);
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
