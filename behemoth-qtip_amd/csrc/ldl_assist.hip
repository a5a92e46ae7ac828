// Host fp64 block LDL with the trailing updates on the GPU (host_ldl.cpp, block_ldl_assisted): the host factors and
// solves one 256-column panel at a time in its own arithmetic, the device holds the symmetric fp64 work matrix and
// applies the rank-256 updates.  v_mfma_f64_16x16x4_f64 accumulates its four products like a chain of fused
// multiply-adds in ascending k (checked bit for bit against std::fma chains), and the host's micro-kernels form every
// element of an update as exactly such a chain over the panel depth from zero followed by one subtraction, so the
// factor is the host's bit for bit.
#include <algorithm>

#include "quantizer_impl.hpp"

namespace qtipmi {
namespace {

typedef double double4_t __attribute__((ext_vector_type(4)));

// A[i][j] = (H[i][j] + H[j][i]) / 2 in fp64, lower triangle (symmetrize_lower_host)
__global__ void symmetrize_lower_kernel(const float* __restrict__ H, long n, double* __restrict__ A) {
  const long j = long(blockIdx.x) * blockDim.x + threadIdx.x, i = blockIdx.y;
  if (j > i || j >= n) return;
  A[i * n + j] = 0.5 * (double(H[i * n + j]) + double(H[j * n + i]));
}

// Xt[p][i] = X[i][p]: the solved rows arrive row by row (nr x kb); the update reads them column by column
__global__ __launch_bounds__(256) void transpose_panel_kernel(const double* __restrict__ X, int nr, int kb,
                                                            double* __restrict__ Xt) {
  __shared__ double tile[32][33];
  const int i0 = blockIdx.x * 32, p0 = blockIdx.y * 32, tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  for (int r = ty; r < 32; r += 8)
    if (i0 + r < nr && p0 + tx < kb) tile[r][tx] = X[long(i0 + r) * kb + p0 + tx];
  __syncthreads();
  for (int r = ty; r < 32; r += 8)
    if (p0 + r < kb && i0 + tx < nr) Xt[long(p0 + r) * nr + i0 + tx] = tile[tx][r];
}

// dst[i][0 .. kb) = A[i][0 .. kb) for `rows` rows (A: row stride lda): the columns of a panel, packed, so that they
// travel to the host as one contiguous copy (a pitched copy of 2 KB rows runs at a fraction of the link's rate)
__global__ __launch_bounds__(256) void gather_panel_kernel(const double* __restrict__ A, long lda, long rows, int kb,
                                                         double* __restrict__ dst) {
  const long per_row = kb / 2, total = rows * per_row;  // kb is even: two doubles per thread
  for (long e = long(blockIdx.x) * blockDim.x + threadIdx.x; e < total; e += long(gridDim.x) * blockDim.x) {
    const long i = e / per_row, c = (e % per_row) * 2;
    *reinterpret_cast<double2*>(dst + i * kb + c) = *reinterpret_cast<const double2*>(A + i * lda + c);
  }
}

// C -= acc for a wave's 64 x 64 outputs (rows i0 .., columns j0 ..; only i < nr, j <= i exist).  A block that lies
// inside the triangle altogether (nearly all do) fetches the 16 values of a row block together, so it waits for 4
// round trips to memory, not 64; the others go element by element.
__device__ __forceinline__ void subtract_tile(const double4_t (&acc)[4][4], double* __restrict__ C, long ldc, int nr,
                                              int i0, int j0, int lane) {
  if (i0 + 64 <= nr && j0 + 63 <= i0) {  // the same for the whole wave
    double* base = C + long(i0 + (lane >> 4)) * ldc + j0 + (lane & 15);
#pragma unroll
    for (int mi = 0; mi < 4; ++mi) {
      double c[4][4];
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const double* row = base + long(mi * 16 + 4 * v) * ldc;
#pragma unroll
        for (int ni = 0; ni < 4; ++ni) c[ni][v] = row[ni * 16];
      }
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        double* row = base + long(mi * 16 + 4 * v) * ldc;
#pragma unroll
        for (int ni = 0; ni < 4; ++ni) row[ni * 16] = c[ni][v] - acc[mi][ni][v];
      }
    }
    return;
  }
#pragma unroll
  for (int mi = 0; mi < 4; ++mi)
#pragma unroll
    for (int ni = 0; ni < 4; ++ni)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int gi = i0 + mi * 16 + (lane >> 4) + 4 * v, gj = j0 + ni * 16 + (lane & 15);
        if (gi < nr && gj <= gi) C[long(gi) * ldc + gj] -= acc[mi][ni][v];
      }
}

// C[i][j] -= sum_p X[i][p] * X[j][p] for one 128 x 128 tile of the nr x nr lower triangle, every element one chain
// over p = 0 .. kb-1 from zero, then one subtraction.  Xt: kb x nr (the transposed solved rows, row stride ldx; nr and
// ldx multiples of 4, kb a multiple of 8), C: row stride ldc.  strip_tiles = 0: the grid enumerates the tiles
// (bi, bj <= bi) of the whole triangle; strip_tiles = w > 0: only the first w tile columns, grid = w x row tiles
// (the columns of the next panel, which the host wants back before the rest of the update has run).
// 256 threads, 2 x 2 waves of 64 x 64.  The workgroups share the chip with the Viterbi kernel's (168 registers, 50 KB
// of LDS each, three per CU), so this one stays within 168 registers and 48 KB of LDS and takes the place of one of
// them, not two: the operand slices go from global memory straight into LDS (global_load_lds_dwordx4: a wave's 64
// lanes fill one 1 KB row of 128 doubles), eight columns of the panel per stage, three stages in flight, one
// barrier per stage, no staging registers; fragment reads and loads go one at a time under the MFMAs (see the loop).
// Lanes beyond nr in the last tile row read whatever follows in Xt (the caller's buffer extends at least 128 doubles
// beyond the last row read); those columns only feed outputs that are never stored.
constexpr int UT = 128;
constexpr int VK = 8, VSTAGES = 3;
__global__ __launch_bounds__(256, 3) void rank_update_lower_kernel(const double* __restrict__ Xt, long ldx, int nr,
                                                                     int kb, double* __restrict__ C, long ldc,
                                                                     int strip_tiles) {
  int bi, bj;
  if (strip_tiles > 0) {
    bi = blockIdx.x / strip_tiles;
    bj = blockIdx.x % strip_tiles;
    if (bj > bi) return;
  } else {
    // tile index t -> row bi with bi (bi + 1) / 2 <= t: the square root in fp32, then one step either way
    const int t = blockIdx.x;
    bi = int((__builtin_sqrtf(8.0f * float(t) + 1.0f) - 1.0f) * 0.5f);
    while (bi * (bi + 1) / 2 > t) --bi;
    while ((bi + 1) * (bi + 2) / 2 <= t) ++bi;
    bj = t - bi * (bi + 1) / 2;
  }
  const int i0 = bi * UT, j0 = bj * UT;
  __shared__ __attribute__((aligned(16))) double S[VSTAGES][2][VK][UT];  // [stage][Xi | Xj][k][column]
  const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6), wm = wave >> 1, wn = wave & 1;
  double4_t acc[4][4];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b) acc[a][b] = double4_t{0, 0, 0, 0};
  // wave w brings rows 2w and 2w + 1 of a stage's Xi and Xj slices; gi / gj: this lane's piece of the next slice to
  // be requested, `asked` its number
  const double* gi = Xt + long(2 * wave) * ldx + i0 + 2 * lane;
  const double* gj = Xt + long(2 * wave) * ldx + j0 + 2 * lane;
  const long slice_stride = long(VK) * ldx;
  int asked = 0;
  typedef __attribute__((address_space(3))) void* lds_ptr;
  auto load1 = [&](int st, int q) {  // into stage st; q = 0, 1: rows 2w, 2w + 1 of Xi; 2, 3: of Xj
    const int r = q & 1;
    if (q < 2) __builtin_amdgcn_global_load_lds(gi + r * ldx, (lds_ptr)&S[st][0][2 * wave + r][0], 16, 0, 0);
    else __builtin_amdgcn_global_load_lds(gj + r * ldx, (lds_ptr)&S[st][1][2 * wave + r][0], 16, 0, 0);
  };
  auto asked_one = [&] {
    gi += slice_stride, gj += slice_stride, ++asked;
    // the two running pointers as they are: without this the compiler keeps one pointer per load of the unrolled
    // loop, two dozen registers that the accumulators leave no room for
    asm volatile("" : "+v"(gi), "+v"(gj));
  };
  const int slices = kb / VK;  // kb is a multiple of 16
  // fragments of the 4 k of step ks (0, 1) of the slice in stage st: a[set][mi], b[set][ni]
  const int c16 = lane & 15, kq = lane >> 4;
  double fa[2][4], fb[2][4];
  auto read1 = [&](int st, int ks, int set, int j) {  // j = 0..7 in the order the MFMAs first use them: a0 b0 b1 b2 b3 a1 a2 a3
    const int kr = 4 * ks + kq;
    if (j == 0 || j >= 5) {
      const int mi = j == 0 ? 0 : j - 4;
      fa[set][mi] = S[st][0][kr][wm * 64 + mi * 16 + c16];
    } else {
      const int ni = j - 1;
      fb[set][ni] = S[st][1][kr][wn * 64 + ni * 16 + c16];
    }
  };
  auto mfma = [&](int set, int j) {
    const int mi = j >> 2, ni = j & 3;
    acc[mi][ni] = __builtin_amdgcn_mfma_f64_16x16x4f64(fa[set][mi], fb[set][ni], acc[mi][ni], 0, 0, 0);
  };
  // Slices 0 and 1 requested, slice 0 landed (this wave's loads, then everyone's: a bare barrier, which does not wait
  // for the loads still in flight), slice 2 requested, the fragments of slice 0's first 4 k read.
  load1(0, 0), load1(0, 1), load1(0, 2), load1(0, 3);
  asked_one();
  if (slices > 1) {
    load1(1, 0), load1(1, 1), load1(1, 2), load1(1, 3);
    asked_one();
  }
  if (slices > 1) __builtin_amdgcn_s_waitcnt(0x0F74);  // vmcnt(4)
  else __builtin_amdgcn_s_waitcnt(0x0F70);             // vmcnt(0)
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  if (asked < slices) {
    load1(2, 0), load1(2, 1), load1(2, 2), load1(2, 3);
    asked_one();
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) read1(0, 0, 0, j);
  // One slice: 32 MFMAs, two steps of 4 k on fragment sets 0 and 1.  The workgroup runs beside the Viterbi kernel's,
  // one wave per SIMD with nothing to hide a wait behind but its own MFMAs (32 cycles each, during which the wave may
  // issue other work): under every other MFMA of a step it reads one fragment of the next step, and under MFMAs 1, 5,
  // 9, 13 of the second step it requests one row of slice sl + 3 - after the barrier in the middle, which says slice
  // sl + 1 has landed everywhere and every wave has asked for its last fragments of slice sl, whose stage is
  // therefore free.  The scheduling barriers pin that order.  kSteady: every slice asked for exists and one more is
  // on its way beyond sl + 1, so vmcnt(4) = "slice sl + 1 is here"; the last slices run the same code with the
  // conditions and a full wait.
#define QTIP_SB __builtin_amdgcn_sched_barrier(0)
  auto slice = [&](auto steady, auto stage, int sl) {  // slice sl, which lies in stage sl % VSTAGES = stage
    constexpr bool kSteady = decltype(steady)::value;
    constexpr int st = decltype(stage)::value, nst = (st + 1) % VSTAGES;
    const bool next = kSteady || sl + 1 < slices;
#define QTIP_M0(j) { mfma(0, j); QTIP_SB; }
#define QTIP_R0(j) { mfma(0, j); QTIP_SB; read1(st, 1, 1, (j) / 2); QTIP_SB; }
    QTIP_SB;
    QTIP_R0(0) QTIP_M0(1) QTIP_R0(2) QTIP_M0(3) QTIP_R0(4) QTIP_M0(5) QTIP_R0(6) QTIP_M0(7)
    QTIP_R0(8) QTIP_M0(9) QTIP_R0(10) QTIP_M0(11) QTIP_R0(12) QTIP_M0(13) QTIP_R0(14) QTIP_M0(15)
    if (next) {
      // this wave's part of slice sl + 1 has landed and its reads of slice sl have returned
      if (kSteady) __builtin_amdgcn_s_waitcnt(0x0074);  // vmcnt(4) lgkmcnt(0)
      else __builtin_amdgcn_s_waitcnt(0x0070);          // vmcnt(0) lgkmcnt(0)
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
    }
    const bool go = kSteady || asked < slices;
#define QTIP_M1(j) { mfma(1, j); QTIP_SB; }
#define QTIP_R1(j) { mfma(1, j); QTIP_SB; if (next) read1(nst, 0, 0, (j) / 2); QTIP_SB; }
#define QTIP_L1(j) { mfma(1, j); QTIP_SB; if (go) load1(st, ((j) - 1) / 4); QTIP_SB; }
    QTIP_SB;
    QTIP_R1(0) QTIP_L1(1) QTIP_R1(2) QTIP_M1(3) QTIP_R1(4) QTIP_L1(5) QTIP_R1(6) QTIP_M1(7)
    QTIP_R1(8) QTIP_L1(9) QTIP_R1(10) QTIP_M1(11) QTIP_R1(12) QTIP_L1(13) QTIP_R1(14) QTIP_M1(15)
    if (go) asked_one();
  };
  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1>;
  using S2 = std::integral_constant<int, 2>;
  static_assert(VSTAGES == 3);
  int sl = 0;
  for (; sl + 5 < slices; sl += 3) {
    slice(std::true_type{}, S0{}, sl);
    slice(std::true_type{}, S1{}, sl + 1);
    slice(std::true_type{}, S2{}, sl + 2);
  }
  for (; sl < slices; sl += 3) {  // the last 3 to 5 slices (or all, of fewer)
    slice(std::false_type{}, S0{}, sl);
    if (sl + 1 < slices) slice(std::false_type{}, S1{}, sl + 1);
    if (sl + 2 < slices) slice(std::false_type{}, S2{}, sl + 2);
  }
#undef QTIP_M0
#undef QTIP_R0
#undef QTIP_M1
#undef QTIP_R1
#undef QTIP_L1
#undef QTIP_SB
  // the lane number anew: the loop leaves no register to keep it in
  const int ln = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
  subtract_tile(acc, C, ldc, nr, i0 + wm * 64, j0 + wn * 64, ln);
}

// The panels travel one ahead of the updates: as soon as panel k is solved its rows go up, the update of the next
// panel's columns alone (a strip of the trailing matrix) is queued, those columns start on their way down into the
// other page-locked buffer, and only then the rest of update k is queued - the host factors and solves panel k + 1
// while that rest runs.  Every element still receives exactly one update per panel, the same chain as before.
struct DeviceTrailing final : PanelAssist {
  qtip_ctx* c;
  long n;
  hipStream_t s;
  const float* host_L;
  float* dev_L;  // optional: L is also left on the device, column block by column block as it is assembled
  hipEvent_t fetched = nullptr;
  int cur = 0;          // page-locked buffer holding the panel the host works on
  long ahead_k = -1;    // first column of the panel on its way into buffer cur ^ 1
  DeviceTrailing(qtip_ctx* c_, long n_, const float* hL, float* dL) : c(c_), n(n_), s(c_->ldl_stream), host_L(hL), dev_L(dL) {
    QTIP_HIP(hipEventCreateWithFlags(&fetched, hipEventDisableTiming));
  }
  ~DeviceTrailing() override {
    if (fetched) (void)hipEventDestroy(fetched);
  }
  void copy_down(long k, long kb, double* dst) {
    const long rows = n - k, pairs = rows * (kb / 2);
    gather_panel_kernel<<<dim3(unsigned(std::min<long>((pairs + 255) / 256, 4096))), dim3(256), 0, s>>>(
        c->ldl_A.p + k * n + k, n, rows, int(kb), c->ldl_P.p);
    QTIP_HIP(hipGetLastError());
    QTIP_HIP(hipMemcpyAsync(dst, c->ldl_P.p, size_t(rows) * kb * 8, hipMemcpyDeviceToHost, s));
  }
  void assembled(int k, int kb) override {
    if (!dev_L) return;
    QTIP_HIP(hipMemcpy2DAsync(dev_L + k, size_t(n) * 4, host_L + k, size_t(n) * 4, size_t(kb) * 4, size_t(n),
                              hipMemcpyHostToDevice, s));
  }
  double* fetch(int k, int kb) override {
    if (ahead_k == k) {
      cur ^= 1;
      QTIP_HIP(hipEventSynchronize(fetched));
    } else {
      copy_down(k, kb, c->ldl_panel[cur].p);
      QTIP_HIP(hipStreamSynchronize(s));
    }
    ahead_k = -1;
    return c->ldl_panel[cur].p;
  }
  void update(const double* Xt, long ldx, long nr, int kb, double* C, int strip_tiles) {
    const long nt = (nr + UT - 1) / UT, grid = strip_tiles ? nt * strip_tiles : nt * (nt + 1) / 2;
    // what the kernel assumes: whole stages of 8 panel columns, and readable memory up to the end of the last tile
    // row's 128 columns in every row of Xt
    QTIP_REQUIRE(kb % VK == 0 && Xt >= c->ldl_Xt.p && size_t(Xt - c->ldl_Xt.p) + size_t(kb - 1) * ldx + size_t(nt) * UT <= c->ldl_Xt.n,
                 "LDL update: operand shape the kernel does not cover (kb = %d, nr = %ld)", kb, nr);
    rank_update_lower_kernel<<<dim3(unsigned(grid)), dim3(256), 0, s>>>(Xt, ldx, int(nr), kb, C, n, strip_tiles);
    QTIP_HIP(hipGetLastError());
  }
  void solved(int k, int kb, const double* panel) override {
    const long r0 = k + kb, nr = n - r0;
    if (nr <= 0) return;
    // the stream orders this copy before the next fetch into the same page-locked buffer
    QTIP_HIP(hipMemcpyAsync(c->ldl_X.p, panel + long(kb) * kb, size_t(nr) * kb * 8, hipMemcpyHostToDevice, s));
    transpose_panel_kernel<<<dim3(unsigned((nr + 31) / 32), unsigned((kb + 31) / 32)), dim3(256), 0, s>>>(
        c->ldl_X.p, int(nr), kb, c->ldl_Xt.p);
    QTIP_HIP(hipGetLastError());
    double* C = c->ldl_A.p + r0 * n + r0;
    const long next_kb = std::min<long>(ldl_panel_width(), nr), strip = (next_kb + UT - 1) / UT, done = strip * UT;
    update(c->ldl_Xt.p, nr, nr, kb, C, int(strip));
    copy_down(r0, next_kb, c->ldl_panel[cur ^ 1].p);
    QTIP_HIP(hipEventRecord(fetched, s));
    ahead_k = r0;
    if (nr > done) update(c->ldl_Xt.p + done, nr, nr - done, kb, C + done * n + done, 0);
  }
};

__global__ void add_to_diagonal_kernel(double* __restrict__ A, long n, double v) {
  const long i = blockIdx.x * long(blockDim.x) + threadIdx.x;
  if (i < n) A[i * n + i] += v;
}

}  // namespace

// The Hessian preparation of the calibrated NVFP4 quantizer (nvfp4_prepare_host) with the trailing updates of its
// Cholesky factorization on the device: same panels, same chains, hence the same L and dw bit for bit.
void nvfp4_prepare_assisted_impl(qtip_ctx* c, const float* host_H, int n, double sigma_reg, int threads, float* host_L,
                                 float* host_dw) {
  QTIP_REQUIRE(c && host_H && host_L && host_dw && n > 0 && n % 16 == 0, "nvfp4_prepare (device updates): bad arguments (n = %d)", n);
  QTIP_REQUIRE(n <= 65535, "nvfp4_prepare (device updates): n = %d is beyond one grid dimension", n);
  double dsum = 0;
  for (int i = 0; i < n; ++i) dsum += host_H[size_t(i) * n + i];
  const double creg = sigma_reg * dsum / n;
  if (!c->ldl_stream) QTIP_HIP(hipStreamCreateWithFlags(&c->ldl_stream, hipStreamNonBlocking));
  hipStream_t s = c->ldl_stream;
  const size_t nn = size_t(n) * n, nb = size_t(ldl_panel_width());
  c->ldl_A.ensure(nn);
  c->ldl_H.ensure(nn);
  c->ldl_X.ensure(size_t(n) * nb);
  c->ldl_Xt.ensure(size_t(n) * nb);
  c->ldl_P.ensure(size_t(n) * nb);
  for (auto& buf : c->ldl_panel)
    if (buf.n < size_t(n) * nb) buf.alloc(size_t(n) * nb);
  QTIP_HIP(hipMemcpyAsync(c->ldl_H.p, host_H, nn * 4, hipMemcpyHostToDevice, s));
  symmetrize_lower_kernel<<<dim3(unsigned((n + 255) / 256), unsigned(n)), dim3(256), 0, s>>>(c->ldl_H.p, n, c->ldl_A.p);
  QTIP_HIP(hipGetLastError());
  add_to_diagonal_kernel<<<dim3(unsigned((n + 255) / 256)), dim3(256), 0, s>>>(c->ldl_A.p, n, creg);
  QTIP_HIP(hipGetLastError());
  DeviceTrailing dev(c, n, nullptr, nullptr);
  bool ok = false;
  try {
    ok = scalar_ldl_assisted(n, host_L, host_dw, threads, dev);
  } catch (...) {
    (void)hipStreamSynchronize(s);
    throw;
  }
  QTIP_HIP(hipStreamSynchronize(s));
  if (!ok) throw Error(QTIP_E_NOT_PD, "NVFP4 calibration: Hessian not positive definite");
}

// dev_HRr (optional): the rotated Hessian already on the device (then host_HRr is not read)
// dev_L (optional): n x n device buffer that receives L as well
void ldl_hessian_assisted_impl(qtip_ctx* c, const float* host_HRr, int n, int threads, float* host_L,
                               const float* dev_HRr, float* dev_L) {
  QTIP_REQUIRE(c && n > 0 && n % 16 == 0 && (host_HRr || dev_HRr) && host_L,
               "ldl_hessian (device updates): bad arguments (n = %d)", n);
  QTIP_REQUIRE(n <= 65535, "ldl_hessian (device updates): n = %d is beyond one grid dimension", n);
  if (!c->ldl_stream) QTIP_HIP(hipStreamCreateWithFlags(&c->ldl_stream, hipStreamNonBlocking));
  hipStream_t s = c->ldl_stream;
  const size_t nn = size_t(n) * n, nb = size_t(ldl_panel_width());
  c->ldl_A.ensure(nn);
  if (!dev_HRr) c->ldl_H.ensure(nn);
  c->ldl_X.ensure(size_t(n) * nb);
  c->ldl_Xt.ensure(size_t(n) * nb);
  c->ldl_P.ensure(size_t(n) * nb);
  for (auto& buf : c->ldl_panel)
    if (buf.n < size_t(n) * nb) buf.alloc(size_t(n) * nb);
  if (!dev_HRr) QTIP_HIP(hipMemcpyAsync(c->ldl_H.p, host_HRr, nn * 4, hipMemcpyHostToDevice, s));
  symmetrize_lower_kernel<<<dim3(unsigned((n + 255) / 256), unsigned(n)), dim3(256), 0, s>>>(dev_HRr ? dev_HRr : c->ldl_H.p, n,
                                                                                              c->ldl_A.p);
  QTIP_HIP(hipGetLastError());
  DeviceTrailing dev(c, n, host_L, dev_L);
  bool ok = false;
  try {
    ok = block_ldl_assisted(n, host_L, threads, dev);
  } catch (...) {
    (void)hipStreamSynchronize(s);  // copies that read the caller's L must not outlive the call
    throw;
  }
  QTIP_HIP(hipStreamSynchronize(s));
  if (!ok) throw Error(QTIP_E_NOT_PD, "block LDL failed (H not PD)");
}

}  // namespace qtipmi
