// NVFP4 fallback quantizer, host side: the format's scalar helpers, the plain nearest-value quantizer and the
// dequantizer (reference src/nvfp4.hpp:15-57, src/nvfp4.cpp:12-70), the Hessian preparation of the calibrated
// quantizer (src/nvfp4_gpu.hip:181-207) and the driver of its device block loop (src/nvfp4_gpu.hip:209-241).
#include <cmath>
#include <cstring>

#include "host_team.hpp"
#include "nvfp4_codec.hpp"
#include "quantizer_impl.hpp"

namespace qtipmi {
namespace {

// one fp32 global scale per matrix: the largest magnitude lands on the largest representable product 448 * 6
float global_scale(const float* w, size_t numel) {
  float top = 0;
  bool finite = true;
  for (size_t i = 0; i < numel; ++i) {
    const float a = std::fabs(w[i]);
    finite = finite && a <= 3.4028234663852886e38f;  // false for infinity and NaN
    top = a > top ? a : top;
  }
  QTIP_REQUIRE(finite, "NVFP4: the matrix holds a value that is not finite");
  const float g = top > 0 ? top / (448.f * 6) : 1.f;
  QTIP_REQUIRE(g > 0 && g <= 3.4028234663852886e38f, "NVFP4: global scale %g is not a positive finite float", double(g));
  return g;
}

// value of a scale byte as stored: NaN for the two NaN codes, negative for a set sign bit
inline float scale_byte_value(uint8_t b) {
  if ((b & 0x7f) == 0x7f) return NAN;
  const float v = nvcodec::e4m3_value(b & 0x7fu);
  return b & 0x80 ? -v : v;
}

}  // namespace

uint8_t f32_to_fp8e4m3(float x) {  // src/nvfp4.hpp:15-33
  const uint8_t sign = uint8_t(nvcodec::bits_of(x) >> 31 << 7);
  if (x != x) return uint8_t(sign | 127);
  return uint8_t(sign | nvcodec::e4m3_of_magnitude(x));
}

void nvfp4_quantize_host(const float* w, int m, int n, uint8_t* packed, uint8_t* scales, float* global) {
  QTIP_REQUIRE(w && packed && scales && global && m > 0 && n > 0 && n % 16 == 0, "NVFP4 needs n %% 16 == 0 (m=%d n=%d)", m, n);
  const long blocks = long(m) * n / 16;
  const float g = global_scale(w, size_t(blocks) * 16);
  *global = g;
  HostTeam team(blocks >= (1 << 16) ? 16 : 1);
  team.parallel_for(blocks, 4096, [&](long b) {
    const float* x = w + b * 16;
    float top = 0;
    for (int j = 0; j < 16; ++j) top = std::fmax(top, std::fabs(x[j]));
    const uint32_t code = nvcodec::e4m3_of_magnitude(top / (6 * g));
    scales[b] = uint8_t(code);
    const float unit = nvcodec::e4m3_value(code) * g;
    uint8_t* out = packed + b * 8;
    for (int j = 0; j < 8; ++j) {
      // a zero unit (an all-zero block, or one below the smallest scale) stores plain zeros
      const float lo = unit ? x[2 * j] / unit : 0.f, hi = unit ? x[2 * j + 1] / unit : 0.f;
      const uint32_t nl = (nvcodec::bits_of(lo) >> 31 << 3) | nvcodec::e2m1_of_magnitude(std::fabs(lo));
      const uint32_t nh = (nvcodec::bits_of(hi) >> 31 << 3) | nvcodec::e2m1_of_magnitude(std::fabs(hi));
      out[j] = uint8_t(nl | (nh << 4));
    }
  });
}

void nvfp4_dequantize_host(const uint8_t* packed, const uint8_t* scales, float global, int m, int n, float* out) {
  QTIP_REQUIRE(packed && scales && out && m > 0 && n > 0 && n % 16 == 0, "NVFP4 dequantize: bad arguments (m=%d n=%d)", m, n);
  QTIP_REQUIRE(global > 0 && global <= 3.4028234663852886e38f, "NVFP4 dequantize: global scale %g is not a positive finite float",
               double(global));
  const long blocks = long(m) * n / 16;
  for (long b = 0; b < blocks; ++b) {
    const float s = scale_byte_value(scales[b]);
    QTIP_REQUIRE(s >= 0 && s <= 448.f, "NVFP4 dequantize: block %ld has the scale byte 0x%02x (NaN or negative)", b, scales[b]);
  }
  HostTeam team(blocks >= (1 << 16) ? 16 : 1);
  team.parallel_for(blocks, 4096, [&](long b) {
    const float s = scale_byte_value(scales[b]);
    for (int j = 0; j < 16; ++j) {
      const uint32_t nib = (packed[b * 8 + j / 2] >> (4 * (j & 1))) & 15u;
      const float mag = nvcodec::e2m1_value(nib & 7u);
      out[b * 16 + j] = nvcodec::through_bf16((nib & 8u ? -mag : mag) * s * global);
    }
  });
}

// tr((W - What) H (W - What)^T) / m in fp64.  Four rows of the difference share a pass over H; every row's sums run
// over ascending columns, and the rows' results are added in row order.
double nvfp4_proxy_error_host(const float* w, const float* what, int m, int n, const float* H) {
  QTIP_REQUIRE(w && what && m > 0 && n > 0, "nvfp4_proxy_error: bad arguments");
  constexpr int kRows = 4;
  const long groups = (long(m) + kRows - 1) / kRows;
  std::vector<double> per_row(size_t(m), 0.0);
  HostTeam team(16);
  team.parallel_for(groups, 1, [&](long gi) {
    const int r0 = int(gi) * kRows, rows = std::min(kRows, m - r0);
    std::vector<double> e(size_t(kRows) * n, 0.0);
    for (int r = 0; r < rows; ++r)
      for (int j = 0; j < n; ++j) e[size_t(r) * n + j] = double(w[size_t(r0 + r) * n + j]) - double(what[size_t(r0 + r) * n + j]);
    double quad[kRows] = {0, 0, 0, 0};
    if (!H) {
      for (int r = 0; r < rows; ++r)
        for (int j = 0; j < n; ++j) quad[r] += e[size_t(r) * n + j] * e[size_t(r) * n + j];
    } else {
      for (int i = 0; i < n; ++i) {
        const float* hi = H + size_t(i) * n;
        double dot[kRows] = {0, 0, 0, 0};
        for (int j = 0; j < n; ++j) {
          const double h = double(hi[j]);
          for (int r = 0; r < kRows; ++r) dot[r] += h * e[size_t(r) * n + j];
        }
        for (int r = 0; r < kRows; ++r) quad[r] += e[size_t(r) * n + i] * dot[r];
      }
    }
    for (int r = 0; r < rows; ++r) per_row[size_t(r0 + r)] = quad[r];
  });
  double total = 0;
  for (double v : per_row) total += v;
  return total / m;
}

// Regularised Hessian -> what the block loop needs.  calibrate: unit-lower L (H = L D L^T) and dw = D; otherwise
// dw = diag(H) + creg and L is not touched.
void nvfp4_prepare_host(const float* H, int n, double sigma_reg, bool calibrate, int threads, float* L, float* dw) {
  QTIP_REQUIRE(H && dw && n > 0 && n % 16 == 0 && (!calibrate || L), "nvfp4_prepare: bad arguments");
  double dsum = 0;
  for (int i = 0; i < n; ++i) dsum += H[size_t(i) * n + i];
  const double creg = sigma_reg * dsum / n;
  if (!calibrate) {
    for (int i = 0; i < n; ++i) dw[i] = float(H[size_t(i) * n + i] + creg);
    return;
  }
  HostScratch work(size_t(n) * n * sizeof(double));
  double* A = static_cast<double*>(work.get());
  symmetrize_lower_host(H, n, A, threads);
  for (long i = 0; i < n; ++i) A[size_t(i) * n + i] += creg;
  if (!cholesky_lower_host(A, n, threads)) throw Error(QTIP_E_NOT_PD, "NVFP4 calibration: Hessian not positive definite");
#pragma omp parallel for schedule(static)
  for (long i = 0; i < n; ++i) {
    float* li = L + size_t(i) * n;
    for (long j = 0; j < i; ++j) li[j] = float(A[size_t(i) * n + j] / A[size_t(j) * n + j]);
    std::memset(li + i, 0, sizeof(float) * size_t(n - i));
  }
  for (long j = 0; j < n; ++j) {
    const double d = A[size_t(j) * n + j];
    dw[j] = float(d * d);
  }
}

// The block loop for the matrices of one group.  host_L / host_dw as nvfp4_prepare_host leaves them (host_L null:
// no calibration; host_dw null: uniform weights for the scale search).
void nvfp4_quantize_prepared_impl(qtip_ctx* c, int nmat, const qtip_nvfp4_matrix* mats, int n, const float* host_L,
                                  const float* host_dw, bool search) {
  QTIP_REQUIRE(nmat >= 0 && (nmat == 0 || mats) && n > 0 && n % 16 == 0, "NVFP4 group geometry");
  hipStream_t s = c->stream;
  const bool cal = host_L != nullptr;
  DBuf<float> d_L, d_dw;
  if (cal) {
    d_L.alloc(size_t(n) * n);
    QTIP_HIP(hipMemcpyAsync(d_L, host_L, d_L.bytes(), hipMemcpyHostToDevice, s));
  }
  if (host_dw) {
    d_dw.alloc(size_t(n));
    QTIP_HIP(hipMemcpyAsync(d_dw, host_dw, d_dw.bytes(), hipMemcpyHostToDevice, s));
  }
  for (int mi = 0; mi < nmat; ++mi) {
    const qtip_nvfp4_matrix& M = mats[mi];
    QTIP_REQUIRE(M.m > 0 && M.w && M.packed && M.scales, "NVFP4 matrix %d is incomplete", mi);
    const long m = M.m;
    const float g = global_scale(M.w, size_t(m) * n);
    const_cast<qtip_nvfp4_matrix&>(M).global = g;
    // E: the residuals W - q of the finished columns, transposed like W; all of them when they are fed back
    DBuf<float> W(size_t(m) * n), WT(size_t(m) * n), FT, E(cal ? size_t(m) * n : size_t(16) * m);
    DBuf<uint8_t> pT(size_t(m) * n / 2), sT(size_t(m) * n / 16), pk(size_t(m) * n / 2), sc(size_t(m) * n / 16);
    QTIP_HIP(hipMemcpyAsync(W, M.w, W.bytes(), hipMemcpyHostToDevice, s));
    c->rht.transpose(W, m, n, n, WT, m);
    W.release();
    // Columns go in buffers of 128 from the last to the first.  A buffer first gathers the feedback of every block
    // behind it in one pass; inside the buffer every block then feeds the columns of the buffer left of it.  Values
    // and order of the additions are those of the block-by-block form.
    const long top = (long(n) - 1) / 128 * 128;
    if (cal) {
      FT.alloc(size_t(m) * n);
      QTIP_HIP(hipMemsetAsync(FT.p + size_t(top) * m, 0, size_t(n - top) * m * sizeof(float), s));
    }
    for (long cb = top; cb >= 0; cb -= 128) {
      const long hi = std::min<long>(n, cb + 128);
      if (cal && hi < n) launch_nvfp4_gather(FT, m, n, cb, E, d_L, s);
      for (long c0 = hi - 16; c0 >= cb; c0 -= 16) {
        float* e = cal ? E.p + size_t(c0) * m : E.p;
        launch_nvfp4_block(WT, cal ? FT.p : nullptr, m, n, c0, cal ? d_L.p : nullptr, host_dw ? d_dw.p : nullptr, g,
                           cal, search, pT, sT, e, s);
        if (cal) launch_nvfp4_feedback(FT, m, n, c0, cb, e, d_L, s);
      }
    }
    launch_transpose_u8(pT, n / 2, m, pk, s);
    launch_transpose_u8(sT, n / 16, m, sc, s);
    QTIP_HIP(hipMemcpyAsync(M.packed, pk, pk.bytes(), hipMemcpyDeviceToHost, s));
    QTIP_HIP(hipMemcpyAsync(M.scales, sc, sc.bytes(), hipMemcpyDeviceToHost, s));
    QTIP_HIP(hipStreamSynchronize(s));
  }
}

}  // namespace qtipmi
