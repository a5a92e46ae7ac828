// NVFP4 fallback quantizer, host side: the format's scalar helpers, the plain nearest-value quantizer and the
// dequantizer (reference src/nvfp4.hpp:15-57, src/nvfp4.cpp:12-70), the Hessian preparation of the calibrated
// quantizer (src/nvfp4_gpu.hip:181-207) and the driver of its device block loop (src/nvfp4_gpu.hip:209-241).
#include <cmath>
#include <cstring>

#include "quantizer_impl.hpp"

namespace qtipmi {
namespace {

unsigned round_even(float v) {
  const float f = std::floor(v), r = v - f;
  const unsigned n = unsigned(f);
  return n + unsigned(r > .5f || (r == .5f && (n & 1u)));
}
float fp8e4m3_to_f32(uint8_t b) {  // src/common.hpp:81-88
  const uint32_t s = b >> 7, e = (b >> 3) & 0xf, m = b & 7;
  float v;
  if (e == 0) v = std::ldexp(float(m), -9);
  else if (e == 15 && m == 7) v = NAN;
  else v = std::ldexp(float(m | 8), int(e) - 10);
  return s ? -v : v;
}
const float kLevels[8] = {0, .5f, 1, 1.5f, 2, 3, 4, 6};
uint8_t fp4_code(float x) {  // nearest E2M1 value, ties to the even code (src/nvfp4.cpp:27-38)
  const float a = std::fabs(x);
  float best = INFINITY;
  int code = 0;
  for (int i = 0; i < 8; ++i) {
    const float e = std::fabs(a - kLevels[i]);
    if (e < best || (e == best && (i % 2 == 0))) {
      best = e;
      code = i;
    }
  }
  return uint8_t(code | (std::signbit(x) ? 8 : 0));
}
float global_scale(const float* w, size_t numel) {
  float maximum = 0;
  for (size_t i = 0; i < numel; ++i) {
    QTIP_REQUIRE(std::isfinite(w[i]), "nonfinite NVFP4 input");
    maximum = std::max(maximum, std::fabs(w[i]));
  }
  const float g = maximum ? maximum / (448.f * 6) : 1.f;
  QTIP_REQUIRE(g > 0 && std::isfinite(g), "NVFP4 global scale underflow/overflow");
  return g;
}

}  // namespace

uint8_t f32_to_fp8e4m3(float x) {  // src/nvfp4.hpp:15-33
  const uint8_t sign = std::signbit(x) ? 128 : 0;
  if (std::isnan(x)) return uint8_t(sign | 127);
  x = std::min(std::fabs(x), 448.f);
  if (x < std::ldexp(1.f, -6)) return uint8_t(sign | round_even(x * 512.f));
  int exp;
  const float frac = std::frexp(x, &exp) * 2;
  unsigned mant = round_even((frac - 1) * 8);
  int ee = exp + 6;
  if (mant == 8) {
    mant = 0;
    ++ee;
  }
  return uint8_t(sign | std::min(126u, (unsigned(ee) << 3) | mant));
}

void nvfp4_quantize_host(const float* w, int m, int n, uint8_t* packed, uint8_t* scales, float* global) {
  QTIP_REQUIRE(w && packed && scales && global && m > 0 && n > 0 && n % 16 == 0, "NVFP4 needs n %% 16 == 0 (m=%d n=%d)", m, n);
  const size_t numel = size_t(m) * n;
  const float g = global_scale(w, numel);
  *global = g;
#pragma omp parallel for schedule(static) if (numel >= (1u << 20))
  for (size_t b = 0; b < numel / 16; ++b) {
    float mx = 0;
    for (int j = 0; j < 16; ++j) mx = std::max(mx, std::fabs(w[b * 16 + j]));
    const uint8_t sc = f32_to_fp8e4m3(mx / (6 * g));
    scales[b] = sc;
    const float scale = fp8e4m3_to_f32(sc) * g;
    for (int j = 0; j < 16; j += 2)
      packed[b * 8 + j / 2] = uint8_t(fp4_code(scale ? w[b * 16 + j] / scale : 0) | (fp4_code(scale ? w[b * 16 + j + 1] / scale : 0) << 4));
  }
}

void nvfp4_dequantize_host(const uint8_t* packed, const uint8_t* scales, float global, int m, int n, float* out) {
  QTIP_REQUIRE(packed && scales && out && m > 0 && n > 0 && n % 16 == 0 && global > 0 && std::isfinite(global),
               "invalid NVFP4 payload");
  const size_t numel = size_t(m) * n;
  bool bad = false;
#pragma omp parallel for schedule(static) reduction(|| : bad) if (numel >= (1u << 20))
  for (size_t i = 0; i < numel; ++i) {
    const uint8_t code = (packed[i / 2] >> (i % 2 * 4)) & 15;
    const float s = fp8e4m3_to_f32(scales[i / 16]);
    bad = bad || !(s >= 0 && std::isfinite(s));
    out[i] = bf16_to_f32(f32_to_bf16((code & 8 ? -1.f : 1.f) * kLevels[code & 7] * s * global));
  }
  QTIP_REQUIRE(!bad, "invalid NVFP4 block scale");
}

double nvfp4_proxy_error_host(const float* w, const float* what, int m, int n, const float* H) {
  QTIP_REQUIRE(w && what && m > 0 && n > 0, "nvfp4_proxy_error: bad arguments");
  double total = 0;
#pragma omp parallel for reduction(+ : total) schedule(static)
  for (int r = 0; r < m; ++r) {
    std::vector<double> e(static_cast<size_t>(n), 0.0);
    for (int j = 0; j < n; ++j) e[size_t(j)] = double(w[size_t(r) * n + j]) - what[size_t(r) * n + j];
    double row = 0;
    if (!H) {
      for (int j = 0; j < n; ++j) row += e[size_t(j)] * e[size_t(j)];
    } else {
      for (int i = 0; i < n; ++i) {
        double acc = 0;
        for (int j = 0; j < n; ++j) acc += double(H[size_t(i) * n + j]) * e[size_t(j)];
        row += e[size_t(i)] * acc;
      }
    }
    total += row;
  }
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
