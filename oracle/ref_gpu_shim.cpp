// Test infrastructure only: extern "C" doorway into the reference's own device path and into the CPU LDLQ of its
// GPU test, compiled for gfx950 from the sources where they lie under /root/reference by oracle/Makefile into
// oracle/_ref/libqtip_ref_gpu.so.  Nothing on the product path may load this library.
//
//   ref_ldlq                      ldlq_ref, tests/test_gpu.cpp:180-225 (CPU only; a static function of the test
//                                 program, reached by compiling that file into this unit with its main renamed)
//   ref_gpu_quantize_group        quantize_group, src/quantizer.cpp:340-348 (src/quantizer.hpp:72-74)
//   ref_gpu_quantize_seqs         the two-pass tail-biting Viterbi as the test drives it, tests/test_gpu.cpp:67-88
//   ref_gpu_nvfp4_quantize_group  nvfp4_quantize_group, src/nvfp4_gpu.hip:174-243
//   ref_gpu_hadamard_rows         k_hadamard_rows, src/kernels.hip:293-313 (src/gpu.hpp:232)
#define main ref_test_gpu_main
#include "test_gpu.cpp"
#undef main

#include "nvfp4_gpu.hpp"

namespace {
void ensure_stream() {
  if (!S) HIP_CHECK(hipStreamCreate(&S));
}
}  // namespace

extern "C" {

void ref_ldlq(const float* Wr, const float* L, int m, int n, float* hatWr, uint16_t* Q) {
  std::vector<float> w(Wr, Wr + size_t(m) * n), l(L, L + size_t(n) * n), h;
  std::vector<uint16_t> q;
  ldlq_ref(w, l, m, n, h, q);
  std::memcpy(hatWr, h.data(), h.size() * 4);
  std::memcpy(Q, q.data(), q.size() * 2);
}

// X: rows x ld fp32 on the host, transformed in place on the device (rows of length n)
void ref_gpu_hadamard_rows(float* X, long rows, int n, long ld, int transpose) {
  ensure_stream();
  float* d = nullptr;
  const size_t bytes = size_t(rows) * size_t(ld) * sizeof(float);
  HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&d), bytes));
  HIP_CHECK(hipMemcpy(d, X, bytes, hipMemcpyHostToDevice));
  k_hadamard_rows(d, rows, n, ld, transpose != 0, S);
  HIP_CHECK(hipStreamSynchronize(S));
  HIP_CHECK(hipMemcpy(X, d, bytes, hipMemcpyDeviceToHost));
  HIP_CHECK(hipFree(d));
}

// B sequences of 256 fp32 -> states [B][128]; returns the seconds the reference's own timer measured
double ref_gpu_quantize_seqs(const float* X, int B, uint16_t* states) {
  ensure_stream();
  std::vector<float> x(X, X + size_t(B) * 256), hat;
  std::vector<uint16_t> st;
  double secs = 0;
  gpu_quantize_seqs(x, B, st, hat, &secs);
  std::memcpy(states, st.data(), st.size() * 2);
  return secs;
}

// ws[i]: row-major [ms[i]][n] fp32, H n x n fp32.  Outputs per linear (caller-allocated): trellis
// [(m/16)*(n/16)*32] u16, su_bf16 [n], sv [m], hatW [m][n] or null; wscale, proxy, proxy_rot_reg [nlin];
// timing [8] = load, rht, ldl_cpu, ldlq, viterbi, proxy, pack, total.
void ref_gpu_quantize_group(int nlin, const float* const* ws, const int* ms, int n, const float* H, uint64_t seed,
                            double sigma_reg, double scale_override, int ldl_threads, uint16_t* const* trellis,
                            uint16_t* const* su_bf16, float* const* sv, float* const* hatW, float* wscale, double* proxy,
                            double* proxy_rot_reg, double* timing) {
  ensure_stream();
  Gemm g(S);
  std::vector<LinearIn> lins(static_cast<size_t>(nlin));
  for (int i = 0; i < nlin; ++i) lins[size_t(i)].name = "l" + std::to_string(i), lins[size_t(i)].m = ms[i], lins[size_t(i)].w_f32 = ws[i];
  QuantOpts o;
  o.sigma_reg = sigma_reg, o.scale_override = scale_override, o.ldl_threads = ldl_threads;
  o.want_hatW = hatW != nullptr;
  GroupTiming tm;
  std::vector<LinearOut> out = quantize_group(S, g, lins, n, H, seed, o, &tm, "ref");
  for (int i = 0; i < nlin; ++i) {
    const LinearOut& r = out[size_t(i)];
    std::memcpy(trellis[i], r.trellis.data(), r.trellis.size() * 2);
    std::memcpy(su_bf16[i], r.su_bf16.data(), r.su_bf16.size() * 2);
    std::memcpy(sv[i], r.sv.data(), r.sv.size() * 4);
    if (hatW && hatW[i]) std::memcpy(hatW[i], r.hatW.data(), r.hatW.size() * 4);
    wscale[i] = r.wscale, proxy[i] = r.proxy, proxy_rot_reg[i] = r.proxy_rot_reg;
  }
  if (timing) {
    const double t[8] = {tm.load, tm.rht, tm.ldl_cpu, tm.ldlq, tm.viterbi, tm.proxy, tm.pack, tm.total};
    std::memcpy(timing, t, sizeof(t));
  }
}

// ws[i]: row-major [ms[i]][n] fp32; packed[i] / scales[i]: caller-allocated [ms[i]][n/2] and [ms[i]][n/16];
// globals[i]: the matrix's fp32 global scale.  H may be null.  Returns whether the Hessian was used for calibration.
int ref_gpu_nvfp4_quantize_group(int nmat, const float* const* ws, const int* ms, int n, const float* H, int scale_search,
                                 int calibrate, double sigma_reg, uint8_t* const* packed, uint8_t* const* scales,
                                 float* globals) {
  ensure_stream();
  Nvfp4Opts o;
  o.scale_search = scale_search != 0, o.calibrate = calibrate != 0, o.sigma_reg = sigma_reg;
  bool used = false;
  std::vector<Nvfp4Tensor> out =
      nvfp4_quantize_group(S, std::vector<const float*>(ws, ws + nmat), std::vector<int>(ms, ms + nmat), n, H, o, &used);
  for (int i = 0; i < nmat; ++i) {
    std::memcpy(packed[i], out[size_t(i)].packed.data(), out[size_t(i)].packed.size());
    std::memcpy(scales[i], out[size_t(i)].scales.data(), out[size_t(i)].scales.size());
    globals[i] = out[size_t(i)].global;
  }
  return used ? 1 : 0;
}
}
