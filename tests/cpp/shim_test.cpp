// Exercises the C++ shim the way the reference's own GPU test drives quantize_group
// (tests/test_gpu.cpp:301-372): two linears sharing one Hessian, then a CPU decode of the packed output.
// Prints one line per linear; exit code 0 on success.  Built by the Makefile as qtip_shim_test.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "quantizer.hpp"

using namespace qtip;

int main() {
  if (hipSetDevice(0) != hipSuccess) {
    std::fprintf(stderr, "no GPU\n");
    return 2;
  }
  hipStream_t S;
  if (hipStreamCreate(&S) != hipSuccess) return 2;
  Gemm g(S);
  const int n = 256;
  std::mt19937_64 rng(33);
  std::normal_distribution<double> N01(0.0, 1.0);
  std::vector<float> W1(size_t(64) * n), W2(size_t(32) * n), H(size_t(n) * n);
  for (auto& v : W1) v = float(N01(rng) * 0.02);
  for (auto& v : W2) v = float(N01(rng) * 0.05);
  std::vector<double> G(size_t(n) * 3 * n);
  for (auto& x : G) x = N01(rng);
  for (int i = 0; i < n; ++i)
    for (int j = 0; j <= i; ++j) {
      double s = 0;
      for (int p = 0; p < 3 * n; ++p) s += G[size_t(i) * 3 * n + p] * G[size_t(j) * 3 * n + p];
      H[size_t(i) * n + j] = H[size_t(j) * n + i] = float(s / (3 * n));
    }
  std::vector<LinearIn> lins(2);
  lins[0].name = "a", lins[0].m = 64, lins[0].w_f32 = W1.data();
  lins[1].name = "b", lins[1].m = 32, lins[1].w_f32 = W2.data();
  QuantOpts o;
  o.ldl_threads = 4;
  o.want_hatW = true;
  GroupTiming tm;
  auto out = quantize_group(S, g, lins, n, H.data(), 7, o, &tm, "shim_test");
  int fail = 0;
  for (size_t li = 0; li < out.size(); ++li) {
    const LinearOut& lo = out[li];
    const std::vector<float>& W = li == 0 ? W1 : W2;
    // proxy of the returned reconstruction with the unregularised H, in fp64 on the host
    double num = 0, den = 0;
    for (int i = 0; i < lo.m; ++i) {
      std::vector<double> d(n), w(n);
      for (int j = 0; j < n; ++j) d[j] = double(W[size_t(i) * n + j]) - lo.hatW[size_t(i) * n + j], w[j] = W[size_t(i) * n + j];
      for (int a = 0; a < n; ++a)
        for (int b = 0; b < n; ++b) num += d[a] * H[size_t(a) * n + b] * d[b], den += w[a] * H[size_t(a) * n + b] * w[b];
    }
    const double p = num / den;
    std::printf("%s: proxy %.6f host-recomputed %.6f proxy_rot_reg %.6f wscale %.6f words %zu\n", lo.name.c_str(),
                lo.proxy, p, lo.proxy_rot_reg, lo.wscale, lo.trellis.size());
    if (!(lo.proxy > 0 && lo.proxy < 0.2)) ++fail;
    if (std::fabs(p - lo.proxy) / lo.proxy > 1e-3) ++fail;
    if (lo.trellis.size() != size_t(lo.m / 16) * (n / 16) * 32) ++fail;
  }
  // the scheduler over three groups returns what quantize_group returns for each, dequantize_linear reproduces the
  // reconstruction, and the layer file holds the tensors of both linears
  {
    std::vector<GroupSpec> gs(3);
    for (int k = 0; k < 3; ++k) gs[size_t(k)] = GroupSpec{lins, n, H.data(), uint64_t(7 + k), "g" + std::to_string(k)};
    std::vector<GroupTiming> tms;
    std::vector<double> waits;
    auto res = run_groups(gs, o, &tms, &waits);
    if (res.size() != 3 || tms.size() != 3 || waits.size() != 3) ++fail;
    for (size_t li = 0; li < out.size() && res.size() == 3; ++li) {
      if (res[0][li].trellis != out[li].trellis || res[0][li].wscale != out[li].wscale) ++fail;
      if (res[1][li].trellis == out[li].trellis) ++fail;  // another seed, another sign vector
      if (dequantize_linear(res[0][li]) != out[li].hatW) ++fail;
    }
    std::printf("run_groups: 3 groups, ldl %.3fs ldlq %.3fs, mismatches so far %d\n", tms.empty() ? 0.0 : tms[0].ldl_cpu,
                tms.empty() ? 0.0 : tms[0].ldlq, fail);
    SafeTensorsWriter w;
    w.add_qtip_linear("model.layers.0.a.", out[0]);
    w.add_qtip_linear("model.layers.0.b.", out[1]);
    const char* path = "/tmp/qtip_shim_test_layer.safetensors";
    const size_t bytes = w.write(path);
    FILE* f = std::fopen(path, "rb");
    long sz = -1;
    if (f) {
      std::fseek(f, 0, SEEK_END);
      sz = std::ftell(f);
      std::fclose(f);
      std::remove(path);
    }
    std::printf("layer file: %zu bytes\n", bytes);
    if (sz != long(bytes) || bytes < out[0].trellis.size() * 2 + out[1].trellis.size() * 2) ++fail;
  }
  // ldlq_gpu on operands still in the making on the caller's stream (the reference's quantize_group forms WT there and
  // calls ldlq_gpu without a synchronization in between, src/quantizer.cpp:239-265): a long run of fills is queued
  // on S ahead of the copies that bring WT and L to the device, so a library that did not wait for S would read
  // zeros; the states must equal those of the same call on settled operands.  device_lut() is the decoded table.
  {
    const long m = 64, nn = n;
    std::vector<float> hWT(size_t(nn) * m), hL(size_t(nn) * nn, 0.f);
    for (auto& v : hWT) v = float(N01(rng));
    for (int i = 0; i < nn; ++i)
      for (int j = 0; j < (i / 16) * 16; ++j) hL[size_t(i) * nn + j] = float(0.05 * N01(rng));
    float *pWT = nullptr, *pL = nullptr, *dWT = nullptr, *dL = nullptr, *dHat = nullptr, *big = nullptr;
    uint16_t *dQ1 = nullptr, *dQ2 = nullptr;
    const size_t bigBytes = size_t(1) << 31, qn = size_t(m / 16) * (nn / 16) * 128;
    bool ok = hipHostMalloc(reinterpret_cast<void**>(&pWT), hWT.size() * 4, hipHostMallocDefault) == hipSuccess &&
              hipHostMalloc(reinterpret_cast<void**>(&pL), hL.size() * 4, hipHostMallocDefault) == hipSuccess &&
              hipMalloc(reinterpret_cast<void**>(&dWT), hWT.size() * 4) == hipSuccess &&
              hipMalloc(reinterpret_cast<void**>(&dL), hL.size() * 4) == hipSuccess &&
              hipMalloc(reinterpret_cast<void**>(&dHat), hWT.size() * 4) == hipSuccess &&
              hipMalloc(reinterpret_cast<void**>(&dQ1), qn * 2) == hipSuccess &&
              hipMalloc(reinterpret_cast<void**>(&dQ2), qn * 2) == hipSuccess &&
              hipMalloc(reinterpret_cast<void**>(&big), bigBytes) == hipSuccess;
    if (ok) {
      std::memcpy(pWT, hWT.data(), hWT.size() * 4);
      std::memcpy(pL, hL.data(), hL.size() * 4);
      ok = hipMemset(dWT, 0, hWT.size() * 4) == hipSuccess && hipMemset(dL, 0, hL.size() * 4) == hipSuccess &&
           hipDeviceSynchronize() == hipSuccess;
      for (int rep = 0; ok && rep < 16; ++rep) ok = hipMemsetAsync(big, rep, bigBytes, S) == hipSuccess;  // ~10 ms of fills
      ok = ok && hipMemcpyAsync(dWT, pWT, hWT.size() * 4, hipMemcpyHostToDevice, S) == hipSuccess &&
           hipMemcpyAsync(dL, pL, hL.size() * 4, hipMemcpyHostToDevice, S) == hipSuccess;
      if (ok) ldlq_gpu(S, g, dWT, dL, nn, m, dHat, dQ1, 1024, device_lut(), nullptr);
      ok = ok && hipStreamSynchronize(S) == hipSuccess;
      if (ok) ldlq_gpu(S, g, dWT, dL, nn, m, dHat, dQ2, 1024, device_lut(), nullptr);
      std::vector<uint16_t> q1(qn), q2(qn);
      ok = ok && hipMemcpy(q1.data(), dQ1, qn * 2, hipMemcpyDeviceToHost) == hipSuccess &&
           hipMemcpy(q2.data(), dQ2, qn * 2, hipMemcpyDeviceToHost) == hipSuccess;
      size_t same = 0, zero = 0;
      for (size_t i = 0; i < qn; ++i) same += q1[i] == q2[i], zero += q2[i] == 0;
      std::printf("ldlq_gpu on operands still being copied on the caller's stream: %zu of %zu state words equal\n", same, qn);
      if (same != qn || zero > qn / 2) ++fail;
      // device_lut(): fp16 pair per state; against the host's decoded table at a few states
      std::vector<uint32_t> h2(65536);
      std::vector<float> l0(65536), l1(65536);
      const uint32_t* dl = device_lut();
      ok = ok && dl != nullptr && hipMemcpy(h2.data(), dl, h2.size() * 4, hipMemcpyDeviceToHost) == hipSuccess &&
           qtip_get_lut(detail::context(), l0.data(), l1.data()) == QTIP_OK;
      auto half = [](uint16_t h) {
        const int e = (h >> 10) & 31, mnt = h & 1023;
        const float v = e == 0 ? std::ldexp(float(mnt), -24) : std::ldexp(float(mnt | 1024), e - 25);
        return (h >> 15) ? -v : v;
      };
      for (uint32_t st = 0; ok && st < 65536; st += 97)
        if (half(uint16_t(h2[st])) != l0[st] || half(uint16_t(h2[st] >> 16)) != l1[st]) ok = false;
    }
    if (!ok) ++fail;
    std::printf("caller-stream ordering and device_lut: mismatches so far %d\n", fail);
    (void)hipFree(big), (void)hipFree(dQ2), (void)hipFree(dQ1), (void)hipFree(dHat), (void)hipFree(dL), (void)hipFree(dWT);
    (void)hipHostFree(pL), (void)hipHostFree(pWT);
  }
  // dump_dir (src/quantizer.cpp:230-234, 321-337): W as fp32 and the reconstruction, one raw file each
  {
    QuantOpts od;
    od.ldl_threads = 4;
    od.dump_dir = "/tmp";
    std::vector<uint16_t> wb(size_t(32) * n);  // a bf16 source: the dump holds its widened values
    for (size_t i = 0; i < wb.size(); ++i) {
      uint32_t u;
      std::memcpy(&u, &W2[i], 4);
      wb[i] = uint16_t(u >> 16);
    }
    std::vector<LinearIn> lb(1);
    lb[0].name = "dump", lb[0].m = 32, lb[0].w_bf16 = wb.data();
    GroupTiming t2;
    auto od_out = quantize_group(S, g, lb, n, H.data(), 11, od, &t2, "shimtest");
    od.dump_dir.clear();
    od.want_hatW = true;
    auto od_ref = quantize_group(S, g, lb, n, H.data(), 11, od, &t2, "shimtest");
    auto slurp = [](const char* path) {
      std::vector<float> v;
      if (FILE* f = std::fopen(path, "rb")) {
        std::fseek(f, 0, SEEK_END);
        v.resize(size_t(std::ftell(f)) / 4);
        std::fseek(f, 0, SEEK_SET);
        if (std::fread(v.data(), 4, v.size(), f) != v.size()) v.clear();
        std::fclose(f);
        std::remove(path);
      }
      return v;
    };
    const std::vector<float> dw = slurp("/tmp/shimtest_dump.W.f32"), dh = slurp("/tmp/shimtest_dump.hatW.f32");
    bool okw = dw.size() == wb.size();
    for (size_t i = 0; okw && i < dw.size(); ++i) {
      const uint32_t u = uint32_t(wb[i]) << 16;
      float f;
      std::memcpy(&f, &u, 4);
      okw = dw[i] == f;
    }
    if (!okw || dh != od_ref[0].hatW || !od_out[0].hatW.empty() || od_out[0].trellis != od_ref[0].trellis) ++fail;
    std::printf("dump_dir: W %zu values, hatW %zu values, mismatches so far %d\n", dw.size(), dh.size(), fail);
  }
  // NVFP4 fallback (the criteria of tests/test_nvfp4.cpp:59-105): upgrades off == the plain quantizer byte for byte,
  // calibrated rounding lowers the Hessian-weighted error, a group equals single calls
  {
    auto proxy = [&](const std::vector<float>& W, const Nvfp4Tensor& t) {
      std::vector<float> q = nvfp4_dequantize(t);
      double tot = 0;
      for (int i = 0; i < t.m; ++i) {
        std::vector<double> e(static_cast<size_t>(n), 0.0);
        for (int j = 0; j < n; ++j) e[size_t(j)] = double(W[size_t(i) * n + j]) - q[size_t(i) * n + j];
        for (int a = 0; a < n; ++a) {
          double acc = 0;
          for (int b = 0; b < n; ++b) acc += double(H[size_t(a) * n + b]) * e[size_t(b)];
          tot += e[size_t(a)] * acc;
        }
      }
      return tot / t.m;
    };
    Nvfp4Tensor plain = nvfp4_quantize(W1.data(), 64, n);
    Nvfp4Opts off;
    off.scale_search = off.calibrate = false;
    bool used = true;
    auto a = nvfp4_quantize_group(S, {W1.data()}, {64}, n, nullptr, off, &used);
    if (used || a[0].packed != plain.packed || a[0].scales != plain.scales || a[0].global != plain.global) ++fail;
    auto b = nvfp4_quantize_group(S, {W1.data(), W2.data()}, {64, 32}, n, H.data(), Nvfp4Opts{}, &used);
    auto c = nvfp4_quantize_group(S, {W2.data()}, {32}, n, H.data(), Nvfp4Opts{});
    if (!used || b[1].packed != c[0].packed || b[1].scales != c[0].scales) ++fail;
    const double p0 = proxy(W1, plain), p1 = proxy(W1, b[0]);
    std::printf("nvfp4: proxy plain %.6g calibrated %.6g (%.1f%%), %lld bytes\n", p0, p1, 100 * p1 / p0,
                static_cast<long long>(b[0].size_bytes()));
    if (!(p1 < 0.9 * p0)) ++fail;
    if (f32_to_fp8e4m3(448.f) != 126 || f32_to_fp8e4m3(-1.f) != (128 | 56) || nvfp4_level(0xf) != -6.f) ++fail;
    SafeTensorsWriter w;
    w.add_nvfp4_linear("model.layers.0.a.", b[0]);
    const char* path = "/tmp/qtip_shim_test_nv.safetensors";
    if (w.write(path) < b[0].packed.size() + b[0].scales.size() + 4) ++fail;
    std::remove(path);
  }
  std::printf(fail ? "SHIM TEST FAILED\n" : "SHIM TEST PASSED\n");
  return fail ? 1 : 0;
}
