// C++ shim with the reference's own interface for the group quantizer (src/quantizer.hpp:11-78 of the
// reference: same names, argument meaning and abort-on-error behaviour), implemented on the C ABI of
// libqtip_mi355.so.  A caller such as run_qtip_groups (src/pipeline.cpp:229-312) compiles against this header
// instead of the reference's quantizer.hpp and links libqtip_mi355.so instead of quantizer.cpp + its kernels.
#pragma once
#include <hip/hip_runtime.h>

#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/qtip_mi355.h"

namespace qtip {

// The reference passes its hipBLASLt wrapper through these calls; the MFMA contractions live inside the
// library here, so the type only keeps the signatures source-compatible.
class Gemm {
 public:
  Gemm() = default;
  explicit Gemm(hipStream_t) {}
};

struct QuantOpts {  // src/quantizer.hpp:11-19
  double sigma_reg = 1e-2;
  double scale_override = 0.9;
  int vit_batch = 1024;  // accepted, unused: the tile kernel sizes its own workspace
  int ldl_threads = 16;
  bool share_su = true;
  std::string dump_dir;  // if set: W (fp32) and, unless want_hatW, the reconstructed hatW (fp32) are written per linear
  bool want_hatW = false;
  // not in the reference: the group calls hand the trailing updates of the host LDL to the GPU (the factor is the
  // host's bit for bit); false keeps the factorization on the host alone
  bool ldl_device_updates = true;
  // not in the reference: run_groups runs groups that cannot fill the chip side by side (0: as many as fit, 1: one at
  // a time, as the reference schedules them); the outputs do not depend on it
  int group_lanes = 0;
};

struct LinearIn {  // src/quantizer.hpp:21-28
  std::string name;
  int m = 0;
  const uint8_t* w_fp8 = nullptr;
  const uint16_t* scale_bf16 = nullptr;
  const uint16_t* w_bf16 = nullptr;
  const float* w_f32 = nullptr;
};

struct LinearOut {  // src/quantizer.hpp:30-43
  std::string name;
  int m = 0, n = 0;
  std::vector<uint16_t> trellis;
  std::vector<uint16_t> su_bf16;
  std::vector<float> sv;
  float wscale = 0;
  double proxy = 0;
  double proxy_rot_reg = 0;
  double seconds = 0;
  std::vector<float> hatW;
};

struct GroupTiming {  // src/quantizer.hpp:45-47
  double load = 0, rht = 0, ldl_cpu = 0, ldlq = 0, viterbi = 0, proxy = 0, pack = 0, total = 0;
};

struct HessPrep {  // src/quantizer.hpp:51-59
  int n = 0;
  uint64_t seed = 0;
  std::vector<float> su;
  double creg = 0;
  std::vector<float> HRr;
  std::vector<float> L;
  double t_rot = 0, t_ldl = 0;
};

namespace detail {
[[noreturn]] inline void die(const std::string& msg) {  // src/common.hpp:24-28
  std::fprintf(stderr, "fatal: %s\n", msg.c_str());
  std::fflush(stderr);
  std::abort();
}
inline void check(int rc, const char* what) {
  if (rc != QTIP_OK) die(std::string(what) + ": " + qtip_last_error());
}
inline double now_s() {
  using namespace std::chrono;
  return duration<double>(steady_clock::now().time_since_epoch()).count();
}
// one context per device, created on first use by the worker thread that has made the device current
inline qtip_ctx* context() {
  static std::mutex mu;
  static std::map<int, qtip_ctx*> cache;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) die("hipGetDevice failed");
  std::lock_guard<std::mutex> lk(mu);
  auto it = cache.find(dev);
  if (it != cache.end()) return it->second;
  qtip_ctx* c = nullptr;
  check(qtip_create(dev, &c), "qtip_create");
  cache[dev] = c;
  return c;
}
}  // namespace detail

namespace detail {
// src/quantizer.cpp:118-121
inline void write_f32(const std::string& path, const float* p, size_t count) {
  FILE* f = std::fopen(path.c_str(), "wb");
  if (!f) return;  // the reference's ofstream write fails as silently
  std::fwrite(p, 4, count, f);
  std::fclose(f);
}
// The fp32 weight quantize_group works on, as the reference dumps it (src/quantizer.cpp:214-234): the input itself,
// the bf16 bits widened, or the E4M3 value times its row's bf16 scale (one fp32 product, src/kernels.hip:20-36).
inline std::vector<float> weight_as_f32(const LinearIn& l, int n) {
  const size_t count = size_t(l.m) * size_t(n);
  std::vector<float> w(count);
  auto bf = [](uint16_t h) {
    const uint32_t u = uint32_t(h) << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
  };
  if (l.w_f32) {
    std::memcpy(w.data(), l.w_f32, count * 4);
  } else if (l.w_bf16) {
    for (size_t i = 0; i < count; ++i) w[i] = bf(l.w_bf16[i]);
  } else if (l.w_fp8) {
    for (size_t i = 0; i < count; ++i) {
      const uint8_t b = l.w_fp8[i];
      const uint32_t e = (b >> 3) & 0xf, m = b & 7;
      float v = e == 0 ? std::ldexp(float(m), -9) : (e == 15 && m == 7) ? std::nanf("") : std::ldexp(float(m | 8), int(e) - 10);
      if (b >> 7) v = -v;
      w[i] = l.scale_bf16 ? v * bf(l.scale_bf16[i / size_t(n)]) : v;
    }
  }
  return w;
}
inline void dump_linear(const QuantOpts& opt, const std::string& tag, const LinearIn& l, int n, const float* hatW) {
  if (opt.dump_dir.empty()) return;
  const std::vector<float> w = weight_as_f32(l, n);
  write_f32(opt.dump_dir + "/" + tag + "_" + l.name + ".W.f32", w.data(), w.size());
  if (!opt.want_hatW && hatW) write_f32(opt.dump_dir + "/" + tag + "_" + l.name + ".hatW.f32", hatW, w.size());
}
}  // namespace detail

// The reference queues its work on the caller's stream s.  Here the context's stream first waits for what s holds so
// far (device memory or host buffers that s is still filling are complete before they are read); every call below is
// complete on the host when it returns, as the reference's is.
inline void rotate_hessian(hipStream_t s, const float* H, int n, uint64_t seed, const QuantOpts& opt, HessPrep& hp) {
  const double t0 = detail::now_s();
  detail::check(qtip_stream_wait(detail::context(), s), "rotate_hessian");
  hp.n = n;
  hp.seed = seed;
  hp.su.resize(size_t(n));
  hp.HRr.resize(size_t(n) * n);
  detail::check(qtip_rotate_hessian(detail::context(), H, 0, n, seed, opt.sigma_reg, hp.su.data(), &hp.creg,
                                    hp.HRr.data()),
                "rotate_hessian");
  hp.t_rot = detail::now_s() - t0;
}

inline void ldl_hessian(HessPrep& hp, int threads, const std::string& tag) {
  const double t0 = detail::now_s();
  hp.L.resize(size_t(hp.n) * hp.n);
  const int rc = qtip_ldl_hessian(hp.HRr.data(), hp.n, threads, hp.L.data());
  if (rc != QTIP_OK) detail::die("block LDL failed (H not PD) for " + tag + ": " + qtip_last_error());
  hp.t_ldl = detail::now_s() - t0;
}

inline std::vector<LinearOut> quantize_group(hipStream_t s, Gemm&, const std::vector<LinearIn>& lins, HessPrep& hp,
                                             const QuantOpts& opt, GroupTiming* tm, const std::string& tag) {
  if (!opt.share_su) detail::die("share_su=false not supported (one LDL per group)");
  detail::check(qtip_stream_wait(detail::context(), s), "quantize_group");
  const bool need_hat = opt.want_hatW || !opt.dump_dir.empty();
  const int n = hp.n;
  std::vector<qtip_linear_in> cin(lins.size());
  std::vector<qtip_linear_out> cout(lins.size());
  std::vector<LinearOut> out(lins.size());
  for (size_t i = 0; i < lins.size(); ++i) {
    const LinearIn& l = lins[i];
    cin[i] = qtip_linear_in{l.m, l.w_f32, l.w_bf16, l.w_fp8, l.scale_bf16, 0};
    LinearOut& o = out[i];
    o.name = l.name, o.m = l.m, o.n = n;
    if (l.m <= 0 || l.m % 16 || n % 16) detail::die("bad linear shape for " + tag);
    o.trellis.resize(size_t(l.m / 16) * (n / 16) * 32);
    o.su_bf16.resize(size_t(n));
    o.sv.resize(size_t(l.m));
    if (need_hat) o.hatW.resize(size_t(l.m) * n);
    cout[i] = qtip_linear_out{o.trellis.data(), o.su_bf16.data(), o.sv.data(), need_hat ? o.hatW.data() : nullptr,
                              0.f, 0.0, 0.0, 0.0};
  }
  qtip_opts co;
  qtip_default_opts(&co);
  co.sigma_reg = opt.sigma_reg, co.scale_override = opt.scale_override, co.ldl_threads = opt.ldl_threads;
  co.ldl_device_updates = opt.ldl_device_updates ? 1 : 0;
  qtip_timing ct{};
  ct.rht = hp.t_rot, ct.ldl_cpu = hp.t_ldl;
  detail::check(qtip_quantize_group(detail::context(), int(lins.size()), cin.data(), n, hp.seed, hp.su.data(), hp.creg,
                                    hp.HRr.data(), hp.L.data(), &co, cout.data(), &ct),
                ("quantize_group " + tag).c_str());
  hp.L.clear();  // consumed, as in the reference (src/quantizer.cpp:256-257)
  hp.L.shrink_to_fit();
  for (size_t i = 0; i < lins.size(); ++i) {
    out[i].wscale = cout[i].wscale, out[i].proxy = cout[i].proxy;
    out[i].proxy_rot_reg = cout[i].proxy_rot_reg, out[i].seconds = cout[i].seconds;
    detail::dump_linear(opt, tag, lins[i], n, out[i].hatW.data());
    if (!opt.want_hatW) std::vector<float>().swap(out[i].hatW);
  }
  if (tm) *tm = GroupTiming{ct.load, ct.rht, ct.ldl_cpu, ct.ldlq, ct.viterbi, ct.proxy, ct.pack, ct.total};
  return out;
}

inline std::vector<LinearOut> quantize_group(hipStream_t s, Gemm& gemm, const std::vector<LinearIn>& lins, int n,
                                             const float* H, uint64_t seed, const QuantOpts& opt, GroupTiming* tm,
                                             const std::string& tag) {
  HessPrep hp;
  rotate_hessian(s, H, n, seed, opt, hp);
  ldl_hessian(hp, opt.ldl_threads, tag);
  return quantize_group(s, gemm, lins, hp, opt, tm, tag);
}

// WT n x m, L n x n, hatWT n x m, Q on the device (src/quantizer.hpp:70-73); vit_batch and the LUT pointer are
// accepted for source compatibility (the library holds its own codebook tables).
inline void ldlq_gpu(hipStream_t s, Gemm&, const float* WT, const float* L, long n, long m, float* hatWT, uint16_t* Q,
                     int /*vit_batch*/, const uint32_t* /*lut_h2_dev*/, double* vit_s) {
  // WT and L may still be in the making on s (the reference's quantize_group forms them there and calls this without
  // a synchronization in between, src/quantizer.cpp:239-265); the call returns with hatWT and Q complete
  detail::check(qtip_stream_wait(detail::context(), s), "ldlq_gpu");
  detail::check(qtip_ldlq_dev(detail::context(), WT, L, n, m, hatWT, Q, 0, vit_s), "ldlq_gpu");
}

// src/quantizer.cpp:14-28: the decoded table on the current device, one fp16 pair per state.  (The library's own
// kernels read tables of the 1024 distinct entries; this one exists for callers that hand it to kernels of theirs.)
inline const uint32_t* device_lut() {
  const uint32_t* p = nullptr;
  detail::check(qtip_device_lut(detail::context(), &p), "device_lut");
  return p;
}

// ---------------------------------------------------------------- callers either side of quantize_group
// One Hessian group of a layer as run_qtip_groups forms it (src/pipeline.cpp:240-246,266-280).
struct GroupSpec {
  std::vector<LinearIn> lins;
  int n = 0;
  const float* H = nullptr;  // host, n x n
  uint64_t seed = 0;
  std::string tag;
};

// The body of run_qtip_groups (src/pipeline.cpp:247-309): rotation ahead of use, host LDL of the groups on a side
// thread, quantize_group as factors arrive.  Returns the LinearOuts per group; tms / ldl_wait may be null.
inline std::vector<std::vector<LinearOut>> run_groups(const std::vector<GroupSpec>& groups, const QuantOpts& opt,
                                                      std::vector<GroupTiming>* tms = nullptr,
                                                      std::vector<double>* ldl_wait = nullptr) {
  if (!opt.share_su) detail::die("share_su=false not supported (one LDL per group)");
  const bool need_hat = opt.want_hatW || !opt.dump_dir.empty();
  const size_t ng = groups.size();
  std::vector<std::vector<qtip_linear_in>> cin(ng);
  std::vector<std::vector<qtip_linear_out>> cout(ng);
  std::vector<std::vector<LinearOut>> out(ng);
  std::vector<qtip_group> cg(ng);
  for (size_t g = 0; g < ng; ++g) {
    const GroupSpec& G = groups[g];
    cin[g].resize(G.lins.size()), cout[g].resize(G.lins.size()), out[g].resize(G.lins.size());
    for (size_t i = 0; i < G.lins.size(); ++i) {
      const LinearIn& l = G.lins[i];
      if (l.m <= 0 || l.m % 16 || G.n <= 0 || G.n % 16) detail::die("bad linear shape for " + G.tag);
      cin[g][i] = qtip_linear_in{l.m, l.w_f32, l.w_bf16, l.w_fp8, l.scale_bf16, 0};
      LinearOut& o = out[g][i];
      o.name = l.name, o.m = l.m, o.n = G.n;
      o.trellis.resize(size_t(l.m / 16) * (G.n / 16) * 32);
      o.su_bf16.resize(size_t(G.n));
      o.sv.resize(size_t(l.m));
      if (need_hat) o.hatW.resize(size_t(l.m) * G.n);
      cout[g][i] = qtip_linear_out{o.trellis.data(), o.su_bf16.data(), o.sv.data(),
                                   need_hat ? o.hatW.data() : nullptr, 0.f, 0.0, 0.0, 0.0};
    }
    cg[g] = qtip_group{int(G.lins.size()), cin[g].data(), cout[g].data(), G.n, G.H, 0, G.seed};
  }
  qtip_opts co;
  qtip_default_opts(&co);
  co.sigma_reg = opt.sigma_reg, co.scale_override = opt.scale_override, co.ldl_threads = opt.ldl_threads;
  co.ldl_device_updates = opt.ldl_device_updates ? 1 : 0;
  co.group_lanes = opt.group_lanes;
  std::vector<qtip_timing> ct(ng);
  std::vector<double> waits(ng, 0.0);
  detail::check(qtip_run_groups(detail::context(), int(ng), cg.data(), &co, ct.data(), waits.data()), "run_groups");
  for (size_t g = 0; g < ng; ++g)
    for (size_t i = 0; i < out[g].size(); ++i) {
      out[g][i].wscale = cout[g][i].wscale, out[g][i].proxy = cout[g][i].proxy;
      out[g][i].proxy_rot_reg = cout[g][i].proxy_rot_reg, out[g][i].seconds = cout[g][i].seconds;
      detail::dump_linear(opt, groups[g].tag, groups[g].lins[i], groups[g].n, out[g][i].hatW.data());
      if (!opt.want_hatW) std::vector<float>().swap(out[g][i].hatW);
    }
  if (tms) {
    tms->clear();
    for (auto& t : ct) tms->push_back(GroupTiming{t.load, t.rht, t.ldl_cpu, t.ldlq, t.viterbi, t.proxy, t.pack, t.total});
  }
  if (ldl_wait) *ldl_wait = waits;
  return out;
}

// hatW (m x n, original domain) of a quantized linear from its packed output (the reconstruction of
// src/quantizer.cpp:321-338 started from the trellis words; decode as runtime/src/qtip.cpp:83-118).
inline std::vector<float> dequantize_linear(const LinearOut& lo) {
  std::vector<float> h(size_t(lo.m) * lo.n);
  detail::check(qtip_dequantize_linear(detail::context(), lo.trellis.data(), lo.su_bf16.data(), lo.sv.data(), lo.wscale,
                                       lo.m, lo.n, h.data(), 0),
                "dequantize_linear");
  return h;
}

// ---- NVFP4 fallback format (src/nvfp4.hpp:35-60, src/nvfp4_gpu.hpp:17-30): same names, same bytes.
inline uint8_t f32_to_fp8e4m3(float x) { return qtip_f32_to_fp8e4m3(x); }

struct Nvfp4Tensor {
  int m = 0, n = 0;             // out x in, n a multiple of 16
  std::vector<uint8_t> packed;  // [m][n/2], low nibble = first of two values
  std::vector<uint8_t> scales;  // [m][n/16] E4M3 block scales
  float global = 1;             // F32 global scale
  int64_t size_bytes() const { return int64_t(packed.size()) + int64_t(scales.size()) + 4; }
};

struct Nvfp4Opts {
  bool scale_search = true;
  bool calibrate = true;
  double sigma_reg = 1e-2;
};

inline Nvfp4Tensor nvfp4_quantize(const float* w, int m, int n) {
  Nvfp4Tensor t;
  t.m = m, t.n = n;
  t.packed.resize(size_t(m) * size_t(n > 0 ? n / 2 : 0));
  t.scales.resize(size_t(m) * size_t(n > 0 ? n / 16 : 0));
  detail::check(qtip_nvfp4_quantize(w, m, n, t.packed.data(), t.scales.data(), &t.global), "nvfp4_quantize");
  return t;
}

inline std::vector<float> nvfp4_dequantize(const Nvfp4Tensor& t) {
  std::vector<float> out(size_t(t.m) * size_t(t.n));
  detail::check(qtip_nvfp4_dequantize(t.packed.data(), t.scales.data(), t.global, t.m, t.n, out.data()), "nvfp4_dequantize");
  return out;
}

inline double nvfp4_proxy_error(const float* w, const float* what, int m, int n, const float* H) {
  double v = 0;
  detail::check(qtip_nvfp4_proxy_error(w, what, m, n, H, &v), "nvfp4_proxy_error");
  return v;
}

inline float nvfp4_level(uint8_t code) {
  constexpr float levels[8] = {0, .5f, 1, 1.5f, 2, 3, 4, 6};
  return (code & 8 ? -1.f : 1.f) * levels[code & 7];
}

// The stream argument is accepted for source compatibility; the work runs on the context's own stream and the call
// returns when the tensors are on the host.
inline std::vector<Nvfp4Tensor> nvfp4_quantize_group(hipStream_t, const std::vector<const float*>& ws,
                                                     const std::vector<int>& ms, int n, const float* H,
                                                     const Nvfp4Opts& opt, bool* calibrated = nullptr) {
  if (ws.size() != ms.size()) detail::die("nvfp4_quantize_group: ws and ms differ in length");
  std::vector<Nvfp4Tensor> out(ws.size());
  std::vector<qtip_nvfp4_matrix> mats(ws.size());
  for (size_t i = 0; i < ws.size(); ++i) {
    out[i].m = ms[i], out[i].n = n;
    out[i].packed.resize(size_t(ms[i] > 0 ? ms[i] : 0) * size_t(n > 0 ? n / 2 : 0));
    out[i].scales.resize(size_t(ms[i] > 0 ? ms[i] : 0) * size_t(n > 0 ? n / 16 : 0));
    mats[i] = qtip_nvfp4_matrix{ms[i], ws[i], out[i].packed.data(), out[i].scales.data(), 1.f};
  }
  qtip_nvfp4_opts o{opt.scale_search ? 1 : 0, opt.calibrate ? 1 : 0, opt.sigma_reg, 0};
  int used = 0;
  detail::check(qtip_nvfp4_quantize_group(detail::context(), int(mats.size()), mats.data(), n, H, &o, &used),
                "nvfp4_quantize_group");
  for (size_t i = 0; i < ws.size(); ++i) out[i].global = mats[i].global;
  if (calibrated) *calibrated = used != 0;
  return out;
}

// src/safetensors.hpp:52-70: same calls, same file bytes.
class SafeTensorsWriter {
 public:
  SafeTensorsWriter() { detail::check(qtip_st_create(&w_), "SafeTensorsWriter"); }
  ~SafeTensorsWriter() { qtip_st_destroy(w_); }
  SafeTensorsWriter(const SafeTensorsWriter&) = delete;
  SafeTensorsWriter& operator=(const SafeTensorsWriter&) = delete;
  void add(const std::string& name, const std::string& dtype, const std::vector<int64_t>& shape, const void* data,
           size_t bytes) {
    detail::check(qtip_st_add(w_, name.c_str(), dtype.c_str(), shape.data(), int(shape.size()), data, bytes),
                  "SafeTensorsWriter::add");
  }
  // the six tensors write_layer_file stores for a QTIP linear (src/pipeline.cpp:329-340); tlut_f16 null = HYB table
  void add_qtip_linear(const std::string& prefix, const LinearOut& r, const uint16_t* tlut_f16 = nullptr) {
    qtip_linear_out o{const_cast<uint16_t*>(r.trellis.data()), const_cast<uint16_t*>(r.su_bf16.data()),
                      const_cast<float*>(r.sv.data()), nullptr, r.wscale, 0.0, 0.0, 0.0};
    detail::check(qtip_st_add_qtip_linear(w_, prefix.c_str(), &o, r.m, r.n, tlut_f16), "SafeTensorsWriter::add_qtip_linear");
  }
  // the three tensors write_layer_file stores for an NVFP4 linear (src/pipeline.cpp:342-346)
  void add_nvfp4_linear(const std::string& prefix, const Nvfp4Tensor& t) {
    add(prefix + "weight_packed", "U8", {t.m, int64_t(t.n) / 2}, t.packed.data(), t.packed.size());
    add(prefix + "weight_scale", "F8_E4M3", {t.m, int64_t(t.n) / 16}, t.scales.data(), t.scales.size());
    add(prefix + "weight_global_scale", "F32", {}, &t.global, 4);
  }
  size_t write(const std::string& path, const std::map<std::string, std::string>& metadata = {{"format", "pt"}}) const {
    std::vector<const char*> kv;
    for (auto& e : metadata) kv.push_back(e.first.c_str()), kv.push_back(e.second.c_str());
    static const char* const none[2] = {nullptr, nullptr};
    uint64_t bytes = 0;
    detail::check(qtip_st_write(w_, path.c_str(), kv.empty() ? none : kv.data(), int(metadata.size()), &bytes),
                  "SafeTensorsWriter::write");
    return size_t(bytes);
  }

 private:
  qtip_st_writer* w_ = nullptr;
};

}  // namespace qtip
