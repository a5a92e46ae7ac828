// extern "C" surface of libqtip_mi355.so (declared in include/qtip_mi355.h).  Exceptions thrown by the
// implementation stop here and become return codes plus a thread-local message.
#include <cstring>
#include <exception>
#include <memory>
#include <new>

#include "qtip_internal.hpp"
#include "quantizer_impl.hpp"

namespace qtipmi {
const std::string& last_error_ref();

template <class F>
static int guarded(F&& f) {
  try {
    f();
    return QTIP_OK;
  } catch (const Error& e) {
    set_last_error(e.what());
    return e.code;
  } catch (const std::bad_alloc&) {
    set_last_error("out of host memory");
    return QTIP_E_NOMEM;
  } catch (const std::exception& e) {
    set_last_error(e.what());
    return QTIP_E_ARG;
  }
}

struct DeviceGuard {  // makes the context's device current for the duration of a call
  int prev = -1;
  explicit DeviceGuard(const qtip_ctx* c) {
    QTIP_HIP(hipGetDevice(&prev));
    if (prev != c->device) QTIP_HIP(hipSetDevice(c->device));
  }
  ~DeviceGuard() { (void)hipSetDevice(prev); }
};

void upload_codebook(qtip_ctx* c) {
  c->d_entry_d.ensure(size_t(kLutEntries) * 2);
  c->d_entry_f.ensure(size_t(kLutEntries) * 2);
  QTIP_HIP(hipMemcpyAsync(c->d_entry_d, c->cb.entry_d, sizeof(c->cb.entry_d), hipMemcpyHostToDevice, c->stream));
  QTIP_HIP(hipMemcpyAsync(c->d_entry_f, c->cb.entry_f, sizeof(c->cb.entry_f), hipMemcpyHostToDevice, c->stream));
  QTIP_HIP(hipStreamSynchronize(c->stream));
}

void ensure_viterbi_workspace(qtip_ctx* c) {
  if (c->vit_slots > 0) return;
  c->vit_slots = viterbi_max_slots(c->device);
  c->vit_ws.alloc(viterbi_workspace_bytes(c->vit_slots));
}
}  // namespace qtipmi

using namespace qtipmi;

extern "C" {

const char* qtip_last_error(void) { return last_error_ref().c_str(); }

int qtip_create(int device, qtip_ctx** out) {
  return guarded([&] {
    QTIP_REQUIRE(out != nullptr, "qtip_create: out is null");
    *out = nullptr;
    int count = 0;
    QTIP_HIP(hipGetDeviceCount(&count));
    QTIP_REQUIRE(device >= 0 && device < count, "qtip_create: device %d of %d", device, count);
    hipDeviceProp_t prop;
    QTIP_HIP(hipGetDeviceProperties(&prop, device));
    QTIP_REQUIRE(std::strncmp(prop.gcnArchName, "gfx950", 6) == 0,
                 "qtip_create: device %d is %s; this library carries gfx950 code only", device, prop.gcnArchName);
    auto c = std::make_unique<qtip_ctx>();
    c->device = device;
    int prev = 0;
    QTIP_HIP(hipGetDevice(&prev));
    QTIP_HIP(hipSetDevice(device));
    QTIP_HIP(hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking));
    c->cb.build(nullptr);
    upload_codebook(c.get());
    (void)hipSetDevice(prev);
    *out = c.release();
  });
}

void qtip_destroy(qtip_ctx* ctx) {
  if (!ctx) return;
  int prev = 0;
  (void)hipGetDevice(&prev);
  (void)hipSetDevice(ctx->device);
  if (ctx->stream) {
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipStreamDestroy(ctx->stream);
  }
  delete ctx;
  (void)hipSetDevice(prev);
}

void* qtip_stream(qtip_ctx* ctx) { return ctx ? static_cast<void*>(ctx->stream) : nullptr; }

int qtip_synchronize(qtip_ctx* ctx) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr, "null context");
    QTIP_HIP(hipStreamSynchronize(ctx->stream));
  });
}

int qtip_set_tlut(qtip_ctx* ctx, const float* host_tlut) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr, "null context");
    DeviceGuard g(ctx);
    QTIP_HIP(hipStreamSynchronize(ctx->stream));
    ctx->cb.build(host_tlut);
    upload_codebook(ctx);
  });
}

double qtip_lut_rms(qtip_ctx* ctx) { return ctx ? ctx->cb.lut_rms : 0.0; }

int qtip_get_lut(qtip_ctx* ctx, float* lut0, float* lut1) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr, "null context");
    for (uint32_t s = 0; s < uint32_t(kStates); ++s) {
      const uint32_t e = HostCodebook::entry_of_state(s);
      if (lut0) lut0[s] = ctx->cb.entry_f[e][0];
      if (lut1) lut1[s] = ctx->cb.entry_f[e][1];
    }
  });
}

int qtip_viterbi_tiles_dev(qtip_ctx* ctx, const float* dev_X, long B, uint16_t* dev_states, uint16_t* dev_packed) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr && B >= 0, "viterbi_tiles: bad arguments");
    if (B == 0) return;
    QTIP_REQUIRE(dev_X != nullptr, "viterbi_tiles: X is null");
    DeviceGuard g(ctx);
    ensure_viterbi_workspace(ctx);
    TileJob job;
    job.X = dev_X;
    job.tiles = B;
    job.states = dev_states;
    job.packed = dev_packed;
    launch_viterbi_tiles(job, ctx->d_entry_d, ctx->d_entry_f, ctx->vit_ws, ctx->vit_slots, ctx->stream);
  });
}

int qtip_viterbi_tiles(qtip_ctx* ctx, const float* host_X, long B, uint16_t* host_states, uint16_t* host_packed) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr && B >= 0, "viterbi_tiles: bad arguments");
    if (B == 0) return;
    QTIP_REQUIRE(host_X != nullptr, "viterbi_tiles: X is null");
    DeviceGuard g(ctx);
    DBuf<float> dX(size_t(B) * kSeq);
    DBuf<uint16_t> dS(host_states ? size_t(B) * kSteps : 0), dP(host_packed ? size_t(B) * kWords : 0);
    QTIP_HIP(hipMemcpyAsync(dX, host_X, dX.bytes(), hipMemcpyHostToDevice, ctx->stream));
    int rc = qtip_viterbi_tiles_dev(ctx, dX, B, dS, dP);
    if (rc != QTIP_OK) throw Error(rc, last_error_ref());
    if (host_states) QTIP_HIP(hipMemcpyAsync(host_states, dS, dS.bytes(), hipMemcpyDeviceToHost, ctx->stream));
    if (host_packed) QTIP_HIP(hipMemcpyAsync(host_packed, dP, dP.bytes(), hipMemcpyDeviceToHost, ctx->stream));
    QTIP_HIP(hipStreamSynchronize(ctx->stream));
  });
}

int qtip_decode_states_dev(qtip_ctx* ctx, const uint16_t* dev_states, long B, float* dev_hat) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr && B >= 0 && (B == 0 || (dev_states && dev_hat)), "decode_states: bad arguments");
    DeviceGuard g(ctx);
    launch_decode_states(dev_states, B, dev_hat, ctx->d_entry_f, ctx->stream);
  });
}

int qtip_had_K(int n) { return had_K(n); }

void qtip_sign_vector(uint64_t seed, long count, float* host_out) {
  SplitMix r(seed);
  for (long i = 0; i < count; ++i) host_out[i] = r.sign();
}

void qtip_default_opts(qtip_opts* o) {
  if (!o) return;
  o->sigma_reg = 1e-2;
  o->scale_override = 0.9;
  o->ldl_threads = 16;
  o->feedback = 0;
  o->skip_proxy = 0;
}

void qtip_pack_trellis(const uint16_t* states, long B, uint16_t* packed) { pack_trellis_host(states, B, packed); }
void qtip_unpack_trellis(const uint16_t* packed, long B, uint16_t* states) { unpack_trellis_host(packed, B, states); }
int qtip_swizzle_for_kernel(const uint16_t* packed, int m, int n, uint16_t* out) {
  if (swizzle_host(packed, m, n, out)) return QTIP_OK;
  set_last_error("kernel layout needs m and n to be multiples of 32");
  return QTIP_E_ARG;
}
int qtip_unswizzle_for_kernel(const uint16_t* in, int m, int n, uint16_t* packed) {
  if (unswizzle_host(in, m, n, packed)) return QTIP_OK;
  set_last_error("kernel layout needs m and n to be multiples of 32");
  return QTIP_E_ARG;
}

}  // extern "C"

// ---- TEMPORARY: entry points still to be implemented
extern "C" {
#define QTIP_TODO(name) \
  qtipmi::set_last_error(#name ": not implemented yet"); \
  return QTIP_E_ARG
int qtip_hadamard_rows_dev(qtip_ctx*, float*, long, int, long, int) { QTIP_TODO(qtip_hadamard_rows_dev); }
int qtip_rotate_hessian(qtip_ctx*, const float*, int, int, uint64_t, double, float*, double*, float*) { QTIP_TODO(qtip_rotate_hessian); }
int qtip_ldl_hessian(const float*, int, int, float*) { QTIP_TODO(qtip_ldl_hessian); }
int qtip_ldlq_dev(qtip_ctx*, const float*, const float*, long, long, float*, uint16_t*, double*) { QTIP_TODO(qtip_ldlq_dev); }
int qtip_quantize_group(qtip_ctx*, int, const qtip_linear_in*, int, uint64_t, const float*, double, const float*, const float*, const qtip_opts*, qtip_linear_out*, qtip_timing*) { QTIP_TODO(qtip_quantize_group); }
int qtip_quantize_group_h(qtip_ctx*, int, const qtip_linear_in*, int, const float*, int, uint64_t, const qtip_opts*, qtip_linear_out*, qtip_timing*) { QTIP_TODO(qtip_quantize_group_h); }
}
