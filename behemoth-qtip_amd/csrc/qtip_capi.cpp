// extern "C" surface of libqtip_mi355.so (declared in include/qtip_mi355.h).  Exceptions thrown by the
// implementation stop here and become return codes plus a thread-local message.
#include <algorithm>
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <exception>
#include <vector>
#include <memory>
#include <new>

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
  } catch (...) {
    set_last_error("unknown exception");
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
  int slots = viterbi_max_slots(c->device);
  if (c->vit_slots_limit > 0) slots = std::min(slots, c->vit_slots_limit);
  if (c->vit_slots >= slots) return;
  QTIP_HIP(hipStreamSynchronize(c->stream));  // nothing may still use the smaller workspace
  c->vit_slots = 0;
  c->vit_ws.alloc(viterbi_workspace_bytes(slots));
  c->vit_slots = slots;  // only once the workspace exists
}

// the context's stream waits for `other` (or the reverse): an event recorded on one, waited for on the other
void order_streams(hipStream_t first, hipStream_t then) {
  hipEvent_t e;
  QTIP_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
  hipError_t rc = hipEventRecord(e, first);
  if (rc == hipSuccess) rc = hipStreamWaitEvent(then, e, 0);
  (void)hipEventDestroy(e);  // released once the recorded work has completed
  QTIP_HIP(rc);
}

namespace {
// a context on the current device: stream, codebook (cb_from's, or the default one), Hadamard tables
qtip_ctx* make_context(int device, const HostCodebook* cb_from, hipStream_t own_stream = nullptr) {
  struct Cleanup {
    qtip_ctx* c;
    ~Cleanup() {
      if (c) {
        if (c->stream) (void)hipStreamDestroy(c->stream);
        delete c;
      }
    }
  } guard{new qtip_ctx()};
  qtip_ctx* c = guard.c;
  c->device = device;
  c->stream = own_stream;  // a stream the caller made for this context (released with it), else one made here
  if (!c->stream) QTIP_HIP(hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking));
  c->arena.streams.push_back(&c->stream);
  for (hipStream_t& cs : c->chain_stream) c->arena.streams.push_back(&cs);
  if (cb_from) c->cb = *cb_from;
  else c->cb.build(nullptr);
  upload_codebook(c);
  c->rht.init(device, c->stream);
  c->vit_stats.alloc(4);
  QTIP_HIP(hipMemset(c->vit_stats.p, 0, 4 * sizeof(unsigned)));
  guard.c = nullptr;
  return c;
}

// The side streams of a context - two more LDLQ chains and the factorization's - only run beside its own stream
// and beside each other where each has a hardware queue to itself, and the runtime deals the few queues of a process
// (four unless the environment said otherwise before it started) to streams as they are made, the caller's own
// included; nothing tells which stream got which.  Timing does: a wave that sleeps for half a millisecond on each of
// two streams takes half a millisecond if they have queues of their own and a whole one if they share.  Candidates
// are made one after the other and kept if such a wave on each of the streams kept so far and on the candidate
// finishes in well under two delays (in one of three tries: a stream's first launch also sets its queue up); the
// others are released.  Up to three are kept: chain_stream[0], chain_stream[1], ldl_stream.  With all three LDLQ
// defaults to three chains whatever the environment says.  The caller's streams may share queues with these: they
// are idle while a call of this library runs.  Any failure leaves the streams to be made on first use, as before.
void find_side_streams(qtip_ctx* c) {
  constexpr int kCandidates = 12;
  constexpr double kDelayUs = 500.0;
  std::vector<hipStream_t> kept, dropped;
  hipStream_t upload = nullptr;
  try {
    // a delay on the context's stream, on the first `count` streams kept and on cand, all queued at once: microseconds
    auto side_by_side_us = [&](size_t count, hipStream_t cand) {
      auto wait_all = [&] {
        QTIP_HIP(hipStreamSynchronize(c->stream));
        for (size_t i = 0; i < count; ++i) QTIP_HIP(hipStreamSynchronize(kept[i]));
        QTIP_HIP(hipStreamSynchronize(cand));
      };
      wait_all();
      const auto t0 = std::chrono::steady_clock::now();
      launch_delay(kDelayUs, c->stream);
      for (size_t i = 0; i < count; ++i) launch_delay(kDelayUs, kept[i]);
      launch_delay(kDelayUs, cand);
      wait_all();
      return std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count();
    };
    auto beside = [&](size_t count, hipStream_t cand) {
      for (int attempt = 0; attempt < 3; ++attempt)  // the first launch on a stream also sets its queue up
        if (side_by_side_us(count, cand) < 1.5 * kDelayUs) return true;
      return false;
    };
    launch_delay(1.0, c->stream);  // the kernel's code is on the device before anything is timed
    QTIP_HIP(hipStreamSynchronize(c->stream));
    for (int i = 0; i < kCandidates && kept.size() < 3; ++i) {
      hipStream_t s = nullptr;
      QTIP_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
      dropped.push_back(s);  // until shown otherwise
      if (beside(kept.size(), s)) {
        dropped.pop_back();
        kept.push_back(s);
      }
    }
    // The stream that brings host inputs up needs no queue of its own, but it had better share the factorization's,
    // which has time to spare, than a chain's: a candidate that runs beside the context's stream and the two chain
    // streams shares the third stream's queue or none of these four.
    if (kept.size() == 3) {
      for (size_t i = 0; i < dropped.size() && !upload; ++i)
        if (beside(2, dropped[i])) {
          upload = dropped[i];
          dropped.erase(dropped.begin() + long(i));
        }
      for (int i = 0; i < 8 && !upload; ++i) {  // none among them: a few more candidates, for this alone
        hipStream_t s = nullptr;
        QTIP_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
        dropped.push_back(s);  // until shown otherwise
        if (beside(2, s)) {
          dropped.pop_back();
          upload = s;
        }
      }
    }
  } catch (...) {
    for (hipStream_t s : kept) dropped.push_back(s);
    kept.clear();
    if (upload) dropped.push_back(upload);
    upload = nullptr;
  }
  for (hipStream_t s : dropped) {
    (void)hipStreamSynchronize(s);
    (void)hipStreamDestroy(s);
  }
  if (kept.size() > 0) c->chain_stream[0] = kept[0];
  if (kept.size() == 2) c->ldl_stream = kept[1];  // two chains and the factorization beside them
  if (kept.size() == 3) c->chain_stream[1] = kept[1], c->ldl_stream = kept[2];
  c->upload_stream = upload;
  c->side_streams = int(kept.size());
}

void destroy_context(qtip_ctx* ctx) {
  ctx->arena.children.clear();
  for (qtip_ctx*& l : ctx->lane)
    if (l) {
      destroy_context(l);
      l = nullptr;
    }
  if (ctx->ldl_stream && ctx->ldl_stream != ctx->stream) {  // (a lane factors on its one stream)
    (void)hipStreamSynchronize(ctx->ldl_stream);
    (void)hipStreamDestroy(ctx->ldl_stream);
  }
  ctx->ldl_stream = nullptr;
  if (ctx->upload_stream) {
    (void)hipStreamSynchronize(ctx->upload_stream);
    (void)hipStreamDestroy(ctx->upload_stream);
    ctx->upload_stream = nullptr;
  }
  for (hipStream_t& cs : ctx->chain_stream)
    if (cs) {
      (void)hipStreamSynchronize(cs);
      (void)hipStreamDestroy(cs);
      cs = nullptr;  // the context's buffers go back to its arena below, which must not wait for a stream that is gone
    }
  if (ctx->stream) {
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipStreamDestroy(ctx->stream);
    ctx->stream = nullptr;
  }
  delete ctx;
}
}  // namespace

// A stream for lane k that runs beside the streams of the lanes made before it, found by timing as the side streams
// of a context are: lanes only share the chip if each has a hardware queue of its own, and which queue a new stream
// gets is the runtime's choice (with 16 queues asked for, twelve streams made in a row came out with shared queues
// on some boxes and not on others: 141-151 against 215 Mweights/s for twelve lanes of 1024 x 1024 groups).  The
// parent's own streams may share a lane's queue: they are idle while lanes run.  Null when no candidate passed (the
// process has fewer queues than lanes): the search is then given up for the later lanes too.
hipStream_t lane_stream_beside(qtip_ctx* parent, int k) {
  constexpr int kCandidates = 24;
  constexpr double kDelayUs = 500.0;
  std::vector<hipStream_t> others;
  for (int j = 0; j < k; ++j)
    if (parent->lane[j]) others.push_back(parent->lane[j]->stream);
  if (others.empty() || parent->lane_streams_exhausted) return nullptr;
  std::vector<hipStream_t> dropped;
  hipStream_t found = nullptr;
  try {
    auto wait_all = [&](hipStream_t cand) {
      for (hipStream_t o : others) QTIP_HIP(hipStreamSynchronize(o));
      QTIP_HIP(hipStreamSynchronize(cand));
    };
    auto beside = [&](hipStream_t cand) {
      for (int attempt = 0; attempt < 3; ++attempt) {  // the first launch on a stream also sets its queue up
        wait_all(cand);
        const auto t0 = std::chrono::steady_clock::now();
        for (hipStream_t o : others) launch_delay(kDelayUs, o);
        launch_delay(kDelayUs, cand);
        wait_all(cand);
        if (std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count() < 1.5 * kDelayUs)
          return true;
      }
      return false;
    };
    for (int i = 0; i < kCandidates && !found; ++i) {
      hipStream_t s = nullptr;
      QTIP_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
      dropped.push_back(s);  // until shown otherwise
      if (beside(s)) {
        dropped.pop_back();
        found = s;
      }
    }
  } catch (...) {
    if (found) dropped.push_back(found);
    found = nullptr;
  }
  for (hipStream_t s : dropped) {
    (void)hipStreamSynchronize(s);
    (void)hipStreamDestroy(s);
  }
  if (!found) parent->lane_streams_exhausted = true;
  return found;
}

qtip_ctx* lane_context(qtip_ctx* parent, int k) {
  QTIP_REQUIRE(k >= 0 && k < qtip_ctx::kMaxLanes, "lane %d of %d", k, qtip_ctx::kMaxLanes);
  if (!parent->lane[k]) {
    hipStream_t own = lane_stream_beside(parent, k);
    try {
      parent->lane[k] = make_context(parent->device, &parent->cb, own);
    } catch (...) {
      if (own) (void)hipStreamDestroy(own);
      throw;
    }
    // one stream per lane, the factorization's work included: a stream only runs beside the others if it has a
    // hardware queue to itself, and a process has few of them (GPU_MAX_HW_QUEUES, 4 unless the environment says
    // more); with a stream more per lane for the factorization 1024 x 1024 groups ran at 59 instead of 134 Mweights/s
    parent->lane[k]->ldl_stream = parent->lane[k]->stream;
    parent->lane[k]->arena.parent = &parent->arena;
    parent->arena.children.push_back(&parent->lane[k]->arena);
    parent->lane[k]->vit_mode = parent->vit_mode;
    parent->lane[k]->vit_margin = parent->vit_margin;
  }
  return parent->lane[k];
}

void release_lanes(qtip_ctx* parent) {
  parent->arena.children.clear();
  parent->lane_streams_exhausted = false;
  for (qtip_ctx*& l : parent->lane)
    if (l) {
      destroy_context(l);
      l = nullptr;
    }
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
    int prev = 0;
    QTIP_HIP(hipGetDevice(&prev));
    QTIP_HIP(hipSetDevice(device));
    // a failure below must not leave another device current
    struct Restore {
      int prev;
      ~Restore() { (void)hipSetDevice(prev); }
    } restore{prev};
    qtip_ctx* c = make_context(device, nullptr);
    try {
      viterbi_static_scratch_init(device);
      find_side_streams(c);
    } catch (...) {
      destroy_context(c);
      throw;
    }
    *out = c;
  });
}

void qtip_destroy(qtip_ctx* ctx) {
  if (!ctx) return;
  int prev = 0;
  (void)hipGetDevice(&prev);
  (void)hipSetDevice(ctx->device);
  destroy_context(ctx);
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
    ctx->lut_h2_valid = false;
    release_lanes(ctx);  // they carry the old codebook; the next call that wants lanes makes new ones
  });
}

int qtip_stream_wait(qtip_ctx* ctx, void* caller_stream) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr, "null context");
    DeviceGuard g(ctx);
    order_streams(static_cast<hipStream_t>(caller_stream), ctx->stream);
  });
}

int qtip_stream_signal(qtip_ctx* ctx, void* caller_stream) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr, "null context");
    DeviceGuard g(ctx);
    order_streams(ctx->stream, static_cast<hipStream_t>(caller_stream));
  });
}

int qtip_device_lut(qtip_ctx* ctx, const uint32_t** dev_lut_h2) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr && dev_lut_h2 != nullptr, "device_lut: bad arguments");
    DeviceGuard g(ctx);
    if (!ctx->lut_h2_valid) {
      std::vector<uint32_t> h2(static_cast<size_t>(kStates));
      for (uint32_t s = 0; s < uint32_t(kStates); ++s) {
        const uint32_t e = HostCodebook::entry_of_state(s);
        const uint32_t h0 = uint32_t(ctx->cb.tlut_h[e & 511u][0]) ^ ((e >> 9) ? 0x8000u : 0u);
        h2[s] = h0 | (uint32_t(ctx->cb.tlut_h[e & 511u][1]) << 16);
      }
      ctx->d_lut_h2.ensure(h2.size());
      QTIP_HIP(hipMemcpyAsync(ctx->d_lut_h2, h2.data(), h2.size() * 4, hipMemcpyHostToDevice, ctx->stream));
      QTIP_HIP(hipStreamSynchronize(ctx->stream));
      ctx->lut_h2_valid = true;
    }
    *dev_lut_h2 = ctx->d_lut_h2.p;
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

int qtip_trim(qtip_ctx* ctx, unsigned long long* bytes_released) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr, "null context");
    DeviceGuard g(ctx);
    unsigned long long total = ctx->arena.trim();
    for (qtip_ctx* l : ctx->lane)
      if (l) total += l->arena.trim();
    if (bytes_released) *bytes_released = total;
  });
}

long qtip_selftest_device_alloc_calls(void) { return test_device_alloc_calls(); }

int qtip_set_viterbi_mode(qtip_ctx* ctx, int mode, unsigned margin_units) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr && mode >= 0 && mode <= 3, "set_viterbi_mode: mode must be 0, 1, 2 or 3");
    ctx->vit_mode = mode == 1 ? 1 : 0;
    ctx->vit_wide = mode == 2 ? 0 : mode == 3 ? 1 : -1;
    ctx->vit_margin = margin_units ? margin_units : kViterbiMargin;
    for (qtip_ctx* l : ctx->lane)
      if (l) l->vit_mode = ctx->vit_mode, l->vit_wide = ctx->vit_wide, l->vit_margin = ctx->vit_margin;
  });
}

int qtip_ldlq_default_chains(qtip_ctx* ctx, int* chains) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr && chains != nullptr, "ldlq_default_chains: null argument");
    *chains = ldlq_default_chains(ctx);
  });
}

int qtip_viterbi_stats(qtip_ctx* ctx, unsigned long long* redone_first, unsigned long long* redone_second, int reset) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr, "null context");
    DeviceGuard g(ctx);
    unsigned long long sum[2] = {0, 0};
    auto take = [&](qtip_ctx* c) {
      QTIP_HIP(hipDeviceSynchronize());
      unsigned v[4];
      QTIP_HIP(hipMemcpy(v, c->vit_stats.p, sizeof v, hipMemcpyDeviceToHost));
      sum[0] += v[0], sum[1] += v[1];
      if (reset) QTIP_HIP(hipMemset(c->vit_stats.p, 0, sizeof v));
    };
    take(ctx);
    for (qtip_ctx* l : ctx->lane)
      if (l) take(l);
    if (redone_first) *redone_first = sum[0];
    if (redone_second) *redone_second = sum[1];
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
    ctx->viterbi_settings(job);
    launch_viterbi_tiles(job, ctx->d_entry_d, ctx->d_entry_f, ctx->vit_ws, ctx->vit_slots, ctx->stream);
  });
}

int qtip_viterbi_tiles_dev_noalloc(qtip_ctx* ctx, const float* dev_X, long B, uint16_t* dev_states,
                                   uint16_t* dev_packed) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr && B >= 0, "viterbi_tiles_noalloc: bad arguments");
    QTIP_REQUIRE(B <= QTIP_NOALLOC_MAX_TILES, "viterbi_tiles_noalloc: B = %ld exceeds the maximum of %d tiles per call",
                 B, QTIP_NOALLOC_MAX_TILES);
    if (B == 0) return;
    QTIP_REQUIRE(dev_X != nullptr, "viterbi_tiles_noalloc: X is null");
    DeviceGuard g(ctx);
    void* ws = viterbi_static_scratch(ctx->device);
    QTIP_REQUIRE(ws != nullptr, "viterbi_tiles_noalloc: no static scratch on device %d", ctx->device);
    TileJob job;
    job.X = dev_X;
    job.tiles = B;
    job.states = dev_states;
    job.packed = dev_packed;
    ctx->viterbi_settings(job);
    launch_viterbi_tiles(job, ctx->d_entry_d, ctx->d_entry_f, ws, viterbi_static_slots(), ctx->stream);
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

int qtip_decode_trellis_dev(qtip_ctx* ctx, const uint16_t* dev_trellis, int m, int n, float* dev_hatWr) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr && dev_trellis && dev_hatWr, "decode_trellis: bad arguments");
    DeviceGuard g(ctx);
    launch_decode_trellis(dev_trellis, m, n, ctx->d_entry_f, dev_hatWr, n, ctx->stream);
  });
}

int qtip_dequantize_linear(qtip_ctx* ctx, const uint16_t* host_trellis, const uint16_t* host_su_bf16,
                           const float* host_sv, float wscale, int m, int n, float* hatW, int hatW_on_device) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr && host_trellis && host_su_bf16 && host_sv && hatW, "dequantize_linear: bad arguments");
    QTIP_REQUIRE(m > 0 && n > 0 && m % 32 == 0 && n % 32 == 0, "dequantize_linear: m, n must be multiples of 32 (m=%d n=%d)", m, n);
    QTIP_REQUIRE(had_K(m) > 0 && had_K(n) > 0, "dequantize_linear: no Hadamard transform of size %d x %d", m, n);
    DeviceGuard g(ctx);
    hipStream_t s = ctx->stream;
    const size_t words = size_t(m / 16) * (n / 16) * 32;
    DBuf<uint16_t> tr(words);
    DBuf<float> a(size_t(n) * m), b(size_t(m) * n), d_su(n), d_sv(m);
    std::vector<float> su(n);
    for (int i = 0; i < n; ++i) su[i] = bf16_to_f32(host_su_bf16[i]);
    QTIP_HIP(hipMemcpyAsync(tr, host_trellis, words * 2, hipMemcpyHostToDevice, s));
    QTIP_HIP(hipMemcpyAsync(d_su, su.data(), size_t(n) * 4, hipMemcpyHostToDevice, s));
    QTIP_HIP(hipMemcpyAsync(d_sv, host_sv, size_t(m) * 4, hipMemcpyHostToDevice, s));
    launch_decode_trellis(tr, m, n, ctx->d_entry_f, b, n, s);
    // same operation order as the reconstruction at the end of quantize_group (src/quantizer.cpp:321-338), starting
    // from hatWr^T, so that both give the same bits
    ctx->rht.transpose(b, m, n, n, a, m);
    ctx->rht.hadamard_rows(a, n, m, m, false);
    ctx->rht.transpose(a, n, m, m, b, n);
    ctx->rht.hadamard_rows(b, m, n, n, false);
    ctx->rht.scale(b, m, n, n, wscale);
    launch_scale_rc(b, m, n, n, d_sv, d_su, s);
    QTIP_HIP(hipMemcpyAsync(hatW, b, size_t(m) * n * 4, hatW_on_device ? hipMemcpyDeviceToDevice : hipMemcpyDeviceToHost, s));
    QTIP_HIP(hipStreamSynchronize(s));
  });
}

int qtip_had_K(int n) { return had_K(n); }

void qtip_sign_vector(uint64_t seed, long count, float* host_out) {
  if (!host_out) return;
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
  o->ldl_device_updates = 1;
  o->ldlq_chains = 0;
  o->group_lanes = 0;
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

int qtip_hessian_accumulate_dev(qtip_ctx* ctx, const uint16_t* dev_X_bf16, long rows, int n, float* dev_H) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr, "hessian_accumulate: bad arguments");
    DeviceGuard g(ctx);
    launch_hessian_accumulate(dev_X_bf16, rows, n, dev_H, ctx->hess_img, ctx->stream);
  });
}
int qtip_hessian_finish_dev(qtip_ctx* ctx, float* dev_H, int n, double scale) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr, "hessian_finish: bad arguments");
    DeviceGuard g(ctx);
    launch_hessian_finish(dev_H, n, float(scale), ctx->stream);
  });
}

uint8_t qtip_f32_to_fp8e4m3(float x) { return f32_to_fp8e4m3(x); }
int qtip_nvfp4_quantize(const float* host_w, int m, int n, uint8_t* host_packed, uint8_t* host_scales, float* global) {
  return guarded([&] { nvfp4_quantize_host(host_w, m, n, host_packed, host_scales, global); });
}
int qtip_nvfp4_dequantize(const uint8_t* host_packed, const uint8_t* host_scales, float global, int m, int n,
                          float* host_out) {
  return guarded([&] { nvfp4_dequantize_host(host_packed, host_scales, global, m, n, host_out); });
}
int qtip_nvfp4_proxy_error(const float* host_w, const float* host_what, int m, int n, const float* host_H, double* out) {
  return guarded([&] {
    QTIP_REQUIRE(out != nullptr, "nvfp4_proxy_error: out is null");
    *out = nvfp4_proxy_error_host(host_w, host_what, m, n, host_H);
  });
}
int qtip_nvfp4_prepare(const float* host_H, int n, double sigma_reg, int calibrate, int threads, float* host_L,
                       float* host_dw) {
  return guarded([&] { nvfp4_prepare_host(host_H, n, sigma_reg, calibrate != 0, threads, host_L, host_dw); });
}
int qtip_nvfp4_prepare_device_updates(qtip_ctx* ctx, const float* host_H, int n, double sigma_reg, int threads,
                                      float* host_L, float* host_dw) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr, "nvfp4_prepare_device_updates: bad arguments");
    DeviceGuard g(ctx);
    nvfp4_prepare_assisted_impl(ctx, host_H, n, sigma_reg, threads, host_L, host_dw);
  });
}
int qtip_nvfp4_quantize_prepared(qtip_ctx* ctx, int nmat, qtip_nvfp4_matrix* mats, int n, const float* host_L,
                                 const float* host_dw, int scale_search) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr, "nvfp4_quantize_prepared: bad arguments");
    DeviceGuard g(ctx);
    nvfp4_quantize_prepared_impl(ctx, nmat, mats, n, host_L, host_dw, scale_search != 0);
  });
}
int qtip_nvfp4_quantize_group(qtip_ctx* ctx, int nmat, qtip_nvfp4_matrix* mats, int n, const float* host_H,
                              const qtip_nvfp4_opts* opts, int* calibrated) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr && n > 0 && n % 16 == 0, "nvfp4_quantize_group: bad arguments");
    DeviceGuard g(ctx);
    qtip_nvfp4_opts o{1, 1, 1e-2, 0};
    if (opts) o = *opts;
    const bool cal = o.calibrate != 0 && host_H != nullptr;
    if (calibrated) *calibrated = cal ? 1 : 0;
    std::vector<float> dw;
    float* L = nullptr;
    if (host_H) {
      dw.resize(static_cast<size_t>(n));
      if (cal) {
        // the factor goes through a page-locked buffer the context keeps (the staging of qtip_run_groups): no 3.3 GB
        // of fresh pages per call at n = 28672, and an upload at the bus's rate
        const size_t nn = size_t(n) * n;
        if (ctx->ring_L[0].n < nn) ctx->ring_L[0].alloc(nn);
        L = ctx->ring_L[0].p;
      }
      if (cal && !o.factor_on_host) nvfp4_prepare_assisted_impl(ctx, host_H, n, o.sigma_reg, 16, L, dw.data());
      else nvfp4_prepare_host(host_H, n, o.sigma_reg, cal, 16, L, dw.data());
    }
    nvfp4_quantize_prepared_impl(ctx, nmat, mats, n, L, host_H ? dw.data() : nullptr, o.scale_search != 0);
  });
}

int qtip_run_groups(qtip_ctx* ctx, int ngroups, const qtip_group* groups, const qtip_opts* opts, qtip_timing* timings,
                    double* ldl_wait_s) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr, "run_groups: bad arguments");
    DeviceGuard g(ctx);
    qtip_opts o;
    qtip_default_opts(&o);
    if (opts) o = *opts;
    run_groups_impl(ctx, ngroups, groups, o, timings, ldl_wait_s);
  });
}

int qtip_group_lanes(qtip_ctx* ctx, int ngroups, const qtip_group* groups, const qtip_opts* opts, int* lanes) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr && lanes != nullptr && ngroups >= 0 && (ngroups == 0 || groups),
                 "group_lanes: bad arguments");
    qtip_opts o;
    qtip_default_opts(&o);
    if (opts) o = *opts;
    *lanes = group_lanes_for(ngroups, groups, o, viterbi_max_slots(ctx->device));
  });
}

int qtip_selftest_group_lanes(int device_slots, int ngroups, int m, int n, int requested, int* lanes) {
  // host only: the lane rule for `ngroups` equal groups of one m x n linear each
  return guarded([&] {
    QTIP_REQUIRE(lanes != nullptr && ngroups >= 0 && ngroups <= 4096 && m > 0 && n > 0, "selftest: bad arguments");
    qtip_linear_in lin{};
    lin.m = m;
    std::vector<qtip_group> groups(static_cast<size_t>(ngroups));
    for (qtip_group& g : groups) {
      g = qtip_group{};
      g.nlin = 1, g.lins = &lin, g.n = n;
    }
    qtip_opts o;
    qtip_default_opts(&o);
    o.group_lanes = requested;
    *lanes = group_lanes_for(ngroups, groups.data(), o, device_slots);
  });
}

int qtip_reserve_groups(qtip_ctx* ctx, int n) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr && n > 0, "reserve_groups: bad arguments");
    DeviceGuard g(ctx);
    reserve_group_ring(ctx, n, 3);
  });
}

int qtip_selftest_failed_alloc_is_retried(void) {
  // host only: the next two device allocations are made to fail; a buffer whose allocation failed must stay empty,
  // so that the next ensure() allocates again instead of handing a null pointer to a kernel
  return guarded([&] {
    DBuf<double> b;
    test_fail_next_device_allocs(2);
    for (int attempt = 0; attempt < 2; ++attempt) {
      const long calls = test_device_alloc_calls();
      bool threw = false;
      try {
        b.ensure(1024);
      } catch (const Error& e) {
        threw = e.code == QTIP_E_HIP;
      }
      test_fail_next_device_allocs(1 - attempt);
      QTIP_REQUIRE(threw, "attempt %d: a failed allocation did not raise", attempt);
      QTIP_REQUIRE(test_device_alloc_calls() == calls + 1, "attempt %d: ensure() did not try to allocate", attempt);
      QTIP_REQUIRE(b.p == nullptr && b.n == 0, "attempt %d: a failed allocation left n = %zu", attempt, b.n);
    }
    test_fail_next_device_allocs(0);
    // the same through an arena: a failed allocation is tried once more after the arena has let go of its idle
    // blocks, and a second failure leaves the buffer empty
    DeviceArena arena;
    ArenaScope scope(&arena);
    DBuf<float> a;
    test_fail_next_device_allocs(2);
    const long calls = test_device_alloc_calls();
    bool threw = false;
    try {
      a.ensure(4096);
    } catch (const Error& e) {
      threw = e.code == QTIP_E_HIP;
    }
    test_fail_next_device_allocs(0);
    QTIP_REQUIRE(threw, "arena: a failed allocation did not raise");
    QTIP_REQUIRE(test_device_alloc_calls() == calls + 2, "arena: a failed allocation was not tried again once");
    QTIP_REQUIRE(a.p == nullptr && a.n == 0 && a.from == nullptr, "arena: a failed allocation left n = %zu", a.n);
  });
}

int qtip_selftest_ldl_panel_handover(const float* host_HRr, int n, int threads, float* host_L) {
  return guarded([&] {
    QTIP_REQUIRE(host_HRr && host_L && n > 0 && n % 16 == 0, "ldl self test: bad arguments (n = %d)", n);
    if (!block_ldl_assisted_on_host(host_HRr, n, host_L, threads)) throw Error(QTIP_E_NOT_PD, "block LDL failed (H not PD)");
  });
}

int qtip_st_create(qtip_st_writer** out) {
  return guarded([&] {
    QTIP_REQUIRE(out != nullptr, "st_create: bad arguments");
    *out = st_new();
  });
}
void qtip_st_destroy(qtip_st_writer* w) { st_delete(w); }
int qtip_st_add(qtip_st_writer* w, const char* name, const char* dtype, const int64_t* shape, int rank,
                const void* data, uint64_t bytes) {
  return guarded([&] { st_add(w, name, dtype, shape, rank, data, size_t(bytes)); });
}
int qtip_st_add_qtip_linear(qtip_st_writer* w, const char* prefix, const qtip_linear_out* out, int m, int n,
                            const uint16_t* tlut_f16) {
  return guarded([&] {
    if (tlut_f16) {
      st_add_qtip_linear(w, prefix, out, m, n, tlut_f16);
    } else {
      HostCodebook cb;
      cb.build(nullptr);
      st_add_qtip_linear(w, prefix, out, m, n, &cb.tlut_h[0][0]);
    }
  });
}
int qtip_st_write(qtip_st_writer* w, const char* path, const char* const* metadata_kv, int nmeta,
                  uint64_t* bytes_written) {
  return guarded([&] {
    static const char* const kDefault[2] = {"format", "pt"};
    const size_t b = metadata_kv ? st_write(w, path, metadata_kv, nmeta) : st_write(w, path, kDefault, 1);
    if (bytes_written) *bytes_written = b;
  });
}
int qtip_get_tlut_f16(qtip_ctx* ctx, uint16_t* host_tlut_f16) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr && host_tlut_f16, "get_tlut_f16: bad arguments");
    std::memcpy(host_tlut_f16, &ctx->cb.tlut_h[0][0], 512 * 2 * 2);
  });
}

}  // extern "C"


extern "C" {

int qtip_hadamard_rows_dev(qtip_ctx* ctx, float* dev_X, long rows, int n, long ld, int transpose) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr && (rows == 0 || dev_X != nullptr), "hadamard_rows: bad arguments");
    DeviceGuard g(ctx);
    ctx->rht.hadamard_rows(dev_X, rows, n, ld, transpose != 0);
  });
}

int qtip_rotate_hessian(qtip_ctx* ctx, const float* H, int h_on_device, int n, uint64_t seed, double sigma_reg,
                        float* host_su, double* creg, float* host_HRr) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr, "null context");
    DeviceGuard g(ctx);
    rotate_hessian_impl(ctx, H, h_on_device != 0, n, seed, sigma_reg, host_su, creg, host_HRr);
  });
}

int qtip_ldl_hessian(const float* host_HRr, int n, int threads, float* host_L) {
  return guarded([&] { ldl_hessian_impl(host_HRr, n, threads, host_L); });
}

int qtip_cholesky_inplace(double* host_A, int n, int threads) {
  return guarded([&] {
    QTIP_REQUIRE(host_A != nullptr && n > 0, "cholesky_inplace: bad arguments (n = %d)", n);
    if (!cholesky_lower_host(host_A, n, threads)) throw Error(QTIP_E_NOT_PD, "Cholesky failed (matrix not PD)");
  });
}

int qtip_ldl_hessian_device_updates(qtip_ctx* ctx, const float* host_HRr, int n, int threads, float* host_L) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr, "null context");
    DeviceGuard g(ctx);
    ldl_hessian_assisted_impl(ctx, host_HRr, n, threads, host_L);
  });
}

int qtip_ldl_hessian_device_updates_dev(qtip_ctx* ctx, const float* dev_HRr, int n, int threads, float* host_L,
                                        float* dev_L) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr && dev_HRr != nullptr, "ldl_hessian (device updates): null context or Hessian");
    DeviceGuard g(ctx);
    ldl_hessian_assisted_impl(ctx, nullptr, n, threads, host_L, dev_HRr, dev_L);
  });
}

int qtip_ldlq_dev(qtip_ctx* ctx, const float* dev_WT, const float* dev_L, long n, long m, float* dev_hatWT,
                  uint16_t* dev_Q, int feedback, double* vit_seconds) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr && dev_WT && dev_L && dev_hatWT && dev_Q, "ldlq: bad arguments");
    DeviceGuard g(ctx);
    ldlq_impl(ctx, dev_WT, dev_L, n, m, dev_hatWT, dev_Q, feedback, vit_seconds, 0);
  });
}

int qtip_prod_cache_bf16x3_dev(qtip_ctx* ctx, int N, long K, const float* dev_Lrows, long ldl, const float* dev_WT,
                               const float* dev_hatWT, long ldw, float* dev_P) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr && dev_Lrows && dev_WT && dev_hatWT && dev_P, "prod_cache: bad arguments");
    QTIP_REQUIRE(N > 0 && N % 64 == 0 && K > 0 && K % 64 == 0 && ldl >= 128 && ldw >= N && ldl % 4 == 0 && ldw % 4 == 0,
                 "prod_cache: N and K must be multiples of 64 and the rows 16-byte aligned (N = %d, K = %ld)", N, K);
    DeviceGuard g(ctx);
    hipStream_t s = ctx->stream;
    // images [row][k], k contiguous: L's 128 columns, then the N columns of the residual
    DBuf<uint16_t> img(size_t(2) * (128 + N) * K);
    uint16_t *ah = img.p, *al = ah + size_t(128) * K, *bh = al + size_t(128) * K, *bl = bh + size_t(N) * K;
    launch_split_transpose_bf16(dev_Lrows, nullptr, ldl, K, 128, ah, al, K, false, s);
    launch_split_transpose_bf16(dev_WT, dev_hatWT, ldw, K, N, bh, bl, K, false, s);
    DBuf<float> parts(size_t(kMaxGatherSplits) * 128 * N);
    launch_gemm_img_gather(N, K, ah, al, K, bh, bl, K, dev_P, parts.p, ctx->vit_slots > 0 ? ctx->vit_slots : 768, s);
    QTIP_HIP(hipStreamSynchronize(s));
  });
}

int qtip_quantize_group(qtip_ctx* ctx, int nlin, const qtip_linear_in* lins, int n, uint64_t seed,
                        const float* host_su, double creg, const float* host_HRr, const float* host_L,
                        const qtip_opts* opts, qtip_linear_out* outs, qtip_timing* timing) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr, "null context");
    DeviceGuard g(ctx);
    qtip_opts o;
    qtip_default_opts(&o);
    if (opts) o = *opts;
    quantize_group_impl(ctx, nlin, lins, n, seed, host_su, creg, host_HRr, host_L, o, outs, timing);
  });
}

int qtip_quantize_group_h(qtip_ctx* ctx, int nlin, const qtip_linear_in* lins, int n, const float* H, int h_on_device,
                          uint64_t seed, const qtip_opts* opts, qtip_linear_out* outs, qtip_timing* timing) {
  return guarded([&] {
    QTIP_REQUIRE(ctx != nullptr && n > 0, "quantize_group: bad arguments");
    DeviceGuard g(ctx);
    qtip_opts o;
    qtip_default_opts(&o);
    if (opts) o = *opts;
    std::vector<float> su(static_cast<size_t>(n)), HRr(size_t(n) * n), L(size_t(n) * n);
    double creg = 0;
    qtip_timing T{};
    auto t0 = std::chrono::steady_clock::now();
    rotate_hessian_impl(ctx, H, h_on_device != 0, n, seed, o.sigma_reg, su.data(), &creg, HRr.data());
    auto t1 = std::chrono::steady_clock::now();
    if (o.ldl_device_updates) ldl_hessian_assisted_impl(ctx, HRr.data(), n, o.ldl_threads, L.data());
    else ldl_hessian_impl(HRr.data(), n, o.ldl_threads, L.data());
    auto t2 = std::chrono::steady_clock::now();
    T.rht = std::chrono::duration<double>(t1 - t0).count();
    T.ldl_cpu = std::chrono::duration<double>(t2 - t1).count();
    quantize_group_impl(ctx, nlin, lins, n, seed, su.data(), creg, HRr.data(), L.data(), o, outs, &T);
    if (timing) *timing = T;
  });
}

}  // extern "C"
