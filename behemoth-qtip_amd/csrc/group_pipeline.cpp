// Several Hessian groups through one context, scheduled like the reference's run_qtip_groups
// (src/pipeline.cpp:229-312): Hessians are rotated on the GPU ahead of use, a side thread runs the host fp64 LDL of
// the groups in order, and the calling thread quantizes group g as soon as its factor is there, so the LDL of group
// g+1 overlaps the GPU work of group g.  The reference rotates all Hessians of a layer up front and keeps every HRr;
// here rotation runs two groups ahead through a ring of three page-locked (HRr, L) pairs kept by the context, so
// host memory stays at 6 n^2 floats however many groups are queued.
#include <chrono>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <exception>
#include <mutex>
#include <thread>
#include <vector>

#include "quantizer_impl.hpp"

namespace qtipmi {
namespace {
double now_s() { return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count(); }
}  // namespace

void reserve_group_ring(qtip_ctx* c, int n, int depth) {
  QTIP_REQUIRE(n > 0 && depth >= 1 && depth <= 3, "reserve: bad arguments");
  const size_t need = size_t(n) * n;
  for (int b = 0; b < depth; ++b) {
    if (c->ring_HRr[b].n < need) {
      c->ring_HRr[b].alloc(need);
      std::memset(c->ring_HRr[b].p, 0, need * 4);
    }
    if (c->ring_L[b].n < need) {
      c->ring_L[b].alloc(need);
      std::memset(c->ring_L[b].p, 0, need * 4);
    }
  }
}

namespace {
// the groups one after the other through context c, the factorization of the next under the GPU work of the present
void run_groups_on(qtip_ctx* c, int ng, const qtip_group* groups, const qtip_opts& opt, qtip_timing* tms,
                   double* ldl_wait) {
  int nmax = 0;
  for (int g = 0; g < ng; ++g) nmax = std::max(nmax, groups[g].n);
  const int R = std::min(3, ng);
  reserve_group_ring(c, nmax, R);
  // with the LDL's updates on the device the rotated Hessian never leaves it: the factorization reads it there and so
  // does the proxy, and the factor goes up column block by column block as it is assembled: one copy down and three up
  // fewer per group on the quantizing stream (HRr in the host ring is then unused)
  const bool keep_dev = opt.ldl_device_updates != 0;
  if (keep_dev)
    for (int b = 0; b < R; ++b) {
      c->ring_dHRr[b].ensure(size_t(nmax) * nmax);
      c->ring_dL[b].ensure(size_t(nmax) * nmax);
    }
  const size_t ngz = size_t(ng);
  std::vector<std::vector<float>> su;
  for (int b = 0; b < R; ++b) su.emplace_back(std::vector<float>(static_cast<size_t>(nmax), 0.0f));
  std::vector<double> creg(ngz, 0.0), t_rot(ngz, 0.0), t_ldl(ngz, 0.0);

  std::mutex mu;
  std::condition_variable cv;
  int rotated = 0, factored = 0, loaded = 0, finished = 0;
  bool stop = false;
  std::exception_ptr ldl_err, load_err;

  // Inputs that arrive as host pointers (the reference's interface, src/quantizer.hpp:21-28, 75-77) are brought to the
  // device by a side thread on a stream of its own, up to three groups ahead, into a ring of four staging slots the
  // context keeps: the quantizing stream then only sees device-to-device copies.  On that stream a Hessian's 3.3 GB
  // and a group's 1.4 GB of weights from pageable memory held one of the LDLQ chains up for their whole length.
  constexpr int U = qtip_ctx::kUploadSlots;
  bool any_host = false;
  for (int g = 0; g < ng; ++g) {
    any_host = any_host || !groups[g].h_on_device;
    for (int i = 0; i < groups[g].nlin; ++i) any_host = any_host || !groups[g].lins[i].on_device;
  }
  std::vector<const float*> dH(ngz);
  std::vector<std::vector<qtip_linear_in>> dl(ngz);
  for (int g = 0; g < ng; ++g) {
    dH[size_t(g)] = groups[g].H;
    dl[size_t(g)].assign(groups[g].lins, groups[g].lins + groups[g].nlin);
  }
  auto padded = [](size_t bytes) { return (bytes + 255) / 256 * 256; };
  // bytes of staging group g's host weights take
  auto weight_bytes = [&](int g) {
    size_t total = 0;
    for (const qtip_linear_in& l : dl[size_t(g)]) {
      if (l.on_device) continue;
      const size_t mn = size_t(l.m) * size_t(groups[g].n);
      total += padded(l.w_f32 ? mn * 4 : l.w_bf16 ? mn * 2 : mn) + (l.w_fp8 && l.scale_bf16 ? padded(size_t(l.m) * 2) : 0);
    }
    return total;
  };
  auto upload = [&](int g) {
    const int b = g % U;
    hipStream_t us = c->upload_stream;
    const size_t nn = size_t(groups[g].n) * groups[g].n;
    if (!groups[g].h_on_device) {
      QTIP_REQUIRE(c->up_H[b].n >= nn, "run_groups: staging slot %d too small for the Hessian of group %d", b, g);
      QTIP_HIP(hipMemcpyAsync(c->up_H[b].p, groups[g].H, nn * 4, hipMemcpyHostToDevice, us));
      dH[size_t(g)] = c->up_H[b].p;
    }
    QTIP_REQUIRE(c->up_W[b].n >= weight_bytes(g), "run_groups: staging slot %d too small for the weights of group %d", b, g);
    size_t at = 0;
    for (qtip_linear_in& l : dl[size_t(g)]) {
      if (l.on_device) continue;
      const size_t mn = size_t(l.m) * size_t(groups[g].n);
      const void* src = l.w_f32 ? static_cast<const void*>(l.w_f32) : l.w_bf16 ? static_cast<const void*>(l.w_bf16)
                                                                            : static_cast<const void*>(l.w_fp8);
      if (!src) continue;  // refused with its message when the group is quantized
      const size_t bytes = l.w_f32 ? mn * 4 : l.w_bf16 ? mn * 2 : mn;
      uint8_t* dst = c->up_W[b].p + at;
      QTIP_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, us));
      at += padded(bytes);
      if (l.w_f32) l.w_f32 = reinterpret_cast<const float*>(dst);
      else if (l.w_bf16) l.w_bf16 = reinterpret_cast<const uint16_t*>(dst);
      else l.w_fp8 = dst;
      if (l.w_fp8 && l.scale_bf16) {
        uint8_t* sd = c->up_W[b].p + at;
        QTIP_HIP(hipMemcpyAsync(sd, l.scale_bf16, size_t(l.m) * 2, hipMemcpyHostToDevice, us));
        at += padded(size_t(l.m) * 2);
        l.scale_bf16 = reinterpret_cast<const uint16_t*>(sd);
      }
      l.on_device = 1;
    }
    QTIP_HIP(hipStreamSynchronize(us));
  };
  std::thread loader;
  if (any_host) {
    if (!c->upload_stream) QTIP_HIP(hipStreamCreateWithFlags(&c->upload_stream, hipStreamNonBlocking));
    // every slot a group will use is sized here, for the largest group that goes through it, before anything runs:
    // growing one later would be a hipFree (a wait for the whole device) and a hipMalloc in the middle of the pipeline
    for (int b = 0; b < std::min(U, ng); ++b) {
      size_t h_need = 0, w_need = 0;
      for (int g = b; g < ng; g += U) {
        if (!groups[g].h_on_device) h_need = std::max(h_need, size_t(groups[g].n) * groups[g].n);
        w_need = std::max(w_need, weight_bytes(g));
      }
      c->up_H[b].ensure(h_need);
      c->up_W[b].ensure(w_need);
    }
    loader = std::thread([&] {
      try {
        QTIP_HIP(hipSetDevice(c->device));  // this thread's own current device
        for (int g = 0; g < ng; ++g) {
          {
            std::unique_lock<std::mutex> lk(mu);
            cv.wait(lk, [&] { return finished >= g - (U - 1) || stop; });  // the slot's last user is through
            if (stop) return;
          }
          upload(g);
          std::lock_guard<std::mutex> lk(mu);
          loaded = g + 1;
          cv.notify_all();
        }
      } catch (...) {
        // copies queued before the failure still read the caller's memory: they are through before the error is seen
        (void)hipStreamSynchronize(c->upload_stream);
        std::lock_guard<std::mutex> lk(mu);
        load_err = std::current_exception();
        cv.notify_all();
      }
    });
  } else {
    loaded = ng;
  }
  struct JoinLoader {  // whatever ends this call, the loader is told and waited for, and so are its copies
    std::thread& t;
    std::mutex& mu;
    std::condition_variable& cv;
    bool& stop;
    hipStream_t& us;
    ~JoinLoader() {
      if (!t.joinable()) return;
      {
        std::lock_guard<std::mutex> lk(mu);
        stop = true;
        cv.notify_all();
      }
      t.join();
      if (us) (void)hipStreamSynchronize(us);
    }
  } join_loader{loader, mu, cv, stop, c->upload_stream};

  auto rotate = [&](int g) {
    {
      std::unique_lock<std::mutex> lk(mu);
      cv.wait(lk, [&] { return loaded > g || load_err; });
      if (loaded <= g) std::rethrow_exception(load_err);
    }
    const double t0 = now_s();
    const int b = g % R;
    rotate_hessian_impl(c, dH[size_t(g)], groups[g].h_on_device != 0 || dH[size_t(g)] != groups[g].H, groups[g].n,
                        groups[g].seed, opt.sigma_reg, su[size_t(b)].data(), &creg[size_t(g)],
                        keep_dev ? nullptr : c->ring_HRr[b].p, keep_dev ? c->ring_dHRr[b].p : nullptr);
    t_rot[size_t(g)] = now_s() - t0;
    std::lock_guard<std::mutex> lk(mu);
    rotated = g + 1;
    cv.notify_all();
  };
  rotate(0);

  std::thread ldl_thread([&] {
    for (int g = 0; g < ng; ++g) {
      {
        std::unique_lock<std::mutex> lk(mu);
        cv.wait(lk, [&] { return rotated > g || stop; });
        if (stop) return;
      }
      const double t0 = now_s();
      std::exception_ptr err;
      try {
        if (opt.ldl_device_updates) {
          QTIP_HIP(hipSetDevice(c->device));  // this thread's own current device
          ldl_hessian_assisted_impl(c, nullptr, groups[g].n, opt.ldl_threads, c->ring_L[g % R].p, c->ring_dHRr[g % R].p,
                                    c->ring_dL[g % R].p);
        } else {
          ldl_hessian_impl(c->ring_HRr[g % R].p, groups[g].n, opt.ldl_threads, c->ring_L[g % R].p);
        }
      } catch (...) {
        err = std::current_exception();
      }
      t_ldl[size_t(g)] = now_s() - t0;
      std::lock_guard<std::mutex> lk(mu);
      factored = g + 1;
      if (err) ldl_err = err;
      cv.notify_all();
      if (err) return;
    }
  });

  // The quantize loop stays on the calling thread at its own priority.  (Running it on a helper thread at nice 10,
  // in the batch class, or both made no difference to the LDL-bound rate: 70.6 / 70.7 / 70.5 / 70.2 Mweights/s on
  // one machine; a low-priority feeder only starves when a profiler makes each launch dearer.)
  std::exception_ptr feed_err;
  auto feed = [&] {
    try {
      if (ng > 1) rotate(1);  // while the first factorisation is already running
      for (int g = 0; g < ng; ++g) {
        const double tw = now_s();
        {
          std::unique_lock<std::mutex> lk(mu);
          cv.wait(lk, [&] { return factored > g || ldl_err; });
          if (factored <= g || (ldl_err && factored == g + 1)) std::rethrow_exception(ldl_err);
        }
        if (ldl_wait) ldl_wait[g] = now_s() - tw;
        if (g + 2 < ng) rotate(g + 2);  // into the buffers group g-1 has finished with
        const int b = g % R;
        qtip_timing T{};
        T.rht = t_rot[size_t(g)];
        T.ldl_cpu = t_ldl[size_t(g)];
        quantize_group_impl(c, groups[g].nlin, dl[size_t(g)].data(), groups[g].n, groups[g].seed, su[size_t(b)].data(),
                            creg[size_t(g)], keep_dev ? nullptr : c->ring_HRr[b].p, c->ring_L[b].p, opt, groups[g].outs, &T,
                            keep_dev ? c->ring_dHRr[b].p : nullptr, keep_dev ? c->ring_dL[b].p : nullptr);
        if (tms) tms[g] = T;
        {
          std::lock_guard<std::mutex> lk(mu);
          finished = g + 1;
          cv.notify_all();
        }
      }
    } catch (...) {
      feed_err = std::current_exception();
      std::lock_guard<std::mutex> lk(mu);
      stop = true;
      cv.notify_all();
    }
  };
  feed();
  ldl_thread.join();
  if (feed_err) std::rethrow_exception(feed_err);
}

// A lane's schedule: its groups one after the other on the lane's one stream - rotate, factor, quantize.  Nothing of a
// lane overlaps with itself; the other lanes fill the chip meanwhile.
void run_groups_in_line(qtip_ctx* c, int ng, const qtip_group* groups, const qtip_opts& opt, qtip_timing* tms,
                        double* ldl_wait) {
  int nmax = 0;
  for (int g = 0; g < ng; ++g) nmax = std::max(nmax, groups[g].n);
  reserve_group_ring(c, nmax, 1);
  const bool keep_dev = opt.ldl_device_updates != 0;
  if (keep_dev) {
    c->ring_dHRr[0].ensure(size_t(nmax) * nmax);
    c->ring_dL[0].ensure(size_t(nmax) * nmax);
  }
  std::vector<float> su(static_cast<size_t>(nmax), 0.0f);
  for (int g = 0; g < ng; ++g) {
    qtip_timing T{};
    double creg = 0.0;
    double t0 = now_s();
    rotate_hessian_impl(c, groups[g].H, groups[g].h_on_device != 0, groups[g].n, groups[g].seed, opt.sigma_reg, su.data(),
                        &creg, keep_dev ? nullptr : c->ring_HRr[0].p, keep_dev ? c->ring_dHRr[0].p : nullptr);
    T.rht = now_s() - t0;
    t0 = now_s();
    if (keep_dev)
      ldl_hessian_assisted_impl(c, nullptr, groups[g].n, opt.ldl_threads, c->ring_L[0].p, c->ring_dHRr[0].p,
                                c->ring_dL[0].p);
    else
      ldl_hessian_impl(c->ring_HRr[0].p, groups[g].n, opt.ldl_threads, c->ring_L[0].p);
    T.ldl_cpu = now_s() - t0;
    if (ldl_wait) ldl_wait[g] = T.ldl_cpu;  // all of it: the lane's GPU work waits for its own factorization
    quantize_group_impl(c, groups[g].nlin, groups[g].lins, groups[g].n, groups[g].seed, su.data(), creg,
                        keep_dev ? nullptr : c->ring_HRr[0].p, c->ring_L[0].p, opt, groups[g].outs, &T,
                        keep_dev ? c->ring_dHRr[0].p : nullptr, keep_dev ? c->ring_dL[0].p : nullptr);
    if (tms) tms[g] = T;
  }
}

long tile_rows_of(const qtip_group& g) {
  long m = 0;
  for (int i = 0; i < g.nlin; ++i) m += g.lins[i].m;
  return (m + 15) / 16;
}
}  // namespace

// Lanes.  A group keeps as many Viterbi workgroups busy as it has 16-row tile rows, and the chip holds
// `device_slots` of them (three per compute unit); the reference's schedule (one group at a time,
// src/pipeline.cpp:229-312) leaves most of the chip idle when the groups are small.  Groups do not depend on each
// other, so such groups run side by side on lanes: a lane has a context of its own (one stream, workspaces, staging)
// and takes its groups one after the other.  Every group is computed by the same code on the same inputs: same
// results whatever the number of lanes.  Automatic: as many lanes as it takes for the largest group's tile rows to
// fill the chip's slots, while the lanes' staging (2 n^2 floats each, on the host and on the device) and fp64 work
// matrices (2 n^2 floats more) stay under 32 GiB.  Lanes whose streams share a hardware queue (a process has
// GPU_MAX_HW_QUEUES of them, 4 unless the environment says more) run one after the other; measured on 1024 x 1024
// groups, 12 lanes were still the fastest choice with 4 queues (54 Mweights/s against 26 for one lane), with 8 (92)
// and with 16 (134), so the rule does not look at the queues.
int group_lanes_for(int ng, const qtip_group* groups, const qtip_opts& opt, int device_slots) {
  QTIP_REQUIRE(opt.group_lanes >= 0 && opt.group_lanes <= qtip_ctx::kMaxLanes,
               "run_groups: 1 to %d lanes (0: automatic), not %d", qtip_ctx::kMaxLanes, opt.group_lanes);
  if (ng < 2 || opt.group_lanes == 1) return 1;
  if (opt.group_lanes > 1) return std::min(opt.group_lanes, ng);
  long rows = 1, nmax = 1;
  for (int g = 0; g < ng; ++g) {
    rows = std::max(rows, tile_rows_of(groups[g]));
    nmax = std::max<long>(nmax, groups[g].n);
  }
  // rounded up: the workgroups beyond the chip's slots wait at the dispatcher and fill the slots the first lane's
  // finished workgroups leave (8192 x 4096 groups, 512 tile rows: 132 Mweights/s on one lane, 150 on two)
  const long by_slots = rows >= device_slots ? 1 : (device_slots + rows - 1) / rows;
  const long by_memory = (32L << 30) / (16 * nmax * nmax);
  const long lanes = std::min<long>({by_slots, by_memory, long(qtip_ctx::kMaxLanes), long(ng)});
  return lanes < 2 ? 1 : int(lanes);
}

void run_groups_impl(qtip_ctx* c, int ng, const qtip_group* groups, const qtip_opts& opt, qtip_timing* tms,
                     double* ldl_wait) {
  QTIP_REQUIRE(ng >= 0 && (ng == 0 || groups), "run_groups: bad arguments");
  if (ng == 0) return;
  for (int g = 0; g < ng; ++g)
    QTIP_REQUIRE(groups[g].n > 0 && groups[g].H && groups[g].nlin > 0 && groups[g].lins && groups[g].outs,
                 "run_groups: group %d is incomplete", g);
  // Mixed sizes (a layer's gate/up group beside its o-proj group): the groups that fill the chip on their own go
  // through the overlapped schedule first, in their order, the others then share the chip on lanes.
  if (opt.group_lanes == 0 && ng >= 3) {
    const long slots = viterbi_max_slots(c->device);
    std::vector<int> large, small;
    for (int g = 0; g < ng; ++g) (tile_rows_of(groups[g]) >= slots ? large : small).push_back(g);
    if (!large.empty() && small.size() >= 2) {
      for (const std::vector<int>* part : {&large, &small}) {
        std::vector<qtip_group> sub;
        for (int g : *part) sub.push_back(groups[g]);
        std::vector<qtip_timing> st(sub.size());
        std::vector<double> sw(sub.size(), 0.0);
        std::exception_ptr err;
        try {
          run_groups_impl(c, int(sub.size()), sub.data(), opt, st.data(), sw.data());
        } catch (...) {
          err = std::current_exception();
        }
        for (size_t i = 0; i < part->size(); ++i) {
          if (tms) tms[(*part)[i]] = st[i];
          if (ldl_wait) ldl_wait[(*part)[i]] = sw[i];
        }
        if (err) std::rethrow_exception(err);
      }
      return;
    }
  }
  const int lanes = group_lanes_for(ng, groups, opt, viterbi_max_slots(c->device));
  if (lanes == 1) {
    // the per-group device buffers of the quantizing thread come from the context's arena and stay there between
    // groups and calls: a hipFree waits for the whole device, the factorization's queued updates included (a dozen
    // of them per group cost 10 ms of a 2.5 s config-5 group)
    ArenaScope memory(&c->arena);
    run_groups_on(c, ng, groups, opt, tms, ldl_wait);
    return;
  }
  // group g goes to lane g % lanes; a lane's context keeps kept-metrics slots for its largest group only, and the
  // host threads of the factorizations are shared out
  struct Lane {
    qtip_ctx* c = nullptr;
    std::vector<qtip_group> groups;
    std::vector<int> index;
    std::vector<qtip_timing> tms;
    std::vector<double> wait;
    std::exception_ptr err;
    bool deferred = false;  // no thread could be started for it: its groups run on the calling thread after lane 0's
  };
  std::vector<Lane> L(static_cast<size_t>(lanes));
  qtip_opts lopt = opt;
  lopt.group_lanes = 1;
  lopt.ldlq_chains = 1;  // the other lanes are what runs under a lane's trace-backs; a chain more is a stream more
  // ldl_threads <= 0 stands for the machine's hardware concurrency (host_ldl.cpp): resolve it before the lanes share it
  const int team = opt.ldl_threads > 0 ? opt.ldl_threads : std::max(1, int(std::thread::hardware_concurrency()));
  lopt.ldl_threads = std::max(1, team / lanes);
  for (int k = 0; k < lanes; ++k) {
    Lane& l = L[size_t(k)];
    l.c = lane_context(c, k);
    long rows = 1;
    for (int g = k; g < ng; g += lanes) {
      l.groups.push_back(groups[g]);
      l.index.push_back(g);
      rows = std::max(rows, tile_rows_of(groups[g]));
    }
    l.c->vit_slots_limit = std::max<int>(l.c->vit_slots_limit, int(std::min<long>(rows, 1L << 20)));
    l.tms.resize(l.groups.size());
    l.wait.resize(l.groups.size());
    order_streams(c->stream, l.c->stream);  // inputs the caller ordered before the context's stream
  }
  auto run_lane = [&](int k) {
    Lane& l = L[size_t(k)];
    try {
      QTIP_HIP(hipSetDevice(c->device));  // this thread's own current device
      // the lane's per-group buffers come from its own arena: a hipFree would wait for every other lane's work
      ArenaScope lane_memory(&l.c->arena);
      run_groups_in_line(l.c, int(l.groups.size()), l.groups.data(), lopt, l.tms.data(), l.wait.data());
    } catch (...) {
      l.err = std::current_exception();
    }
  };
  std::vector<std::thread> th;
  for (int k = 1; k < lanes; ++k) {
    try {
      th.emplace_back(run_lane, k);
    } catch (...) {
      L[size_t(k)].deferred = true;
    }
  }
  run_lane(0);  // the calling thread takes the first lane
  for (int k = 1; k < lanes; ++k)
    if (L[size_t(k)].deferred) run_lane(k);
  for (std::thread& t : th) t.join();
  for (Lane& l : L) {
    order_streams(l.c->stream, c->stream);
    for (size_t i = 0; i < l.index.size(); ++i) {
      if (tms) tms[l.index[i]] = l.tms[i];
      if (ldl_wait) ldl_wait[l.index[i]] = l.wait[i];
    }
  }
  for (Lane& l : L)
    if (l.err) std::rethrow_exception(l.err);
}

}  // namespace qtipmi
