// Several Hessian groups through one context, scheduled like the reference's run_qtip_groups
// (src/pipeline.cpp:229-312): Hessians are rotated on the GPU ahead of use, a side thread runs the host fp64 LDL of
// the groups in order, and the calling thread quantizes group g as soon as its factor is there, so the LDL of group
// g+1 overlaps the GPU work of group g.  The reference rotates all Hessians of a layer up front and keeps every HRr;
// here rotation runs two groups ahead through a ring of three page-locked (HRr, L) pairs kept by the context, so
// host memory stays at 6 n^2 floats however many groups are queued.
#include <chrono>
#include <condition_variable>
#include <cstring>
#include <exception>
#include <mutex>
#include <thread>

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

void run_groups_impl(qtip_ctx* c, int ng, const qtip_group* groups, const qtip_opts& opt, qtip_timing* tms,
                     double* ldl_wait) {
  QTIP_REQUIRE(ng >= 0 && (ng == 0 || groups), "run_groups: bad arguments");
  if (ng == 0) return;
  int nmax = 0;
  for (int g = 0; g < ng; ++g) {
    QTIP_REQUIRE(groups[g].n > 0 && groups[g].H && groups[g].nlin > 0 && groups[g].lins && groups[g].outs,
                 "run_groups: group %d is incomplete", g);
    nmax = std::max(nmax, groups[g].n);
  }
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
  int rotated = 0, factored = 0;
  bool stop = false;
  std::exception_ptr ldl_err;

  auto rotate = [&](int g) {
    const double t0 = now_s();
    const int b = g % R;
    rotate_hessian_impl(c, groups[g].H, groups[g].h_on_device != 0, groups[g].n, groups[g].seed, opt.sigma_reg,
                        su[size_t(b)].data(), &creg[size_t(g)], keep_dev ? nullptr : c->ring_HRr[b].p,
                        keep_dev ? c->ring_dHRr[b].p : nullptr);
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
        quantize_group_impl(c, groups[g].nlin, groups[g].lins, groups[g].n, groups[g].seed, su[size_t(b)].data(),
                            creg[size_t(g)], keep_dev ? nullptr : c->ring_HRr[b].p, c->ring_L[b].p, opt, groups[g].outs, &T,
                            keep_dev ? c->ring_dHRr[b].p : nullptr, keep_dev ? c->ring_dL[b].p : nullptr);
        if (tms) tms[g] = T;
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

}  // namespace qtipmi
