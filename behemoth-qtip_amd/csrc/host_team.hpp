// A small team of host threads for the fp64 block LDL: dynamic-chunk parallel loops whose idle members sleep.
//
// The factorization runs on a side thread while another thread of the process keeps the GPU queue fed.  Team members
// that have run out of work must give their core up at once (a futex wait after a few microseconds of polling):
// members that poll for long at the end of every loop, as an OpenMP runtime may, take the core the feeding thread and
// the HIP runtime's helper threads need, and the scheduler then takes it from a member that still has work.
#pragma once
#include <atomic>
#include <condition_variable>
#include <mutex>
#include <thread>
#include <vector>

#if defined(__x86_64__)
#include <immintrin.h>
#endif

namespace qtipmi {

class HostTeam {
 public:
  explicit HostTeam(int threads) : n_(threads < 1 ? 1 : threads) {
    for (int i = 1; i < n_; ++i) workers_.emplace_back([this] { worker(); });
  }
  ~HostTeam() {
    {
      std::lock_guard<std::mutex> lk(mu_);
      stop_ = true;
      epoch_.fetch_add(1, std::memory_order_release);
    }
    start_.notify_all();
    for (auto& t : workers_) t.join();
  }
  HostTeam(const HostTeam&) = delete;
  HostTeam& operator=(const HostTeam&) = delete;
  int size() const { return n_; }

  // f(i) for every i in [0, count), handed out in chunks of `chunk` consecutive indices, first come first served.
  // f must not throw.  Returns when every index is done.
  template <class F>
  void parallel_for(long count, long chunk, F&& f) {
    if (count <= 0) return;
    if (chunk < 1) chunk = 1;
    if (n_ == 1 || count <= chunk) {
      for (long i = 0; i < count; ++i) f(i);
      return;
    }
    Job job{count, chunk, [](void* ctx, long i) { (*static_cast<std::remove_reference_t<F>*>(ctx))(i); }, &f};
    {
      std::lock_guard<std::mutex> lk(mu_);
      job_ = job;
      next_.store(0, std::memory_order_relaxed);
      pending_.store(n_ - 1, std::memory_order_relaxed);
      epoch_.fetch_add(1, std::memory_order_release);
    }
    start_.notify_all();
    run(job);
    for (int spin = 0; spin < kSpin && pending_.load(std::memory_order_acquire) != 0; ++spin) relax();
    if (pending_.load(std::memory_order_acquire) != 0) {
      std::unique_lock<std::mutex> lk(mu_);
      done_.wait(lk, [&] { return pending_.load(std::memory_order_acquire) == 0; });
    }
  }

 private:
  struct Job {
    long count = 0, chunk = 1;
    void (*call)(void*, long) = nullptr;
    void* ctx = nullptr;
  };
  static constexpr int kSpin = 2000;  // polls (a few tens of microseconds) before a member goes to sleep
  static void relax() {
#if defined(__x86_64__)
    _mm_pause();
#endif
  }
  void run(const Job& j) {
    for (;;) {
      const long i0 = next_.fetch_add(j.chunk, std::memory_order_relaxed);
      if (i0 >= j.count) return;
      const long i1 = i0 + j.chunk < j.count ? i0 + j.chunk : j.count;
      for (long i = i0; i < i1; ++i) j.call(j.ctx, i);
    }
  }
  void worker() {
    unsigned long seen = 0;
    for (;;) {
      for (int spin = 0; spin < kSpin && epoch_.load(std::memory_order_acquire) == seen; ++spin) relax();
      Job j;
      {
        std::unique_lock<std::mutex> lk(mu_);
        start_.wait(lk, [&] { return epoch_.load(std::memory_order_acquire) != seen; });
        seen = epoch_.load(std::memory_order_acquire);
        if (stop_) return;
        j = job_;
      }
      run(j);
      if (pending_.fetch_sub(1, std::memory_order_acq_rel) == 1) {
        std::lock_guard<std::mutex> lk(mu_);
        done_.notify_one();
      }
    }
  }

  const int n_;
  std::vector<std::thread> workers_;
  std::mutex mu_;
  std::condition_variable start_, done_;
  std::atomic<unsigned long> epoch_{0};
  std::atomic<long> next_{0};
  std::atomic<int> pending_{0};
  Job job_;
  bool stop_ = false;
};

}  // namespace qtipmi
