// Group quantizer: Hessian rotation, host LDL, weight RHT + scaling, LDLQ driver, proxy, packing.
// Operation order, seeds and formulas follow the reference's src/quantizer.cpp:30-346 (cited per step).
#include "quantizer_impl.hpp"

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <exception>
#include <mutex>
#include <system_error>
#include <thread>
#include <vector>

namespace qtipmi {
namespace {
// Waits for the stream without spinning on a core: the host LDL of the next group runs on all cores meanwhile.
void wait_stream_sleeping(hipStream_t s) {
  hipEvent_t e;
  QTIP_HIP(hipEventCreateWithFlags(&e, hipEventBlockingSync | hipEventDisableTiming));
  hipError_t rc = hipEventRecord(e, s);
  if (rc == hipSuccess) rc = hipEventSynchronize(e);
  (void)hipEventDestroy(e);
  QTIP_HIP(rc);
}

double now_s() {
  using namespace std::chrono;
  return duration<double>(steady_clock::now().time_since_epoch()).count();
}

// Events of one call, destroyed on every way out of it.
struct Events {
  std::vector<hipEvent_t> ev;
  Events() = default;
  Events(const Events&) = delete;
  Events& operator=(const Events&) = delete;
  ~Events() {
    for (hipEvent_t e : ev) (void)hipEventDestroy(e);
  }
  hipEvent_t add(unsigned flags) {
    hipEvent_t e;
    QTIP_HIP(hipEventCreateWithFlags(&e, flags));
    ev.push_back(e);
    return e;
  }
};
}  // namespace

// ---------------------------------------------------------------- rotate_hessian, src/quantizer.cpp:124-152
void rotate_hessian_impl(qtip_ctx* c, const float* H, bool on_device, int n, uint64_t seed, double sigma_reg,
                         float* host_su, double* creg, float* host_HRr, float* dev_HRr) {
  // dev_HRr (optional): n x n device buffer of the caller in which the rotated Hessian is left; host_HRr may then be
  // null (no copy to the host)
  QTIP_REQUIRE(n > 0 && H && host_su && creg && (host_HRr || dev_HRr), "rotate_hessian: bad arguments");
  QTIP_REQUIRE(had_K(n) > 0, "unsupported hadamard dim %d", n);
  hipStream_t s = c->stream;
  SplitMix rng(seed);
  for (int i = 0; i < n; ++i) host_su[i] = rng.sign();
  DBuf<float> d_su{size_t(n)};
  QTIP_HIP(hipMemcpyAsync(d_su, host_su, size_t(n) * 4, hipMemcpyHostToDevice, s));
  DBuf<float> Ht(size_t(n) * n), HR_own(dev_HRr ? 0 : size_t(n) * n);
  float* const HR = dev_HRr ? dev_HRr : HR_own.p;
  QTIP_HIP(hipMemcpyAsync(Ht, H, size_t(n) * n * 4, on_device ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice, s));
  // regularize_H: H += sigma_reg * mean(diag(H)) * I, before the rotation
  const double dsum = c->rht.reduce(Ht, n, nullptr, 0, n, n, 3);
  *creg = sigma_reg * dsum / n;
  c->rht.add_diag(Ht, n, float(*creg));
  // HRr = hadUt(hadUt(H * su su^T)^T)
  c->rht.hadamard_rows(Ht, n, n, n, true, d_su, d_su);
  c->rht.transpose(Ht, n, n, n, HR, n);
  c->rht.hadamard_rows(HR, n, n, n, true);
  if (host_HRr) QTIP_HIP(hipMemcpyAsync(host_HRr, HR, size_t(n) * n * 4, hipMemcpyDeviceToHost, s));
  QTIP_HIP(hipStreamSynchronize(s));
}

// ---------------------------------------------------------------- ldl_hessian, src/quantizer.cpp:154-165
void ldl_hessian_impl(const float* host_HRr, int n, int threads, float* host_L) {
  QTIP_REQUIRE(n > 0 && n % 16 == 0 && host_HRr && host_L, "ldl_hessian: bad arguments (n = %d)", n);
  // n x n fp64 work matrix (6.6 GB at n = 28672): taken from a process-wide pool so that repeated groups do not
  // pay for mapping and faulting it in again
  HostScratch A(size_t(n) * n * sizeof(double));
  double* a = static_cast<double*>(A.get());
  symmetrize_lower_host(host_HRr, n, a, threads);
  if (!block_ldl_host(a, n, host_L, threads)) throw Error(QTIP_E_NOT_PD, "block LDL failed (H not PD)");
}

// ---------------------------------------------------------------- ldlq_gpu, src/quantizer.cpp:30-89
// Given L, the tile rows of a group are independent of each other (the feedback of a weight row comes from its own
// residuals only), so the tile rows are dealt to up to three chains, each with its own stream, feedback slab and share
// of the kept-metrics slots, which walk the column blocks by themselves.  The chains start a third of a tile's time
// apart and keep that distance: while the workgroups of one chain walk their trace-backs (a chain of HBM round
// trips during which they issue next to nothing), those of the other two, resident on the same compute units, run
// their forward passes.  One chain alone leaves the chip idle for the length of every trace-back.
int ldlq_default_chains(qtip_ctx* c) {
  static const int env_chains = [] {
    const char* q = getenv("GPU_MAX_HW_QUEUES");
    return q && atoi(q) >= 6 ? 3 : 2;
  }();
  if (c->default_chains == 0) c->default_chains = c->side_streams >= 3 ? 3 : env_chains;
  return c->default_chains;
}

void ldlq_impl(qtip_ctx* c, const float* WT, const float* L, long n, long m, float* hatWT, uint16_t* Q, int feedback,
               double* vit_seconds, int chains) {
  QTIP_REQUIRE(n % 128 == 0, "LDLQ needs n %% 128 == 0 (n = %ld)", n);
  QTIP_REQUIRE(chains >= 0 && chains <= qtip_ctx::kMaxChains, "LDLQ runs as 1 to %d chains (0: default), not %d", qtip_ctx::kMaxChains, chains);
  QTIP_REQUIRE(m % 16 == 0 && m > 0, "LDLQ needs m %% 16 == 0 (m = %ld)", m);
  QTIP_REQUIRE(feedback == 0 || feedback == 1, "unknown feedback mode %d", feedback);
  hipStream_t s = c->stream;
  ensure_viterbi_workspace(c);
  const long ntr = m / 16, nblk = n / 16;
  // chains: only where every chain still fills its share of the chip.  Default: three where the context found its two
  // chain streams and the LDL's stream running beside its own stream and beside each other when it was made (each on
  // a hardware queue of its own), or where the environment says the process was given six queues or more; else two.
  // Either way a default of three is on probation: the first call that runs three chains looks at its launches' own
  // time stamps and the context goes back to two for good when the first launches of the chains ran one after the
  // other.
  int nch = chains == 0 ? ldlq_default_chains(c) : chains;
  while (nch > 1 && ntr < long(nch) * (c->vit_slots / nch)) --nch;
  struct Chain {
    hipStream_t s;
    long tile0, tiles;   // tile rows tile0 .. tile0 + tiles - 1
    long r0, rows;       // weight rows (columns of WT) 16 tile0 .., 16 tiles of them
    int slot0, slots;    // share of the kept-metrics workspace
    double *prod, *parts;     // feedback 0: 128 x rows slab and the split-K partial slabs
    float *prod32, *parts32;  // feedback 1: the same in fp32
  } ch[qtip_ctx::kMaxChains];
  for (int k = 0; k < nch; ++k) {
    if (k > 0 && !c->chain_stream[k - 1]) QTIP_HIP(hipStreamCreateWithFlags(&c->chain_stream[k - 1], hipStreamNonBlocking));
    ch[k].s = k == 0 ? s : c->chain_stream[k - 1];
    ch[k].tile0 = ntr * k / nch;
    ch[k].tiles = ntr * (k + 1) / nch - ch[k].tile0;
    ch[k].r0 = 16 * ch[k].tile0;
    ch[k].rows = 16 * ch[k].tiles;
    ch[k].slot0 = c->vit_slots * k / nch;
    ch[k].slots = c->vit_slots * (k + 1) / nch - ch[k].slot0;
  }
  // The feedback of the rows quantized in earlier buffers is gathered per buffer into a 128 x rows slab per chain:
  // feedback 0 in fp64 (fp64 MFMA), feedback 1 in fp32 from bf16 hi/lo split operands (the reference GPU's arithmetic)
  const int max_splits = kMaxGatherSplits;
  DBuf<double> prod(feedback == 0 ? size_t(128) * m : 0), parts(feedback == 0 ? size_t(max_splits) * 128 * m : 0);
  DBuf<float> prod32(feedback == 1 ? size_t(128) * m : 0), parts32(feedback == 1 ? size_t(max_splits) * 128 * m : 0);
  for (int k = 0; k < nch; ++k) {
    ch[k].prod = feedback == 0 ? prod.p + size_t(128) * ch[k].r0 : nullptr;
    ch[k].parts = feedback == 0 ? parts.p + size_t(max_splits) * 128 * ch[k].r0 : nullptr;
    ch[k].prod32 = feedback == 1 ? prod32.p + size_t(128) * ch[k].r0 : nullptr;
    ch[k].parts32 = feedback == 1 ? parts32.p + size_t(max_splits) * 128 * ch[k].r0 : nullptr;
  }
  // feedback 1: the operands of the gathered product as bf16 hi / lo images with k contiguous: L transposed, made
  // here once; the residual WT - hatWT, weight row major, written by the Viterbi launches as they decode
  DBuf<uint16_t> limg(feedback == 1 ? size_t(2) * n * n : 0), dimg(feedback == 1 ? size_t(2) * m * n : 0);
  if (feedback == 1) launch_split_transpose_bf16(L, nullptr, n, n, n, limg.p, limg.p + size_t(n) * n, n, true, s);
  QTIP_HIP(hipMemsetAsync(hatWT, 0, size_t(n) * m * 4, s));
  Events timed, pacing, joins;  // timed: a (start, stop) pair per Viterbi launch, stamped by the launch itself
  // the other chains start once the caller's inputs and the cleared outputs are there, a third (two thirds) of a
  // tile's time later; a launch walks tiles / slots of them
  if (nch > 1) {
    hipEvent_t ready = joins.add(hipEventDisableTiming);
    QTIP_HIP(hipEventRecord(ready, s));
    for (int k = 1; k < nch; ++k) {
      QTIP_HIP(hipStreamWaitEvent(ch[k].s, ready, 0));
      // (tile_us: what a resident workgroup took per tile in this context's last timed call)
      const double launch_us = c->vit_tile_us * double((ch[k].tiles + ch[k].slots - 1) / ch[k].slots);
      launch_delay(launch_us * k / nch, ch[k].s);
    }
  }
  // The queue is kept kAhead buffers (a gather and a Viterbi launch of ~10 ms each) ahead of the GPU and no further: without a bound the
  // submitting thread would spin on a full queue and take a core from the host LDL of the next group; with less
  // slack a submitting thread that the scheduler holds back for a few milliseconds leaves the GPU idle.
  constexpr long kAhead = 4;
  hipEvent_t pace[qtip_ctx::kMaxChains][kAhead + 1];
  for (int k = 0; k < nch; ++k)
    for (auto& e : pace[k]) e = pacing.add(hipEventBlockingSync | hipEventDisableTiming);
  try {
    long nbuf_done = 0;
    for (long cur = nblk; cur > 0; cur -= 8, ++nbuf_done) {
      const int bufend = int(16 * cur), c0 = bufend - 128;
      for (int k = 0; k < nch; ++k) {
        const Chain& C = ch[k];
        if (nbuf_done >= kAhead) QTIP_HIP(hipEventSynchronize(pace[k][(nbuf_done - kAhead) % (kAhead + 1)]));
        // prod[r][:] = sum_{k >= bufend} L[k][c0 + r] (WT - hatWT)[k][:], r < 128
        const float* Lp = L + long(bufend) * n + c0;
        const float *Wp = WT + long(bufend) * m + C.r0, *Hp = hatWT + long(bufend) * m + C.r0;
        // (the split-K partial slabs are summed by the Viterbi launch as it forms its targets, in the order the
        // product's own reduction kernel would add them)
        int splits = 1;
        if (bufend == n) {
          if (feedback == 0) QTIP_HIP(hipMemsetAsync(C.prod, 0, size_t(128) * C.rows * sizeof(double), C.s));
          else QTIP_HIP(hipMemsetAsync(C.prod32, 0, size_t(128) * C.rows * sizeof(float), C.s));
        } else if (feedback == 0) {
          splits = launch_gemm_tn_f64_gather(int(C.rows), n - bufend, Lp, n, Wp, Hp, m, C.prod, C.parts, C.slots, C.s, false);
        } else {
          const uint16_t* la = limg.p + size_t(c0) * n + bufend;
          const uint16_t* da = dimg.p + size_t(C.r0) * n + bufend;
          splits = launch_gemm_img_gather(int(C.rows), n - bufend, la, la + size_t(n) * n, n, da, da + size_t(m) * n, n,
                                          C.prod32, C.parts32, C.slots, C.s, false);
        }
        {
          // one launch per buffer: a workgroup takes its tile row through the 8 column blocks, last to first, and
          // forms each block's targets (in-buffer feedback) itself; no workgroup waits for another between blocks
          TileJob job;
          job.tiles = C.tiles;
          job.WT = WT + C.r0;
          job.L = L;
          job.ldl = n;
          job.bufend = bufend;
          if (feedback == 0) job.prod64 = splits > 1 ? C.parts : C.prod;
          else job.prod32 = splits > 1 ? C.parts32 : C.prod32;
          job.prod_row0 = c0, job.ldp = C.rows;
          job.prod_splits = splits, job.prod_split_stride = long(128) * C.rows;
          job.states = Q + size_t(C.tile0) * nblk * 128;
          job.q_tile_stride = nblk;
          job.q_offset = c0 / 16;
          job.hatWT = hatWT + C.r0;
          job.ldw = m;
          if (feedback == 1) job.dimg_h = dimg.p + size_t(C.r0) * n, job.dimg_l = job.dimg_h + size_t(m) * n, job.ldd = n;
          job.col0 = c0;
          job.blocks = 8;
          c->viterbi_settings(job);
          if (nch > 1) job.wide = 0;  // the chains fill the chip between them: one launch is not the measure
          hipEvent_t t0 = nullptr, t1 = nullptr;
          if (vit_seconds) t0 = timed.add(hipEventDefault), t1 = timed.add(hipEventDefault);
          launch_viterbi_tiles(job, c->d_entry_d, c->d_entry_f, c->vit_ws.p + viterbi_workspace_bytes(C.slot0), C.slots,
                               C.s, t0, t1);
        }
        QTIP_HIP(hipEventRecord(pace[k][nbuf_done % (kAhead + 1)], C.s));
      }
    }
    // the caller's stream continues when every chain is through
    for (int k = 1; k < nch; ++k) {
      hipEvent_t done = joins.add(hipEventDisableTiming);
      QTIP_HIP(hipEventRecord(done, ch[k].s));
      QTIP_HIP(hipStreamWaitEvent(s, done, 0));
    }
  } catch (...) {
    // nothing queued on a chain may outlive the buffers of this call
    for (int k = 0; k < nch; ++k) (void)hipStreamSynchronize(ch[k].s);
    throw;
  }
  wait_stream_sleeping(s);
  if (vit_seconds) {
    // the chains' launches overlap: the time the column blocks take is the launches' total over the chains
    double t = 0;
    for (size_t i = 0; i + 1 < timed.ev.size(); i += 2) {
      float ms = 0;
      QTIP_HIP(hipEventElapsedTime(&ms, timed.ev[i], timed.ev[i + 1]));
      t += ms * 1e-3;
    }
    *vit_seconds = t / nch;
    // per tile and resident workgroup: a launch takes its tile rows through 8 column blocks, tiles / slots rounds of them
    const size_t launches = timed.ev.size() / 2;
    if (launches > 0) {
      const double rounds = double((ch[0].tiles + ch[0].slots - 1) / ch[0].slots);
      const double tile_us = t / double(launches) / (8.0 * rounds) * 1e6;
      if (tile_us > 50.0 && tile_us < 20000.0) c->vit_tile_us = tile_us;
    }
    // three chains by default, on probation: did the first launches of the chains run side by side?  (One pair of
    // events per launch, in the order chain 0, 1, 2 of the first buffer.)
    if (chains == 0 && nch == 3 && !c->chains_checked && timed.ev.size() >= 6) {
      c->chains_checked = true;
      float first_ms = 0, start1 = 0, start2 = 0;
      QTIP_HIP(hipEventElapsedTime(&first_ms, timed.ev[0], timed.ev[1]));
      QTIP_HIP(hipEventElapsedTime(&start1, timed.ev[0], timed.ev[2]));
      QTIP_HIP(hipEventElapsedTime(&start2, timed.ev[0], timed.ev[4]));
      if (start1 >= first_ms || start2 >= first_ms) c->default_chains = 2;  // a chain waited for another's launch to end
    }
  }
}

// ---------------------------------------------------------------- quantize_group, src/quantizer.cpp:176-346
// In three phases: prepare (weights -> rotated, scaled Wr^T, Wscale), LDLQ + Viterbi, finish (proxy errors, packing,
// optional reconstruction); each is synchronous on return.  (A scheduler that ran the first and the last phase of
// neighbouring groups on a second context beside a group's LDLQ was built on this split and measured: the proxy's
// matrix-core kernel, 256 accumulators and 64 KB of LDS per workgroup, takes the place of two Viterbi workgroups
// wherever it gets in and takes 1.39 s instead of 0.067 s; with only the rotation and the weight transform run ahead
// those take 0.99 s instead of 0.02 s.  210.8 and 212.0 Mweights/s against 215-217 with the phases one after the
// other on one stream: the chip has no idle capacity beside the Viterbi launches.)
void group_prepare(qtip_ctx* c, GroupWork& w, int nlin, const qtip_linear_in* lins, int n, uint64_t seed,
                   const float* host_su, const qtip_opts& opt, qtip_linear_out* outs, const qtip_timing* tm) {
  QTIP_REQUIRE(nlin > 0 && lins && outs && host_su, "quantize_group: bad arguments");
  QTIP_REQUIRE(n % 128 == 0, "LDLQ needs n %% 128 == 0 (n = %d)", n);
  QTIP_REQUIRE(had_K(n) > 0 && n / had_K(n) <= 8192, "unsupported hadamard dim %d", n);
  hipStream_t s = c->stream;
  qtip_timing& T = w.T;
  T = qtip_timing{};
  if (tm) T.rht = tm->rht, T.ldl_cpu = tm->ldl_cpu;
  w.t_start = now_s();
  w.carried = (tm ? tm->rht : 0.0);
  double t0 = w.t_start;
  long mt = 0, maxm = 0;
  w.off.clear();
  for (int li = 0; li < nlin; ++li) {
    const qtip_linear_in& l = lins[li];
    QTIP_REQUIRE(l.m > 0 && l.m % 32 == 0 && n % 32 == 0, "kernel layout needs m, n multiples of 32 (m=%d n=%d)", l.m, n);
    QTIP_REQUIRE(had_K(l.m) > 0 && l.m / had_K(l.m) <= 8192, "unsupported hadamard dim %d", l.m);
    QTIP_REQUIRE((l.w_f32 != nullptr) + (l.w_bf16 != nullptr) + (l.w_fp8 != nullptr) == 1,
                 "linear %d: exactly one of w_f32 / w_bf16 / w_fp8 must be set", li);
    QTIP_REQUIRE(outs[li].trellis && outs[li].su_bf16 && outs[li].sv, "linear %d: output buffers missing", li);
    w.off.push_back(mt);
    mt += l.m;
    maxm = std::max<long>(maxm, l.m);
  }
  w.mt = mt;
  const std::vector<long>& off = w.off;
  w.d_su.alloc(size_t(n));
  w.d_sv.alloc(size_t(mt));
  DBuf<float>&d_su = w.d_su, &d_sv = w.d_sv;
  QTIP_HIP(hipMemcpyAsync(d_su, host_su, size_t(n) * 4, hipMemcpyHostToDevice, s));

  // ---- weights -> Wr^T (n x mt), each linear's column block scaled by 1/Wscale (src/quantizer.cpp:195-249)
  w.WT.alloc(size_t(n) * mt);
  DBuf<float>& WT = w.WT;
  {
    DBuf<float> Wt(size_t(maxm) * n);
    DBuf<uint8_t> raw;
    DBuf<uint16_t> sc;
    for (int li = 0; li < nlin; ++li) {
      const qtip_linear_in& l = lins[li];
      qtip_linear_out& O = outs[li];
      const long m = l.m;
      SplitMix r2(seed * 1000003ull + uint64_t(li) + 1);
      for (long i = 0; i < m; ++i) O.sv[i] = r2.sign();
      for (int i = 0; i < n; ++i) O.su_bf16[i] = f32_to_bf16(host_su[i]);
      QTIP_HIP(hipMemcpyAsync(d_sv + off[li], O.sv, size_t(m) * 4, hipMemcpyHostToDevice, s));
      const hipMemcpyKind kind = l.on_device ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice;
      if (l.w_fp8) {
        raw.ensure(size_t(m) * n);
        QTIP_HIP(hipMemcpyAsync(raw, l.w_fp8, size_t(m) * n, kind, s));
        if (l.scale_bf16) {
          sc.ensure(size_t(m));
          QTIP_HIP(hipMemcpyAsync(sc, l.scale_bf16, size_t(m) * 2, kind, s));
        }
        launch_fp8_to_f32(raw, l.scale_bf16 ? sc.p : nullptr, Wt, m, n, s);
      } else if (l.w_bf16) {
        raw.ensure(size_t(m) * n * 2);
        QTIP_HIP(hipMemcpyAsync(raw, l.w_bf16, size_t(m) * n * 2, kind, s));
        launch_bf16_to_f32(reinterpret_cast<const uint16_t*>(raw.p), Wt, m * n, s);
      } else {
        QTIP_HIP(hipMemcpyAsync(Wt, l.w_f32, size_t(m) * n * 4, kind, s));
      }
      QTIP_HIP(hipStreamSynchronize(s));
      T.load += now_s() - t0;
      t0 = now_s();
      // Wr^T = hadUt_m( hadUt_n( diag(SV) W diag(SU) )^T )
      c->rht.hadamard_rows(Wt, m, n, n, true, d_sv + off[li], d_su);
      c->rht.transpose(Wt, m, n, n, WT + off[li], mt);
      c->rht.hadamard_rows(WT + off[li], n, int(m), mt, true);
      const double ss = c->rht.reduce(WT + off[li], mt, nullptr, 0, n, m, 0);
      const double rms = std::sqrt(ss / (double(n) * double(m)));
      O.wscale = float(rms / (double(float(c->cb.lut_rms)) * opt.scale_override));
      c->rht.scale(WT + off[li], n, m, mt, 1.0f / O.wscale);
      QTIP_HIP(hipStreamSynchronize(s));
      T.rht += now_s() - t0;
      t0 = now_s();
    }
  }
}

void group_ldlq(qtip_ctx* c, GroupWork& w, int n, const float* host_L, const float* dev_L, const qtip_opts& opt) {
  QTIP_REQUIRE(host_L || dev_L, "quantize_group: no factor");
  hipStream_t s = c->stream;
  qtip_timing& T = w.T;
  const long mt = w.mt;
  double t0 = now_s();
  // the factor: the caller's device copy if it kept one, else uploaded
  DBuf<float> Ld(dev_L ? 0 : size_t(n) * n);
  if (!dev_L) QTIP_HIP(hipMemcpyAsync(Ld, host_L, size_t(n) * n * 4, hipMemcpyHostToDevice, s));
  QTIP_HIP(hipStreamSynchronize(s));
  T.load += now_s() - t0;
  t0 = now_s();
  w.hatWT.alloc(size_t(n) * mt);
  w.Q.alloc(size_t(mt / 16) * (n / 16) * 128);
  double vit = 0;
  ldlq_impl(c, w.WT, dev_L ? dev_L : Ld.p, n, mt, w.hatWT, w.Q, opt.feedback, &vit, opt.ldlq_chains);
  T.ldlq += now_s() - t0;
  T.viterbi += vit;
}

void group_finish(qtip_ctx* c, GroupWork& w, int nlin, const qtip_linear_in* lins, int n, double creg,
                  const float* host_HRr, const float* dev_HRr, const qtip_opts& opt, qtip_linear_out* outs,
                  qtip_timing* tm) {
  QTIP_REQUIRE(opt.skip_proxy || host_HRr || dev_HRr, "quantize_group: HRr is needed for the proxy");
  hipStream_t s = c->stream;
  qtip_timing& T = w.T;
  const long mt = w.mt;
  const std::vector<long>& off = w.off;
  DBuf<float>&WT = w.WT, &hatWT = w.hatWT, &d_su = w.d_su, &d_sv = w.d_sv;
  DBuf<uint16_t>& Q = w.Q;
  double t0 = now_s();
  // ---- states -> packed trellis in kernel layout, src/quantizer.cpp:305-320 (packed on the device).  The packing
  // kernel is small and the copy to the caller's (pageable) memory is the copy engines' and a host thread's work:
  // where a chain's stream exists (idle now: LDLQ has been waited for) both run there, from a helper thread, beside
  // the proxy's matrix-core kernels instead of after them.
  const long nblk = n / 16;
  DBuf<uint16_t> tr(size_t(mt / 16) * nblk * 32);
  auto pack_to_host = [&](hipStream_t st) {
    for (int li = 0; li < nlin; ++li) {
      const long m = lins[li].m;
      const size_t tile0 = size_t(off[li] / 16) * nblk;
      launch_pack_swizzle(Q + tile0 * 128, m, n, tr + tile0 * 32, st);
      QTIP_HIP(hipMemcpyAsync(outs[li].trellis, tr + tile0 * 32, size_t(m / 16) * nblk * 32 * 2, hipMemcpyDeviceToHost, st));
    }
    QTIP_HIP(hipStreamSynchronize(st));
  };
  struct Packer {  // joined whatever ends this scope
    std::thread t;
    std::exception_ptr err;
    ~Packer() {
      if (t.joinable()) t.join();
    }
  } packer;
  // (not on a lane: the lanes' own streams already share the hardware queues, and one more stream per lane makes
  // lanes wait for each other)
  bool pack_beside = !opt.skip_proxy && c->chain_stream[0] != nullptr && c->vit_slots_limit == 0;
  if (pack_beside) {
    try {
      packer.t = std::thread([&] {
        try {
          QTIP_HIP(hipSetDevice(c->device));  // this thread's own current device
          pack_to_host(c->chain_stream[0]);
        } catch (...) {
          packer.err = std::current_exception();
        }
      });
    } catch (const std::system_error&) {
      pack_beside = false;  // no thread to be had: after the proxy, on this one
    }
  }
  // ---- proxy (rotated, scaled domain; Wscale cancels), src/quantizer.cpp:268-303
  if (!opt.skip_proxy) {
    // the rotated Hessian: the caller's device copy if it kept one, else uploaded
    DBuf<float> HR_own(dev_HRr ? 0 : size_t(n) * n);
    if (!dev_HRr) QTIP_HIP(hipMemcpyAsync(HR_own, host_HRr, HR_own.bytes(), hipMemcpyHostToDevice, s));
    const float* const HR = dev_HRr ? dev_HRr : HR_own.p;
    DBuf<uint16_t> stack;
    for (int li = 0; li < nlin; ++li) {
      const long m = lins[li].m;
      const double den = quad_trace_bf16x3(n, m, HR, WT + off[li], nullptr, mt, stack, c->scratch, s);
      const double num = quad_trace_bf16x3(n, m, HR, WT + off[li], hatWT + off[li], mt, stack, c->scratch, s);
      const double wn2 = c->rht.reduce(WT + off[li], mt, nullptr, 0, n, m, 0);
      const double dn2 = c->rht.reduce(WT + off[li], mt, hatWT + off[li], mt, n, m, 2);
      outs[li].proxy_rot_reg = num / den;
      outs[li].proxy = (num - creg * dn2) / (den - creg * wn2);
    }
  } else {
    for (int li = 0; li < nlin; ++li) outs[li].proxy = outs[li].proxy_rot_reg = 0;
  }
  QTIP_HIP(hipStreamSynchronize(s));
  T.proxy += now_s() - t0;
  t0 = now_s();

  if (pack_beside) {
    packer.t.join();
    if (packer.err) std::rethrow_exception(packer.err);
  } else {
    pack_to_host(s);
  }
  // ---- optional reconstruction in the original domain, src/quantizer.cpp:321-338:
  //      hatW = diag(SV) U_m (hatWr * Wscale) U_n^T diag(SU)
  for (int li = 0; li < nlin; ++li) {
    if (!outs[li].hatW) continue;
    const long m = lins[li].m;
    DBuf<float> a(size_t(n) * m), b(size_t(m) * n);
    QTIP_HIP(hipMemcpy2DAsync(a, size_t(m) * 4, hatWT + off[li], size_t(mt) * 4, size_t(m) * 4, size_t(n),
                              hipMemcpyDeviceToDevice, s));
    c->rht.hadamard_rows(a, n, int(m), m, false);
    c->rht.transpose(a, n, m, m, b, n);
    c->rht.hadamard_rows(b, m, n, n, false);
    c->rht.scale(b, m, n, n, outs[li].wscale);
    launch_scale_rc(b, m, n, n, d_sv + off[li], d_su, s);
    QTIP_HIP(hipMemcpyAsync(outs[li].hatW, b, size_t(m) * n * 4, hipMemcpyDeviceToHost, s));
    QTIP_HIP(hipStreamSynchronize(s));
  }
  T.pack += now_s() - t0;
  T.total = (now_s() - w.t_start) + w.carried + T.ldl_cpu;
  double wsum = 0;
  for (int li = 0; li < nlin; ++li) wsum += double(lins[li].m) * n;
  for (int li = 0; li < nlin; ++li) outs[li].seconds = T.total * double(lins[li].m) * n / wsum;
  if (tm) *tm = T;
  w.release();
}

void quantize_group_impl(qtip_ctx* c, int nlin, const qtip_linear_in* lins, int n, uint64_t seed, const float* host_su,
                         double creg, const float* host_HRr, const float* host_L, const qtip_opts& opt,
                         qtip_linear_out* outs, qtip_timing* tm, const float* dev_HRr, const float* dev_L) {
  QTIP_REQUIRE(host_L != nullptr, "quantize_group: bad arguments");
  QTIP_REQUIRE(opt.skip_proxy || host_HRr || dev_HRr, "quantize_group: HRr is needed for the proxy");
  GroupWork w;
  group_prepare(c, w, nlin, lins, n, seed, host_su, opt, outs, tm);
  group_ldlq(c, w, n, host_L, dev_L, opt);
  group_finish(c, w, nlin, lins, n, creg, host_HRr, dev_HRr, opt, outs, tm);
}

}  // namespace qtipmi
