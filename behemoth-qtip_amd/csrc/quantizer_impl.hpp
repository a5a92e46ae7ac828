// The context behind the C ABI and the group-quantizer entry points implemented in quantizer_impl.cpp.
#pragma once
#include "ldlq.hpp"
#include "misc.hpp"
#include "qtip_internal.hpp"
#include "rht.hpp"

struct qtip_ctx {
  // first member, so that it outlives every buffer below: a lane's per-group device buffers come from here
  qtipmi::DeviceArena arena;
  int device = 0;
  hipStream_t stream = nullptr;
  qtipmi::HostCodebook cb;
  qtipmi::DBuf<double> d_entry_d;  // [1024][2] decoded codebook entries, fp64
  qtipmi::DBuf<float> d_entry_f;   // [1024][2] the same as fp32
  qtipmi::DBuf<uint32_t> d_lut_h2; // [65536] fp16 pairs per state, built when a caller asks for it
  bool lut_h2_valid = false;
  qtipmi::DBuf<unsigned char> vit_ws;  // kept-metrics slots of the resident Viterbi workgroups
  int vit_slots = 0;
  // Viterbi passes: 0 = 32-bit metrics first, fp64 again where a traced decision is too close (same results);
  // 1 = fp64 only.  vit_stats: two device counters, passes of the first / second kind that were run again.
  int vit_mode = 0;
  int vit_wide = -1;  // TileJob::wide; a lane runs beside other lanes and keeps to the 256-thread workgroups
  uint32_t vit_margin = qtipmi::kViterbiMargin;
  qtipmi::DBuf<unsigned> vit_stats;
  void viterbi_settings(qtipmi::TileJob& job) const {
    job.mode = vit_mode;
    job.wide = vit_slots_limit > 0 ? 0 : vit_wide;
    job.margin = vit_margin;
    job.stats = vit_stats.p;
  }
  int vit_slots_limit = 0;  // a lane (below) keeps slots for this many workgroups only; 0: all the device can hold
  // qtip_run_groups runs groups too small to fill the chip side by side, each on a lane: a context of its own
  // (streams, workspaces, rings) made on first use, kept here and released with this context
  static constexpr int kMaxLanes = 12;
  qtip_ctx* lane[kMaxLanes] = {};
  bool lane_streams_exhausted = false;  // a lane found no stream that runs beside the earlier lanes': no search for the later ones

  // LDLQ runs its tile rows as up to kMaxChains independent chains of launches, on the context's stream and these,
  // so that one chain's trace-backs and gathers run under the others' forward passes
  static constexpr int kMaxChains = 3;
  hipStream_t chain_stream[kMaxChains - 1] = {};
  int default_chains = 0;       // 0: not decided yet (side_streams or the environment's queue count decides, then the first call checks)
  int side_streams = 0;         // how many of chain_stream[0], chain_stream[1], ldl_stream (in this order) were found
                                // to run beside the context's stream and beside each other when the context was made
  bool chains_checked = false;
  double vit_tile_us = 800.0;   // a resident Viterbi workgroup's time per tile, from the last timed LDLQ call
  qtipmi::Rht rht;
  qtipmi::DBuf<double> scratch;
  qtipmi::DBuf<uint16_t> hess_img;  // a batch of qtip_hessian_accumulate_dev as the stage images of its update kernel
  qtipmi::HBuf<float> ring_HRr[3], ring_L[3];  // page-locked staging of run_groups, kept between calls
  // host inputs of qtip_run_groups on their way to the device: a stream and four staging slots (Hessian, weights)
  static constexpr int kUploadSlots = 4;
  hipStream_t upload_stream = nullptr;
  qtipmi::DBuf<float> up_H[kUploadSlots];
  qtipmi::DBuf<uint8_t> up_W[kUploadSlots];
  qtipmi::DBuf<float> ring_dHRr[3], ring_dL[3];  // run_groups with device-updated LDL: rotated Hessians and factors stay here
  // LDL with the trailing updates on the device (ldl_assist.hip): own stream, fp64 work matrix, fp32 upload of HRr,
  // solved panel rows, two page-locked panel buffers (the panels travel one ahead); allocated on first use
  hipStream_t ldl_stream = nullptr;
  qtipmi::DBuf<double> ldl_A, ldl_X, ldl_Xt, ldl_P;
  qtipmi::DBuf<float> ldl_H;
  qtipmi::HBuf<double> ldl_panel[2];
};

namespace qtipmi {
void ensure_viterbi_workspace(qtip_ctx* c);
void rotate_hessian_impl(qtip_ctx* c, const float* H, bool on_device, int n, uint64_t seed, double sigma_reg,
                         float* host_su, double* creg, float* host_HRr, float* dev_HRr = nullptr);
void ldl_hessian_impl(const float* host_HRr, int n, int threads, float* host_L);
void ldl_hessian_assisted_impl(qtip_ctx* c, const float* host_HRr, int n, int threads, float* host_L,
                               const float* dev_HRr = nullptr, float* dev_L = nullptr);
void nvfp4_prepare_assisted_impl(qtip_ctx* c, const float* host_H, int n, double sigma_reg, int threads, float* host_L,
                                 float* host_dw);
void ldlq_impl(qtip_ctx* c, const float* dWT, const float* dL, long n, long m, float* d_hatWT, uint16_t* dQ,
               int feedback, double* vit_seconds, int chains);
int ldlq_default_chains(qtip_ctx* c);  // what chains = 0 stands for in this context (decided on the first call)
// what a group carries from one phase of its quantization to the next (device buffers, offsets of its linears, times)
struct GroupWork {
  long mt = 0;
  std::vector<long> off;
  DBuf<float> d_su, d_sv, WT, hatWT;
  DBuf<uint16_t> Q;
  qtip_timing T{};
  double t_start = 0, carried = 0;
  void release() {
    d_su.release(), d_sv.release(), WT.release(), hatWT.release(), Q.release();
  }
};
void group_prepare(qtip_ctx* c, GroupWork& w, int nlin, const qtip_linear_in* lins, int n, uint64_t seed,
                   const float* host_su, const qtip_opts& opt, qtip_linear_out* outs, const qtip_timing* tm);
void group_ldlq(qtip_ctx* c, GroupWork& w, int n, const float* host_L, const float* dev_L, const qtip_opts& opt);
void group_finish(qtip_ctx* c, GroupWork& w, int nlin, const qtip_linear_in* lins, int n, double creg,
                  const float* host_HRr, const float* dev_HRr, const qtip_opts& opt, qtip_linear_out* outs,
                  qtip_timing* tm);
void quantize_group_impl(qtip_ctx* c, int nlin, const qtip_linear_in* lins, int n, uint64_t seed, const float* host_su,
                         double creg, const float* host_HRr, const float* host_L, const qtip_opts& opt,
                         qtip_linear_out* outs, qtip_timing* tm, const float* dev_HRr = nullptr,
                         const float* dev_L = nullptr);
void reserve_group_ring(qtip_ctx* c, int n, int depth);
// lane k of a context (made on first use with the parent's codebook), and the release of all of them
qtip_ctx* lane_context(qtip_ctx* parent, int k);
void release_lanes(qtip_ctx* parent);
// stream `then` waits for everything queued on `first` so far
void order_streams(hipStream_t first, hipStream_t then);
// how many groups qtip_run_groups runs side by side (1: one after the other on the context itself)
int group_lanes_for(int ngroups, const qtip_group* groups, const qtip_opts& opt, int device_slots);
void run_groups_impl(qtip_ctx* c, int ngroups, const qtip_group* groups, const qtip_opts& opt, qtip_timing* timings,
                     double* ldl_wait);
uint8_t f32_to_fp8e4m3(float x);
void nvfp4_quantize_host(const float* w, int m, int n, uint8_t* packed, uint8_t* scales, float* global);
void nvfp4_dequantize_host(const uint8_t* packed, const uint8_t* scales, float global, int m, int n, float* out);
double nvfp4_proxy_error_host(const float* w, const float* what, int m, int n, const float* H);
void nvfp4_prepare_host(const float* H, int n, double sigma_reg, bool calibrate, int threads, float* L, float* dw);
void nvfp4_quantize_prepared_impl(qtip_ctx* c, int nmat, const qtip_nvfp4_matrix* mats, int n, const float* host_L,
                                  const float* host_dw, bool search);
}  // namespace qtipmi
