/* C ABI of the MI355X (gfx950) QTIP group quantizer: libqtip_mi355.so.
 *
 * Plain pointers and sizes only.  Every call returns 0 on success or a negative QTIP_E_* code;
 * qtip_last_error() returns the message of the calling thread's last failure.  Nothing here aborts
 * the process; the C++ shim (behemoth-qtip_amd/csrc/quantizer.hpp) that mirrors the reference's
 * C++ API restores its abort-on-error behaviour on top of these calls.
 *
 * Each entry point names the reference interface it replaces (paths relative to the reference root).
 * Pointers named host_* are host memory, dev_* device memory of the context's device.
 */
#ifndef QTIP_MI355_H_
#define QTIP_MI355_H_
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  QTIP_OK = 0,
  QTIP_E_ARG = -1,     /* bad argument / unsupported shape (the reference's QCHECK preconditions) */
  QTIP_E_HIP = -2,     /* a HIP runtime call failed */
  QTIP_E_NOT_PD = -3,  /* block LDL failed: Hessian not positive definite or not finite */
  QTIP_E_NOMEM = -4
};

typedef struct qtip_ctx qtip_ctx;

/* One context per worker thread and device (the reference's worker does hipSetDevice + a private
 * non-blocking stream + device_lut(), src/pipeline.cpp:237-238,806-812, src/quantizer.cpp:14-28).
 * The context owns its stream, the codebook tables on the device and reusable workspaces. */
int qtip_create(int device, qtip_ctx** out);
void qtip_destroy(qtip_ctx* ctx);
const char* qtip_last_error(void);
/* hipStream_t of the context, as an opaque pointer */
void* qtip_stream(qtip_ctx* ctx);
int qtip_synchronize(qtip_ctx* ctx);

/* The reference's entry points take the caller's hipStream_t and queue their work on it (src/quantizer.hpp:60-78);
 * this library works on the context's own stream.  These two calls carry the ordering across: after
 * qtip_stream_wait the context's stream starts nothing before everything queued on caller_stream so far is done
 * (call it before an entry point that reads device memory the caller produced asynchronously); after
 * qtip_stream_signal the caller's stream starts nothing before the context's work queued so far is done (call it
 * after an asynchronous *_dev entry point whose results the caller's stream will read).  caller_stream: a
 * hipStream_t as an opaque pointer, NULL for the null stream.  Neither call blocks the host. */
int qtip_stream_wait(qtip_ctx* ctx, void* caller_stream);
int qtip_stream_signal(qtip_ctx* ctx, void* caller_stream);

/* Codebook (replaces the hard-wired codebook(), src/qtip_core.cpp:18-50, and device_lut(),
 * src/quantizer.cpp:14-28).  tlut: 512 x 2 fp32, NULL selects the built-in HYB table.  The table is
 * rounded to fp16 (RNE) and expanded by quantlut_sym as the reference does. */
int qtip_set_tlut(qtip_ctx* ctx, const float* host_tlut);
double qtip_lut_rms(qtip_ctx* ctx);
/* decoded 65536-entry LUT (fp16 values as fp32), either pointer may be NULL */
int qtip_get_lut(qtip_ctx* ctx, float* host_lut0, float* host_lut1);

/* device_lut(), src/quantizer.cpp:14-28: the decoded 65536-entry table on the context's device as the reference's
 * kernels read it, one word per state, fp16 bits of component 0 in the low half and of component 1 in the high half
 * (Codebook::lut_h2, src/qtip_core.cpp:41).  Built on first use and after every qtip_set_tlut; owned by the context,
 * valid until the next qtip_set_tlut or qtip_destroy. */
int qtip_device_lut(qtip_ctx* ctx, const uint32_t** dev_lut_h2);

/* Two-pass tail-biting Viterbi of B independent 256-value sequences (replaces the launch chain
 * k_viterbi_fwd(roll) -> k_viterbi_overlap -> k_viterbi_fwd(overlap) -> k_viterbi_finish of
 * tests/test_gpu.cpp:67-88 / src/quantizer.cpp:57-62; result equals quantize_seq_ref,
 * src/qtip_core.cpp:180-191, bit for bit: fp64 path metrics, no input rounding).
 * X: B x 256 fp32 in sequence order.  states: B x 128 u16 and/or packed: B x 32 u16 (pack_trellis
 * layout, src/qtip_core.cpp:194-208); either may be NULL. */
int qtip_viterbi_tiles(qtip_ctx* ctx, const float* host_X, long B, uint16_t* host_states, uint16_t* host_packed);
/* Same with device pointers; asynchronous on the context's stream. */
int qtip_viterbi_tiles_dev(qtip_ctx* ctx, const float* dev_X, long B, uint16_t* dev_states, uint16_t* dev_packed);

/* qtip_viterbi_tiles_dev without any allocation.  No counterpart in the reference (its launch chain allocates its
 * back-pointer buffer per call, src/quantizer.cpp:38); it is for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  The kept-metrics workspace, which
 * qtip_viterbi_tiles_dev allocates on its first call (2 MiB per resident workgroup, 768 of them), is here a fixed
 * array inside the library's code object: 32 slots, 63 MiB per device, held until the process ends; its address is
 * looked up once per device in qtip_create.  B <= QTIP_NOALLOC_MAX_TILES, else QTIP_E_ARG; 32 tiles run at a time.
 * Results equal qtip_viterbi_tiles_dev's bit for bit.  Asynchronous on the context's stream.  All calls on one device
 * share the array: calls that overlap on one device (two contexts, two streams) race.  Nothing in it needs clearing
 * between calls: a workgroup writes every kept metric before it reads it. */
#define QTIP_NOALLOC_MAX_TILES 4096
int qtip_viterbi_tiles_dev_noalloc(qtip_ctx* ctx, const float* dev_X, long B, uint16_t* dev_states,
                                   uint16_t* dev_packed);

/* How the Viterbi passes of this context (tile calls, LDLQ, groups) keep their path metrics.  No counterpart in the
 * reference, whose device kernel scores in fp32 with the predecessor tag in the low mantissa bits and is exact most of
 * the time only (src/viterbi.hip:106-140).
 * mode 0 (default): each pass runs on unsigned 32-bit metrics first (squared errors formed in fp64 as the CPU
 * algorithm forms them, src/qtip_core.cpp:123-127, rounded once to units of 2^-26, or of the power of two that
 * fits the tile's winner; saturating integer adds, values held to 2^32 - 1), and its trace-back checks that every decision on the surviving path was won by at least margin_units units, which is more
 * than the rounding of 128 terms can move two candidates against each other; a pass that fails the check runs again on
 * fp64 metrics.  The states are those of mode 1 bit for bit.
 * mode 1: fp64 metrics only (viterbi_ref's own arithmetic, src/qtip_core.cpp:129-164).
 * In mode 0 a launch with at most a third as many tiles as the device has workgroup slots (a lone small group)
 * gives every tile a workgroup of 512 threads instead of 256, which shortens a tile's time by about a third; modes
 * 2 and 3 are mode 0 with the 256-thread and the 512-thread form whatever the size of the launch (tests).
 * margin_units: 0 = the default of 160; values below 129 give up the guarantee (tests only), UINT32_MAX sends every
 * pass to fp64. */
int qtip_set_viterbi_mode(qtip_ctx* ctx, int mode, unsigned margin_units);
/* Passes that mode 0 ran again on fp64 metrics since the context was made (or since the last call with reset != 0):
 * first passes (free ends, on the rotated sequence) and second passes (tail-biting).  Waits for the device.
 * Either pointer may be NULL. */
int qtip_viterbi_stats(qtip_ctx* ctx, unsigned long long* redone_first, unsigned long long* redone_second, int reset);
/* What qtip_opts.ldlq_chains = 0 stands for in this context: 2 or 3 (see there).  No counterpart in the reference,
 * whose LDLQ is one sequence of launches (src/quantizer.cpp:42-108). */
int qtip_ldlq_default_chains(qtip_ctx* ctx, int* chains);

/* hat[i] = lut[state[i]] (k_decode_states, src/viterbi.hip:231-238): B x 128 states -> B x 256 fp32 */
int qtip_decode_states_dev(qtip_ctx* ctx, const uint16_t* dev_states, long B, float* dev_hat);

/* Decoder of the packed output (decode_rows / decode_tile, runtime/src/qtip.cpp:83-118, word addressing of
 * HostLinear::word, runtime/include/behemoth/qtip.hpp:63-67): kernel-layout trellis u16[(m/16)*(n/16)*32] ->
 * hatWr m x n fp32 row-major, the rotated and Wscale-free weight (fp16 codebook values).  Asynchronous. */
int qtip_decode_trellis_dev(qtip_ctx* ctx, const uint16_t* dev_trellis, int m, int n, float* dev_hatWr);

/* Weight of one quantized linear in the original domain from what quantize_group returns for it:
 * hatW = diag(SV) U_m (hatWr * Wscale) U_n^T diag(SU), the reconstruction of src/quantizer.cpp:321-338 started from
 * the packed trellis instead of the LDLQ buffer (bit-identical to qtip_linear_out.hatW).  trellis, su_bf16[n], sv[m]
 * are host memory; hatW m x n fp32 is host memory, or device memory when hatW_on_device != 0.  Synchronous. */
int qtip_dequantize_linear(qtip_ctx* ctx, const uint16_t* host_trellis, const uint16_t* host_su_bf16,
                           const float* host_sv, float wscale, int m, int n, float* hatW, int hatW_on_device);

/* In-place row transform x <- (hadK^(T) (x) H_{n/K}) x / sqrt(n) of `rows` rows of length n, row stride ld
 * (k_hadamard_rows, src/kernels.hip:293-313; same fp32 dataflow, so results are bit-identical to it). */
int qtip_hadamard_rows_dev(qtip_ctx* ctx, float* dev_X, long rows, int n, long ld, int transpose);
int qtip_had_K(int n); /* get_hadK, src/qtip_core.cpp:77-81: K, or 0 if unsupported */

/* Sign vector from the splitmix stream (Rng::sign, src/common.hpp:91-107) */
void qtip_sign_vector(uint64_t seed, long count, float* host_out);

/* rotate_hessian, src/quantizer.cpp:124-152.  H: n x n fp32 (host, or device when h_on_device != 0; never
 * written).  Outputs (host): su[n] (+-1), *creg, HRr[n*n]. */
int qtip_rotate_hessian(qtip_ctx* ctx, const float* H, int h_on_device, int n, uint64_t seed, double sigma_reg,
                        float* host_su, double* creg, float* host_HRr);

/* ldl_hessian, src/quantizer.cpp:154-165 (+ block_ldl_to_L, src/qtip_core.cpp:444-487): host only, fp64,
 * uses its own OpenMP team of `threads`; safe to call from a side thread while the GPU works.
 * HRr n x n fp32 in, L n x n fp32 out (strictly block-lower). */
int qtip_ldl_hessian(const float* host_HRr, int n, int threads, float* host_L);

/* cholesky_inplace, src/qtip_core.hpp:24-67 / src/qtip_core.cpp:321-442: lower Cholesky factor of the n x n fp64
 * matrix host_A (row-major, lower triangle read and overwritten, the rest untouched or scratch), the reference's
 * order of operations, hence its bits.  Host only.  QTIP_E_NOT_PD if the matrix is not positive definite. */
int qtip_cholesky_inplace(double* host_A, int n, int threads);

/* The same factorization with the trailing updates of the host's panels on the GPU.  No counterpart in the
 * reference (its ldl_hessian is host only, src/quantizer.cpp:154-165): the host still factors and solves every
 * panel in fp64 with its own code, the device keeps the fp64 work matrix and applies the rank-256 updates on the
 * matrix cores in the host's own order of operations, so host_L is qtip_ldl_hessian's bit for bit.  Works on a
 * stream of its own inside ctx; may run on a side thread while another thread quantizes through the same ctx. */
int qtip_ldl_hessian_device_updates(qtip_ctx* ctx, const float* host_HRr, int n, int threads, float* host_L);

/* The same with the rotated Hessian already on the device (dev_HRr, n x n fp32, read only): the form
 * qtip_run_groups uses for the groups it schedules (the schedule of run_qtip_groups, src/pipeline.cpp:229-312, where
 * the reference calls its host-only ldl_hessian).  host_L as above; dev_L (optional, may be NULL): n x n fp32 device
 * buffer that receives L as well, column block by column block while the factorization runs - host_L is the source
 * of those copies and should then be page-locked. */
int qtip_ldl_hessian_device_updates_dev(qtip_ctx* ctx, const float* dev_HRr, int n, int threads, float* host_L,
                                        float* dev_L);

/* ldlq_gpu, src/quantizer.cpp:30-89.  WT n x m fp32 (scaled), L n x n fp32, both on the device;
 * outputs hatWT n x m fp32 and Q[(m/16)*(n/16)][128] u16 on the device.  feedback as in qtip_opts;
 * vit_seconds may be NULL. */
int qtip_ldlq_dev(qtip_ctx* ctx, const float* dev_WT, const float* dev_L, long n, long m, float* dev_hatWT,
                  uint16_t* dev_Q, int feedback, double* vit_seconds);

/* One linear of a group (LinearIn, src/quantizer.hpp:21-28): exactly one weight pointer is set. */
typedef struct {
  int m;                     /* out features */
  const float* w_f32;        /* [m][n] fp32 */
  const uint16_t* w_bf16;    /* [m][n] raw bf16 bits */
  const uint8_t* w_fp8;      /* [m][n] FP8 E4M3 with ... */
  const uint16_t* scale_bf16;/* ... [m] per-output-channel bf16 scale */
  int on_device;             /* 0: pointers are host memory, 1: device memory */
} qtip_linear_in;

/* Results for one linear (LinearOut, src/quantizer.hpp:30-43); buffers are caller-allocated host memory. */
typedef struct {
  uint16_t* trellis;   /* [(m/16)*(n/16)][32] u16, kernel layout */
  uint16_t* su_bf16;   /* [n] */
  float* sv;           /* [m] +-1 */
  float* hatW;         /* [m][n] or NULL (want_hatW) */
  float wscale;
  double proxy;
  double proxy_rot_reg;
  double seconds;
} qtip_linear_out;

typedef struct { /* QuantOpts, src/quantizer.hpp:11-19 */
  double sigma_reg;      /* 1e-2 */
  double scale_override; /* 0.9 */
  int ldl_threads;       /* 16 */
  int feedback;          /* 0: fp64 feedback sums + fp64 MFMA prod cache (default, tracks the fp64 CPU form);
                            1: fp32 feedback sums + bf16 hi/lo split MFMA prod cache (the reference GPU's arithmetic) */
  int skip_proxy;        /* 1: leave proxy fields 0 */
  int ldl_device_updates;/* 1 (default): qtip_run_groups and qtip_quantize_group_h factor through
                            qtip_ldl_hessian_device_updates (panels on the host, trailing updates on the GPU, same L
                            bit for bit); 0: block LDL on the host alone, as in the reference */
  int ldlq_chains;       /* LDLQ deals the tile rows of a group to this many independent chains of launches (each on
                            a stream of its own inside ctx), so that the trace-backs of one run under the forward
                            passes of the others; same codes whatever the number.  At most 3.  0 (default): 3 if the
                            context, when it was made, found three side streams that run beside its own stream and
                            beside each other (each on a hardware queue of its own: qtip_create times them), or if
                            the environment gave the process at least 6 hardware queues (GPU_MAX_HW_QUEUES, read by
                            the HIP runtime when it starts); else 2 - a chain whose stream shares a queue with
                            another stream runs after it, not beside it.  qtip_ldlq_default_chains tells which */
  int group_lanes;       /* qtip_run_groups runs this many groups side by side, each on a lane of its own inside ctx
                            (one stream, workspaces, staging), group g on lane g mod lanes; same results whatever
                            the number.  At most 12.  1: one group after the other, as the reference schedules them.
                            0 (default): as many as it takes for the largest group's 16-row tile rows to fill the
                            chip's 768 Viterbi workgroup slots (a 1024-row group fills a twelfth of them), 1 for
                            groups of 12288 rows and more.
                            Lanes whose streams share a hardware queue run one after the other: small groups gain
                            most where the process has a queue per lane (GPU_MAX_HW_QUEUES=16 in the environment
                            when the HIP runtime starts; HIP's default is 4) */
} qtip_opts;
void qtip_default_opts(qtip_opts* o);

typedef struct { /* GroupTiming, src/quantizer.hpp:45-47 */
  double load, rht, ldl_cpu, ldlq, viterbi, proxy, pack, total;
} qtip_timing;

/* The cross-buffer feedback ("prod cache") of one 128-column LDLQ buffer in the arithmetic of ldlq_gpu's update,
 * src/quantizer.cpp:66-76 (every fp32 operand as bf16 hi + lo, product = lo*hi + hi*lo + hi*hi on the bf16 matrix
 * cores, fp32 accumulate), in the gathered form qtip_ldlq_dev uses with feedback = 1: all rows quantized so far at once,
 *   P[r * N + j] = sum over k < K of Lrows[k * ldl + r] * (WT[k * ldw + j] - hatWT[k * ldw + j]),  r < 128, j < N,
 * where Lrows points at L[bufend][c0] and WT / hatWT at row bufend of the transposed weights.  The order of the fp32
 * sums is this library's (the reference leaves it to its BLAS).  N and K multiples of 64; synchronous. */
int qtip_prod_cache_bf16x3_dev(qtip_ctx* ctx, int N, long K, const float* dev_Lrows, long ldl, const float* dev_WT,
                               const float* dev_hatWT, long ldw, float* dev_P);

/* quantize_group(s, gemm, lins, hp, opt, tm, tag), src/quantizer.cpp:176-346, with the HessPrep fields passed
 * flat: su[n], creg, HRr[n*n], L[n*n] (host; L is read, never freed).  seed gives the SV streams. */
int qtip_quantize_group(qtip_ctx* ctx, int nlin, const qtip_linear_in* lins, int n, uint64_t seed,
                        const float* host_su, double creg, const float* host_HRr, const float* host_L,
                        const qtip_opts* opts, qtip_linear_out* outs, qtip_timing* timing);

/* quantize_group(s, gemm, lins, n, H, seed, opt, tm, tag), src/quantizer.cpp:167-174: rotate + LDL + quantize. */
int qtip_quantize_group_h(qtip_ctx* ctx, int nlin, const qtip_linear_in* lins, int n, const float* H,
                          int h_on_device, uint64_t seed, const qtip_opts* opts, qtip_linear_out* outs,
                          qtip_timing* timing);

/* Hessian accumulation, the step before the path (hess() in LayerRunner::forward_batch, src/model.cpp:352-363):
 * dev_H (n x n fp32, row-major) += X^T X for a batch of `rows` activation vectors dev_X (rows x n raw bf16 bits,
 * row-major), bf16 products with fp32 accumulation on the matrix cores.  Only the 256 x 256 tiles on or below the
 * diagonal are updated; qtip_hessian_finish_dev mirrors them into the other triangle and multiplies by `scale`
 * (symmetrize_hess, src/model.cpp:260-264, and the 1 / token count of src/pipeline.cpp:160-166).  n % 8 == 0, at
 * most 2097120 rows per call.  The batch is first rewritten in the layout the matrix cores are fed from, into a
 * buffer of the context (rows rounded up to 32 x n rounded up to 256 values of 2 bytes) that stays with it.
 * Asynchronous on the context's stream; calls on one context use that buffer one after the other. */
int qtip_hessian_accumulate_dev(qtip_ctx* ctx, const uint16_t* dev_X_bf16, long rows, int n, float* dev_H);
int qtip_hessian_finish_dev(qtip_ctx* ctx, float* dev_H, int n, double scale);

/* NVFP4 fallback quantizer (src/nvfp4.hpp, src/nvfp4.cpp, src/nvfp4_gpu.hpp, src/nvfp4_gpu.hip): two E2M1 values per
 * byte (low nibble first), one E4M3 scale per 16 input channels of a row, one fp32 global scale per matrix; the
 * tensors a layer file stores as weight_packed U8 [m][n/2], weight_scale F8_E4M3 [m][n/16], weight_global_scale F32. */
uint8_t qtip_f32_to_fp8e4m3(float x); /* src/nvfp4.hpp:15-33 */
/* nvfp4_quantize, src/nvfp4.cpp:12-55 (host, nearest value): w m x n fp32 -> packed, scales, *global */
int qtip_nvfp4_quantize(const float* host_w, int m, int n, uint8_t* host_packed, uint8_t* host_scales, float* global);
/* nvfp4_dequantize, src/nvfp4.cpp:57-70 (host; values rounded to bf16, as execution sees them) */
int qtip_nvfp4_dequantize(const uint8_t* host_packed, const uint8_t* host_scales, float global, int m, int n,
                          float* host_out);
/* nvfp4_proxy_error, src/nvfp4.cpp:72-87 (host, fp64): tr((W - What) H (W - What)^T) / m; host_H null = identity */
int qtip_nvfp4_proxy_error(const float* host_w, const float* host_what, int m, int n, const float* host_H, double* out);
typedef struct { /* Nvfp4Opts, src/nvfp4_gpu.hpp:21-25 */
  int scale_search; /* 1 */
  int calibrate;    /* 1 */
  double sigma_reg; /* 1e-2 */
  int factor_on_host; /* 0 (default): the calibration's Cholesky factorization runs its trailing updates on the GPU
                         (same L and dw bit for bit); 1: on the host alone, as qtip_nvfp4_prepare */
} qtip_nvfp4_opts;
typedef struct { /* one matrix of a group: input and the caller-allocated outputs (Nvfp4Tensor, src/nvfp4.hpp:35-41) */
  int m;
  const float* w;  /* host [m][n] fp32 */
  uint8_t* packed; /* host [m][n/2] */
  uint8_t* scales; /* host [m][n/16] */
  float global;    /* out */
} qtip_nvfp4_matrix;
/* nvfp4_quantize_group, src/nvfp4_gpu.hip:174-241: the matrices share one input Hessian host_H (n x n fp32; may be
 * NULL: no calibration, scale search weighted uniformly).  *calibrated (may be NULL) tells whether H was used for the
 * rounding.  QTIP_E_NOT_PD if the regularised Hessian is not positive definite. */
int qtip_nvfp4_quantize_group(qtip_ctx* ctx, int nmat, qtip_nvfp4_matrix* mats, int n, const float* host_H,
                              const qtip_nvfp4_opts* opts, int* calibrated);
/* The two halves of the call above, for callers that keep the factor: host preparation (src/nvfp4_gpu.hip:181-207:
 * calibrate -> unit-lower L with H = L D L^T and dw = D, else dw = diag(H) + creg, L untouched) and the device block
 * loop (:209-241) on a prepared factor (host_L NULL: no calibration; host_dw NULL: uniform weights). */
int qtip_nvfp4_prepare(const float* host_H, int n, double sigma_reg, int calibrate, int threads, float* host_L,
                       float* host_dw);
int qtip_nvfp4_quantize_prepared(qtip_ctx* ctx, int nmat, qtip_nvfp4_matrix* mats, int n, const float* host_L,
                                 const float* host_dw, int scale_search);
/* qtip_nvfp4_prepare with calibration, the rank-256 trailing updates of its fp64 Cholesky factorization on the GPU
 * (the host still factors and solves every panel): the same L and dw bit for bit, 0.6 s instead of 4.3 s at
 * n = 28672.  No counterpart in the reference, which factors on the host (src/nvfp4_gpu.hip:181-207). */
int qtip_nvfp4_prepare_device_updates(qtip_ctx* ctx, const float* host_H, int n, double sigma_reg, int threads,
                                      float* host_L, float* host_dw);

/* Several groups through one context with the overlap of run_qtip_groups, src/pipeline.cpp:229-312: Hessians are
 * rotated on the GPU ahead of use, a side thread runs the host fp64 LDL of the groups in order, and group g is
 * quantized as soon as its factor is ready (the LDL of group g+1 overlaps the GPU work of group g).  HRr and L live
 * in page-locked staging buffers owned by the context (a ring of three pairs, 6 n^2 floats, kept between calls).
 * timings / ldl_wait_s (seconds the GPU side waited for each group's factor) may be NULL.  On an error the
 * groups before the failing one are complete.
 * Groups too small to fill the chip run side by side (qtip_opts.group_lanes: group g on lane g mod lanes, each lane
 * takes its groups one after the other on a stream of its own; same results); then an error leaves the groups before the
 * failing one on its lane complete, the other lanes finish their groups, and the first failing lane's error is
 * reported.  With group_lanes = 0 and groups of mixed sizes, the groups of 12288 rows and more run first, in their
 * order, one after the other, and the smaller ones then share the chip on lanes. */
typedef struct {
  int nlin;
  const qtip_linear_in* lins;
  qtip_linear_out* outs; /* nlin entries, caller-allocated buffers as for qtip_quantize_group */
  int n;
  const float* H; /* n x n fp32, host or device */
  int h_on_device;
  uint64_t seed;
} qtip_group;
int qtip_run_groups(qtip_ctx* ctx, int ngroups, const qtip_group* groups, const qtip_opts* opts, qtip_timing* timings,
                    double* ldl_wait_s);
/* The number of lanes qtip_run_groups would use for these groups and options (1: one group after the other).  Reads
 * only nlin, lins[].m and n of each group.  No counterpart in the reference, which runs one group at a time. */
int qtip_group_lanes(qtip_ctx* ctx, int ngroups, const qtip_group* groups, const qtip_opts* opts, int* lanes);
/* Host-only check of the lane rule: `ngroups` equal groups of one m x n linear on a device with `device_slots`
 * Viterbi workgroup slots, qtip_opts.group_lanes = requested. */
int qtip_selftest_group_lanes(int device_slots, int ngroups, int m, int n, int requested, int* lanes);
/* Allocates the staging ring of qtip_run_groups for Hessians up to n x n ahead of the first call (optional). */
int qtip_reserve_groups(qtip_ctx* ctx, int n);

/* Layer file writer: the safetensors container of SafeTensorsWriter, src/safetensors.cpp:93-137 (u64 header length,
 * JSON header with sorted keys padded to 8 bytes, tensors back to back in name order, written to path + ".tmp" and
 * renamed).  Host only; no context needed.  dtype strings are safetensors names ("I16", "BF16", "F32", "F16", "I64",
 * "F8_E4M3", "U8", ...); data is copied by qtip_st_add; adding a name twice replaces the tensor. */
typedef struct qtip_st_writer qtip_st_writer;
int qtip_st_create(qtip_st_writer** out);
void qtip_st_destroy(qtip_st_writer* w);
int qtip_st_add(qtip_st_writer* w, const char* name, const char* dtype, const int64_t* shape, int rank,
                const void* data, uint64_t bytes);
/* The six tensors of one QTIP linear under `prefix` (e.g. "model.layers.3.mlp.down_proj."), as write_layer_file
 * stores them (src/pipeline.cpp:329-340): trellis I16 [(m/16)(n/16)][32], SU BF16 [n], SV F32 [m] = sv * wscale,
 * tlut F16 [512][2], rcp I64 = 0, tp_rank I64 = 8.  tlut_f16 NULL takes the built-in HYB table. */
int qtip_st_add_qtip_linear(qtip_st_writer* w, const char* prefix, const qtip_linear_out* out, int m, int n,
                            const uint16_t* tlut_f16);
/* metadata_kv: 2 * nmeta strings (key, value, ...); NULL writes the reference's default {"format": "pt"}.
 * *bytes_written (may be NULL) receives the file size. */
int qtip_st_write(qtip_st_writer* w, const char* path, const char* const* metadata_kv, int nmeta,
                  uint64_t* bytes_written);
/* fp16 bits of the context's codebook table [512][2] (Codebook::tlut_h, src/qtip_core.hpp:24-31) */
int qtip_get_tlut_f16(qtip_ctx* ctx, uint16_t* host_tlut_f16);

/* Device memory the context keeps between calls for reuse (per-group buffers of qtip_run_groups and
 * qtip_quantize_group*, about 13 GB after 12288 x 28672 groups, and the same per lane) goes back to the runtime;
 * buffers in use are not touched.  No counterpart in the reference, whose buffers are freed on return
 * (RAII DBuf, src/gpu.hpp:139-160).  The library does the same by itself when an allocation finds the device out of
 * memory.  *bytes_released may be NULL.  Must not overlap another call on the same context. */
int qtip_trim(qtip_ctx* ctx, unsigned long long* bytes_released);

/* Host-only: the number of device allocations (hipMalloc) the library has made in this process so far; a test of
 * qtip_viterbi_tiles_dev_noalloc reads it before and after the call.  No counterpart in the reference. */
long qtip_selftest_device_alloc_calls(void);

/* Host-only self test (no GPU needed, no counterpart in the reference): a device buffer of the context whose
 * allocation failed stays empty, so the next call allocates again instead of launching on a null pointer.  0 = ok. */
int qtip_selftest_failed_alloc_is_retried(void);

/* Host-only self test (no GPU needed, no counterpart in the reference): the block LDL through the panel hand-over
 * that qtip_ldl_hessian_device_updates uses (a panel's columns fetched, factored and solved by the host, the rows
 * handed back, L assembled from them as they pass), with the trailing matrix held and updated by plain host code
 * instead of the device.  host_L must come out as qtip_ldl_hessian's, bit for bit. */
int qtip_selftest_ldl_panel_handover(const float* host_HRr, int n, int threads, float* host_L);

/* Host packers (pack_trellis / unpack_trellis / swizzle_for_kernel / unswizzle_for_kernel,
 * src/qtip_core.cpp:194-253) */
void qtip_pack_trellis(const uint16_t* states, long B, uint16_t* packed);
void qtip_unpack_trellis(const uint16_t* packed, long B, uint16_t* states);
int qtip_swizzle_for_kernel(const uint16_t* packed, int m, int n, uint16_t* out);
int qtip_unswizzle_for_kernel(const uint16_t* in, int m, int n, uint16_t* packed);

#ifdef __cplusplus
}
#endif
#endif
