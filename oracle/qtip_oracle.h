/* TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
 *
 * CPU restatement (plain C, fp64 where the reference is fp64) of the algorithm of the reference's
 * per-Hessian-group QTIP quantize path.  Only tests/, __graft_entry__.smoke() and bench.py's
 * cpu_baseline leg may load this library, and only as the checker.  The product library must never
 * link, load or call it.
 *
 * Each function names the reference lines it restates (paths relative to the reference root).
 * How each function is pinned (golden vectors of the reference's own tests, the compiled reference
 * in oracle/_ref, closed forms, brute force) is listed in tests/test_oracle_*.py; a function without
 * such a check is marked "parity unpinned" here.
 */
#ifndef QTIP_ORACLE_H_
#define QTIP_ORACLE_H_
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { QO_L = 16, QO_KV = 4, QO_SEQ = 256, QO_STEPS = 128, QO_STATES = 65536, QO_GROUPS = 4096, QO_WORDS = 32 };

/* ---- number formats, src/common.hpp:37-78 */
uint16_t qo_f32_to_fp16(float f);
float qo_fp16_to_f32(uint16_t h);
float qo_round_fp16(float f);
uint16_t qo_f32_to_bf16(float f);
float qo_bf16_to_f32(uint16_t h);

/* ---- splitmix64 stream, src/common.hpp:91-107.  kind 0 next(), 1 uniform(), 2 normal(), 3 sign() */
void qo_rng(uint64_t seed, int kind, long count, double* out_f, uint64_t* out_u);

/* ---- codebook, src/qtip_core.cpp:18-46.  tlut: 512x2 fp32.  Outputs have 65536 entries each. */
void qo_build_codebook(const float* tlut, float* lut0, float* lut1, uint32_t* lut_h2, double* lut_rms);
const uint32_t* qo_hyb_tlut_bits(void); /* the default HYB tlut, 1024 fp32 bit patterns */

/* ---- tile <-> sequence permutation, src/qtip_core.cpp:52-73 */
void qo_perm256(int* perm, int* inv);

/* ---- Hadamard, src/qtip_core.cpp:77-120 (fp64) and src/kernels.hip:214-254,293-313 (fp32 dataflow) */
int qo_had_K(int n);
int qo_hadamard_rows(double* X, long rows, int n, long ld, int transpose);
int qo_hadamard_rows_f32(float* X, long rows, int n, long ld, int transpose);

/* ---- Viterbi, src/qtip_core.cpp:123-191 */
double qo_viterbi(const float* lut0, const float* lut1, const float* X, int overlap, uint16_t* states);
double qo_viterbi_fast(const float* lut0, const float* lut1, const float* X, int overlap, uint16_t* states);
double qo_quantize_seq(const float* lut0, const float* lut1, const float* X, uint16_t* states, float* hatX);
/* B independent sequences, OpenMP over sequences (threads <= 0: library default). fast != 0 uses qo_viterbi_fast */
void qo_quantize_tiles(const float* lut0, const float* lut1, const float* X, long B, uint16_t* states, float* hatX,
                       int threads, int fast);
void qo_decode_states(const float* lut0, const float* lut1, const uint16_t* states, float* hatX);
double qo_path_cost(const float* lut0, const float* lut1, const float* X, const uint16_t* states);

/* ---- packing, src/qtip_core.cpp:194-253 */
void qo_pack_trellis(const uint16_t* states, long B, uint16_t* packed);
void qo_unpack_trellis(const uint16_t* packed, long B, uint16_t* states);
int qo_swizzle_for_kernel(const uint16_t* packed, int m, int n, uint16_t* out);
int qo_unswizzle_for_kernel(const uint16_t* in, int m, int n, uint16_t* packed);

/* ---- fp64 Cholesky and block LDL, src/qtip_core.cpp:321-487 (textbook order, unblocked) */
int qo_cholesky(double* A, int n);
int qo_block_ldl_to_L(double* A, int n, float* L);

/* ---- LDLQ with 128-column buffers, tests/test_gpu.cpp:180-225.  Wr m x n, L n x n; outputs hatWr m x n,
 *      Q[(m/16)*(n/16)][128].  lut0/lut1 give the codebook. */
int qo_ldlq(const float* lut0, const float* lut1, const float* Wr, const float* L, int m, int n, float* hatWr,
            uint16_t* Q, int threads);
/* Same quantizer written without buffers or prod cache: every column block's target is formed directly from
 * all later columns.  Used to pin qo_ldlq. */
int qo_ldlq_naive(const float* lut0, const float* lut1, const float* Wr, const float* L, int m, int n, float* hatWr,
                  uint16_t* Q, int threads);

/* ---- Hessian rotation + regularisation, src/quantizer.cpp:124-152 (fp32 dataflow of the GPU kernels) */
int qo_rotate_hessian(const float* H, int n, uint64_t seed, double sigma_reg, float* su, double* creg, float* HRr);
/* src/quantizer.cpp:154-165 */
int qo_ldl_hessian(const float* HRr, int n, float* L);

/* ---- whole group, src/quantizer.cpp:176-346.  nlin linears W[i] (m[i] x n, fp32, row-major), shared Hessian.
 * Per linear li the outputs are written at: trellis + 32*(off_i/16)*(n/16), sv + off_i, wscale[li], proxy[li],
 * proxy_rot_reg[li]; states Q (optional) as [(mt/16)*(n/16)][128]; hatWT/WT (optional) n x mt. */
int qo_quantize_group(const float* tlut, int nlin, const float* const* W, const int* m, int n, const float* H,
                      uint64_t seed, double sigma_reg, double scale_override, uint16_t* trellis, uint16_t* su_bf16,
                      float* sv, float* wscale, double* proxy, double* proxy_rot_reg, uint16_t* Q, float* WT_out,
                      float* hatWT_out, int threads);

/* tr(D H D^T)/tr(W H W^T) in fp64; W, hatW m x n row-major, H n x n */
double qo_proxy(const float* W, const float* hatW, const float* H, int m, int n, int threads);

/* ---- NVFP4 fallback quantizer (two E2M1 values per byte, one E4M3 scale per 16 input channels, one fp32 global
 *      scale per matrix).  Format and the plain quantizer: src/nvfp4.hpp:15-33,54-57, src/nvfp4.cpp:12-87.  Scale
 *      search and Hessian-calibrated rounding: a CPU restatement of the reference's GPU kernels
 *      (src/nvfp4_gpu.hip:66-228) in the same fp32 operation order; its three "sum += a * b" statements are fused
 *      multiply-adds, as hipcc's default contraction compiles them.  Pinned by the bytes the reference's own device
 *      path returned on a gfx950 GPU (tests/golden/ref_nvfp4_gpu_*) and, on a GPU, by that library itself. */
uint8_t qo_f32_to_fp8e4m3(float x);
float qo_fp8e4m3_to_f32(uint8_t b);
/* nvfp4_quantize, src/nvfp4.cpp:12-55: w m x n fp32 -> packed [m][n/2], scales [m][n/16], *global.  -1 if n % 16. */
int qo_nvfp4_quantize(const float* w, int m, int n, uint8_t* packed, uint8_t* scales, float* global);
/* nvfp4_dequantize, src/nvfp4.cpp:57-70 (values rounded to bf16) */
void qo_nvfp4_dequantize(const uint8_t* packed, const uint8_t* scales, float global, int m, int n, float* out);
/* nvfp4_proxy_error, src/nvfp4.cpp:72-87: tr(E H E^T) / m, H may be NULL (identity) */
double qo_nvfp4_proxy_error(const float* w, const float* what, int m, int n, const float* H);
/* Host preparation of nvfp4_quantize_group, src/nvfp4_gpu.hip:181-207: regularised H -> unit-lower L (n x n fp32,
 * H = L D L^T) and dw = D when calibrate, else dw = diag(H) + creg and L untouched.  0 ok, -1 not positive definite. */
int qo_nvfp4_prepare(const float* H, int n, double sigma_reg, int calibrate, float* L, float* dw);
/* The block loop of nvfp4_quantize_group, src/nvfp4_gpu.hip:217-228 with nv_block_kernel :66-158 and
 * nv_feedback_kernel :161-172: 16-column blocks from the last to the first.  L / dw may be NULL (no calibration /
 * uniform weights); global as returned by qo_nvfp4_quantize. */
void qo_nvfp4_blocks(const float* w, int m, int n, const float* L, const float* dw, float global, int calibrate,
                     int search, uint8_t* packed, uint8_t* scales);

#ifdef __cplusplus
}
#endif
#endif
