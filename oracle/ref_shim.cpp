// Test infrastructure only: extern "C" doorway into the reference's own CPU core (qtip_core.cpp),
// compiled from the sources where they lie under /root/reference by oracle/Makefile into
// oracle/_ref/libqtip_ref.so.  Nothing on the product path may load this library.
//
// Every function forwards to the reference function named in its comment
// (declarations: src/qtip_core.hpp:24-67, src/common.hpp:42-107).
#include <cstdint>
#include <cstring>
#include <vector>

#include "common.hpp"
#include "nvfp4.hpp"
#include "qtip_core.hpp"

using namespace qtip;

extern "C" {

// codebook() src/qtip_core.cpp:47-50 -- copies out the 65536-entry decoded LUT of the built-in HYB tlut
void ref_codebook(float* lut0, float* lut1, uint32_t* lut_h2, double* lut_rms, float* tlut) {
  const Codebook& cb = codebook();
  if (lut0) std::memcpy(lut0, cb.lut0.data(), kStates * 4);
  if (lut1) std::memcpy(lut1, cb.lut1.data(), kStates * 4);
  if (lut_h2) std::memcpy(lut_h2, cb.lut_h2.data(), kStates * 4);
  if (lut_rms) *lut_rms = cb.lut_rms;
  if (tlut) std::memcpy(tlut, cb.tlut, sizeof(cb.tlut));
}

// Replace the decoded LUT the reference's Viterbi reads (a synthetic tlut has no other way in:
// build_codebook() src/qtip_core.cpp:18-46 hard-wires the HYB table).  The caller supplies a LUT
// built by the oracle, whose construction is pinned separately against tests/refvec/lut.bin.
void ref_override_codebook(const float* lut0, const float* lut1, const uint32_t* lut_h2, double lut_rms) {
  Codebook& cb = const_cast<Codebook&>(codebook());
  std::memcpy(cb.lut0.data(), lut0, kStates * 4);
  std::memcpy(cb.lut1.data(), lut1, kStates * 4);
  std::memcpy(cb.lut_h2.data(), lut_h2, kStates * 4);
  cb.lut_rms = lut_rms;
}

void ref_perm256(int* perm, int* inv) {  // src/qtip_core.cpp:52-73
  std::memcpy(perm, perm256(), 256 * sizeof(int));
  std::memcpy(inv, inv_perm256(), 256 * sizeof(int));
}
int ref_had_K(int n) { return had_K(n); }  // src/qtip_core.cpp:77-81
void ref_hadamard_rows(double* X, long rows, int n, long ld, int transpose) {  // :83-120
  hadamard_rows_ref(X, rows, n, ld, transpose != 0);
}
double ref_viterbi(const float* X, int overlap, uint16_t* states) { return viterbi_ref(X, overlap, states); }  // :129-164
double ref_quantize_seq(const float* X, uint16_t* states, float* hatX) { return quantize_seq_ref(X, states, hatX); }  // :180-191
void ref_decode_states(const uint16_t* states, float* hatX) { decode_states(states, hatX); }  // :166-172
double ref_path_cost(const float* X, const uint16_t* states) { return path_cost(X, states); }  // :174-178
void ref_pack_trellis(const uint16_t* st, long B, uint16_t* packed) { pack_trellis(st, B, packed); }  // :194-208
void ref_unpack_trellis(const uint16_t* packed, long B, uint16_t* st) { unpack_trellis(packed, B, st); }  // :210-228
void ref_swizzle(const uint16_t* packed, int m, int n, uint16_t* out) { swizzle_for_kernel(packed, m, n, out); }  // :233-243
void ref_unswizzle(const uint16_t* in, int m, int n, uint16_t* packed) { unswizzle_for_kernel(in, m, n, packed); }  // :244-253
int ref_cholesky(double* A, int n, int threads) { return cholesky_inplace(A, n, threads) ? 1 : 0; }  // :321-442
int ref_block_ldl(double* A, int n, float* L, int threads) { return block_ldl_to_L(A, n, L, threads) ? 1 : 0; }  // :444-487

uint16_t ref_f32_to_fp16(float f) { return f32_to_fp16(f); }  // src/common.hpp:57-78
float ref_fp16_to_f32(uint16_t h) { return fp16_to_f32(h); }  // :49-56
uint16_t ref_f32_to_bf16(float f) { return f32_to_bf16(f); }  // :42-48
float ref_bf16_to_f32(uint16_t h) { return bf16_to_f32(h); }  // :37-41

// Rng src/common.hpp:91-107: kind 0 = next(), 1 = uniform(), 2 = normal(), 3 = sign()
void ref_rng(uint64_t seed, int kind, long count, double* out_f, uint64_t* out_u) {
  Rng r(seed);
  for (long i = 0; i < count; ++i) {
    switch (kind) {
      case 0: out_u[i] = r.next(); break;
      case 1: out_f[i] = r.uniform(); break;
      case 2: out_f[i] = r.normal(); break;
      default: out_f[i] = r.sign(); break;
    }
  }
}
// NVFP4 fallback quantizer, src/nvfp4.hpp / src/nvfp4.cpp
unsigned ref_f32_to_fp8e4m3(float x) { return f32_to_fp8e4m3(x); }  // src/nvfp4.hpp:15-33
float ref_nvfp4_quantize(const float* w, int m, int n, uint8_t* packed, uint8_t* scales) {  // src/nvfp4.cpp:12-55
  Nvfp4Tensor t = nvfp4_quantize(w, m, n);
  std::memcpy(packed, t.packed.data(), t.packed.size());
  std::memcpy(scales, t.scales.data(), t.scales.size());
  return t.global;
}
void ref_nvfp4_dequantize(const uint8_t* packed, const uint8_t* scales, float global, int m, int n, float* out) {  // :57-70
  Nvfp4Tensor t;
  t.m = m, t.n = n, t.global = global;
  t.packed.assign(packed, packed + size_t(m) * n / 2);
  t.scales.assign(scales, scales + size_t(m) * n / 16);
  std::vector<float> v = nvfp4_dequantize(t);
  std::memcpy(out, v.data(), v.size() * 4);
}
double ref_nvfp4_proxy_error(const float* w, const float* what, int m, int n, const float* H) {  // :72-87
  return nvfp4_proxy_error(w, what, m, n, H);
}
}
