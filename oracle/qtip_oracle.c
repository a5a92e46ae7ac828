/* TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.  See qtip_oracle.h.
 *
 * Built with -ffp-contract=off: every fused multiply-add below is written out with fma(), so the
 * arithmetic does not depend on compiler flags.  The reference's own build (GCC -O3, default
 * -ffp-contract=fast, FMA host) evaluates its squared error as fma(a, a, b*b); tests check this
 * file against that compiled code bit for bit (returned path metrics included).
 */
#include "qtip_oracle.h"

#include <math.h>
#include <omp.h>
#include <stdlib.h>
#include <string.h>

#include "../behemoth-qtip_amd/csrc/data/qtip_tables.h"

/* ------------------------------------------------------------------ number formats */
float qo_bf16_to_f32(uint16_t h) { /* src/common.hpp:37-41 */
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}
uint16_t qo_f32_to_bf16(float f) { /* src/common.hpp:42-48, round to nearest even */
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
float qo_fp16_to_f32(uint16_t h) { /* src/common.hpp:49-56 */
  uint32_t s = (h >> 15) & 1, e = (h >> 10) & 0x1f, m = h & 0x3ff;
  float v;
  if (e == 0) v = ldexpf((float)m, -24);
  else if (e == 31) v = m ? NAN : INFINITY;
  else v = ldexpf((float)(m | 0x400), (int)e - 25);
  return s ? -v : v;
}
uint16_t qo_f32_to_fp16(float f) { /* src/common.hpp:57-78, round to nearest even */
  uint32_t u;
  memcpy(&u, &f, 4);
  uint32_t sign = (u >> 16) & 0x8000u;
  uint32_t a = u & 0x7fffffffu;
  if (a >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (a > 0x7f800000u ? 0x200u : 0u));
  if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);
  if (a < 0x38800000u) { /* fp16 subnormal or zero: value / 2^-24 rounded to nearest even */
    float af;
    memcpy(&af, &a, 4);
    float r = nearbyintf(af * 16777216.0f);
    return (uint16_t)(sign | (uint32_t)r);
  }
  uint32_t e = (a >> 23) - 112;
  uint32_t m = a & 0x7fffffu;
  uint32_t h = (e << 10) | (m >> 13);
  uint32_t rem = m & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
  return (uint16_t)(sign | h);
}
float qo_round_fp16(float f) { return qo_fp16_to_f32(qo_f32_to_fp16(f)); }

/* ------------------------------------------------------------------ rng, src/common.hpp:91-107 */
typedef struct { uint64_t s; } qo_rng_t;
static void rng_init(qo_rng_t* r, uint64_t seed) { r->s = seed * 0x9E3779B97F4A7C15ull + 0x1234567ull; }
static uint64_t rng_next(qo_rng_t* r) {
  uint64_t z = (r->s += 0x9E3779B97F4A7C15ull);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
static double rng_uniform(qo_rng_t* r) { return (double)(rng_next(r) >> 11) * (1.0 / 9007199254740992.0); }
static double rng_normal(qo_rng_t* r) {
  double u1 = rng_uniform(r), u2 = rng_uniform(r);
  if (u1 < 1e-300) u1 = 1e-300;
  return sqrt(-2.0 * log(u1)) * cos(6.283185307179586 * u2);
}
static float rng_sign(qo_rng_t* r) { return (rng_next(r) >> 63) ? -1.0f : 1.0f; }
void qo_rng(uint64_t seed, int kind, long count, double* out_f, uint64_t* out_u) {
  qo_rng_t r;
  rng_init(&r, seed);
  for (long i = 0; i < count; ++i) {
    if (kind == 0) out_u[i] = rng_next(&r);
    else if (kind == 1) out_f[i] = rng_uniform(&r);
    else if (kind == 2) out_f[i] = rng_normal(&r);
    else out_f[i] = rng_sign(&r);
  }
}

/* ------------------------------------------------------------------ codebook, src/qtip_core.cpp:18-46 */
const uint32_t* qo_hyb_tlut_bits(void) { return qtip_hyb_tlut_bits; }
void qo_build_codebook(const float* tlut, float* lut0, float* lut1, uint32_t* lut_h2, double* lut_rms) {
  double ss = 0;
  for (uint32_t s = 0; s < QO_STATES; ++s) {
    uint64_t p = (uint64_t)(s + 1) * (uint64_t)s; /* quantlut_sym */
    int flip = (int)((p >> 15) & 1);
    int idx = (int)((p >> (16 - 9 - 1)) & 511);
    uint16_t h0 = qo_f32_to_fp16(tlut[idx * 2 + 0]), h1 = qo_f32_to_fp16(tlut[idx * 2 + 1]);
    if (flip) h0 ^= 0x8000;
    float a = qo_fp16_to_f32(h0), b = qo_fp16_to_f32(h1);
    if (lut0) lut0[s] = a;
    if (lut1) lut1[s] = b;
    if (lut_h2) lut_h2[s] = (uint32_t)h0 | ((uint32_t)h1 << 16);
    ss += (double)a * a + (double)b * b;
  }
  if (lut_rms) *lut_rms = sqrt(ss / (2.0 * QO_STATES));
}

/* ------------------------------------------------------------------ permutation, src/qtip_core.cpp:52-73 */
void qo_perm256(int* perm, int* inv) {
  int p = 0;
  int loc[256];
  /* arange(256).reshape(2, 8, 2, 4, 2).permute(1, 3, 2, 0, 4) */
  for (int b = 0; b < 8; ++b)
    for (int d = 0; d < 4; ++d)
      for (int c = 0; c < 2; ++c)
        for (int a = 0; a < 2; ++a)
          for (int e = 0; e < 2; ++e) loc[p++] = a * 128 + b * 16 + c * 8 + d * 2 + e;
  for (int i = 0; i < 256; ++i) {
    if (perm) perm[i] = loc[i];
    if (inv) inv[loc[i]] = i;
  }
}

/* ------------------------------------------------------------------ Hadamard */
static int is_pow2(long n) { return n > 0 && (n & (n - 1)) == 0; }
int qo_had_K(int n) { /* src/qtip_core.cpp:77-81: first K of the order list dividing n decides */
  for (int i = 0; i < QTIP_NUM_HAD; ++i) {
    int K = qtip_had_order[i];
    if (n % K == 0) return is_pow2(n / K) ? K : 0;
  }
  return is_pow2(n) ? 1 : 0;
}

int qo_hadamard_rows(double* X, long rows, int n, long ld, int transpose) { /* src/qtip_core.cpp:83-120 */
  int K = qo_had_K(n);
  if (K <= 0) return -1;
  const uint32_t* hb = K > 1 ? qtip_had_bits(K) : 0;
  int P = n / K;
  double sc = 1.0 / sqrt((double)n);
#pragma omp parallel
  {
    double* y = (double*)malloc(sizeof(double) * (size_t)n);
    double* z = (double*)malloc(sizeof(double) * (size_t)n);
#pragma omp for schedule(static)
    for (long r = 0; r < rows; ++r) {
      double* x = X + r * ld;
      memcpy(y, x, sizeof(double) * (size_t)n);
      for (int c = 0; c < K; ++c) { /* natural-order FWHT on each contiguous chunk */
        double* v = y + (long)c * P;
        for (int h = 1; h < P; h <<= 1)
          for (int i = 0; i < P; i += 2 * h)
            for (int j = i; j < i + h; ++j) {
              double a = v[j], b = v[j + h];
              v[j] = a + b;
              v[j + h] = a - b;
            }
      }
      if (K > 1) {
        for (int k2 = 0; k2 < K; ++k2)
          for (int i = 0; i < P; ++i) {
            double s = 0;
            for (int k = 0; k < K; ++k) {
              int h = transpose ? qtip_had_entry(hb, K, k, k2) : qtip_had_entry(hb, K, k2, k);
              s += (double)h * y[(long)k * P + i];
            }
            z[(long)k2 * P + i] = s;
          }
        for (int i = 0; i < n; ++i) x[i] = z[i] * sc;
      } else {
        for (int i = 0; i < n; ++i) x[i] = y[i] * sc;
      }
    }
    free(y);
    free(z);
  }
  return 0;
}

/* fp32 dataflow of the reference's GPU Hadamard (src/kernels.hip:214-254 kernels, :293-313 driver):
 * stage 1 butterflies h = 1, 2, 4 ... on each chunk, scaled by (K == 1 ? sc : 1); stage 2 signed sum over
 * k ascending starting from 0, times sc; sc = 1.0f / sqrtf(n). */
int qo_hadamard_rows_f32(float* X, long rows, int n, long ld, int transpose) {
  int K = qo_had_K(n);
  if (K <= 0) return -1;
  int P = n / K;
  if (P > 8192) return -2; /* src/kernels.hip:297 */
  const uint32_t* hb = K > 1 ? qtip_had_bits(K) : 0;
  float sc = 1.0f / sqrtf((float)n);
  float scale1 = K == 1 ? sc : 1.0f;
#pragma omp parallel
  {
    float* y = (float*)malloc(sizeof(float) * (size_t)n);
#pragma omp for schedule(static)
    for (long r = 0; r < rows; ++r) {
      float* x = X + r * ld;
      memcpy(y, x, sizeof(float) * (size_t)n);
      for (int c = 0; c < K; ++c) {
        float* v = y + (long)c * P;
        for (int h = 1; h < P; h <<= 1)
          for (int i = 0; i < P; i += 2 * h)
            for (int j = i; j < i + h; ++j) {
              float a = v[j], b = v[j + h];
              v[j] = a + b;
              v[j + h] = a - b;
            }
        for (int i = 0; i < P; ++i) v[i] = v[i] * scale1;
      }
      if (K > 1) {
        for (int k2 = 0; k2 < K; ++k2)
          for (int i = 0; i < P; ++i) {
            float s = 0;
            for (int k = 0; k < K; ++k) {
              int h = transpose ? qtip_had_entry(hb, K, k, k2) : qtip_had_entry(hb, K, k2, k);
              float t = y[(long)k * P + i];
              s += h > 0 ? t : -t;
            }
            x[(long)k2 * P + i] = s * sc;
          }
      } else {
        memcpy(x, y, sizeof(float) * (size_t)n);
      }
    }
    free(y);
  }
  return 0;
}

/* ------------------------------------------------------------------ Viterbi, src/qtip_core.cpp:123-164 */
static inline double sq_err(const float* lut0, const float* lut1, uint32_t s, double x0, double x1) {
  double a = (double)lut0[s] - x0, b = (double)lut1[s] - x1;
  return fma(a, a, b * b);
}

double qo_viterbi(const float* lut0, const float* lut1, const float* X, int overlap, uint16_t* states) {
  const double INF = INFINITY;
  double* cost = (double*)malloc(sizeof(double) * QO_STATES);
  double* ncost = (double*)malloc(sizeof(double) * QO_STATES);
  double* M = (double*)malloc(sizeof(double) * QO_GROUPS);
  uint8_t* A = (uint8_t*)malloc((size_t)QO_STEPS * QO_GROUPS);
  for (uint32_t s = 0; s < QO_STATES; ++s) {
    cost[s] = sq_err(lut0, lut1, s, X[0], X[1]);
    if (overlap >= 0 && (int)(s >> QO_KV) != overlap) cost[s] = INF;
  }
  for (int i = 1; i < QO_STEPS; ++i) {
    for (int j = 0; j < QO_GROUPS; ++j) {
      double best = cost[j];
      int bd = 0;
      for (int d = 1; d < 16; ++d) {
        double c = cost[j | (d << 12)];
        if (c < best) best = c, bd = d;
      }
      M[j] = best;
      A[(size_t)i * QO_GROUPS + j] = (uint8_t)bd;
    }
    double x0 = X[2 * i], x1 = X[2 * i + 1];
    for (uint32_t s = 0; s < QO_STATES; ++s) ncost[s] = sq_err(lut0, lut1, s, x0, x1) + M[s >> QO_KV];
    double* t = cost;
    cost = ncost;
    ncost = t;
  }
  double best = INF;
  uint32_t bs = 0;
  for (uint32_t s = 0; s < QO_STATES; ++s) {
    if (overlap >= 0 && (int)(s & (QO_GROUPS - 1)) != overlap) continue;
    if (cost[s] < best) best = cost[s], bs = s;
  }
  states[QO_STEPS - 1] = (uint16_t)bs;
  for (int i = QO_STEPS - 1; i > 0; --i) {
    uint32_t j = states[i] >> QO_KV;
    states[i - 1] = (uint16_t)(j | ((uint32_t)A[(size_t)i * QO_GROUPS + j] << 12));
  }
  free(cost);
  free(ncost);
  free(M);
  free(A);
  return best;
}

/* Same recursion with the per-step squared errors tabulated once per distinct LUT entry: lut[s] depends
 * on s only through the 10 bits ((s*(s+1)) >> 6) & 1023, so there are 1024 distinct error values per step.
 * Valid only for LUTs produced by qo_build_codebook.  Values, comparisons and their order are unchanged. */
double qo_viterbi_fast(const float* lut0, const float* lut1, const float* X, int overlap, uint16_t* states) {
  const double INF = INFINITY;
  static uint16_t* code = 0;
  static uint32_t rep[1024];
#pragma omp critical(qo_code_init)
  {
    if (!code) {
      uint16_t* c = (uint16_t*)malloc(sizeof(uint16_t) * QO_STATES);
      for (int k = 0; k < 1024; ++k) rep[k] = 0xffffffffu;
      for (uint32_t s = 0; s < QO_STATES; ++s) {
        c[s] = (uint16_t)(((s * (s + 1)) >> 6) & 1023);
        if (rep[c[s]] == 0xffffffffu) rep[c[s]] = s;
      }
      code = c;
    }
  }
  double* cost = (double*)malloc(sizeof(double) * QO_STATES);
  double* ncost = (double*)malloc(sizeof(double) * QO_STATES);
  double* M = (double*)malloc(sizeof(double) * QO_GROUPS);
  uint8_t* A = (uint8_t*)malloc((size_t)QO_STEPS * QO_GROUPS);
  double E[1024];
  for (int k = 0; k < 1024; ++k) E[k] = sq_err(lut0, lut1, rep[k], X[0], X[1]);
  for (uint32_t s = 0; s < QO_STATES; ++s) {
    cost[s] = E[code[s]];
    if (overlap >= 0 && (int)(s >> QO_KV) != overlap) cost[s] = INF;
  }
  for (int i = 1; i < QO_STEPS; ++i) {
    for (int j = 0; j < QO_GROUPS; ++j) M[j] = cost[j];
    memset(A + (size_t)i * QO_GROUPS, 0, QO_GROUPS);
    for (int d = 1; d < 16; ++d) {
      const double* cd = cost + ((size_t)d << 12);
      uint8_t* Ai = A + (size_t)i * QO_GROUPS;
      for (int j = 0; j < QO_GROUPS; ++j)
        if (cd[j] < M[j]) M[j] = cd[j], Ai[j] = (uint8_t)d;
    }
    double x0 = X[2 * i], x1 = X[2 * i + 1];
    for (int k = 0; k < 1024; ++k) E[k] = sq_err(lut0, lut1, rep[k], x0, x1);
    for (uint32_t s = 0; s < QO_STATES; ++s) ncost[s] = E[code[s]] + M[s >> QO_KV];
    double* t = cost;
    cost = ncost;
    ncost = t;
  }
  double best = INF;
  uint32_t bs = 0;
  for (uint32_t s = 0; s < QO_STATES; ++s) {
    if (overlap >= 0 && (int)(s & (QO_GROUPS - 1)) != overlap) continue;
    if (cost[s] < best) best = cost[s], bs = s;
  }
  states[QO_STEPS - 1] = (uint16_t)bs;
  for (int i = QO_STEPS - 1; i > 0; --i) {
    uint32_t j = states[i] >> QO_KV;
    states[i - 1] = (uint16_t)(j | ((uint32_t)A[(size_t)i * QO_GROUPS + j] << 12));
  }
  free(cost);
  free(ncost);
  free(M);
  free(A);
  return best;
}

void qo_decode_states(const float* lut0, const float* lut1, const uint16_t* states, float* hatX) { /* :166-172 */
  for (int i = 0; i < QO_STEPS; ++i) {
    hatX[2 * i] = lut0[states[i]];
    hatX[2 * i + 1] = lut1[states[i]];
  }
}

double qo_path_cost(const float* lut0, const float* lut1, const float* X, const uint16_t* states) { /* :174-178 */
  double c = 0;
  for (int i = 0; i < QO_STEPS; ++i) c += sq_err(lut0, lut1, states[i], X[2 * i], X[2 * i + 1]);
  return c;
}

static double quantize_seq_impl(const float* lut0, const float* lut1, const float* X, uint16_t* states, float* hatX,
                                int fast) { /* src/qtip_core.cpp:180-191 */
  float R[QO_SEQ];
  const int sh = QO_SEQ / 4 * 2; /* T // (2V) * V = 128 */
  for (int t = 0; t < QO_SEQ; ++t) R[t] = X[(t - sh + QO_SEQ) % QO_SEQ];
  uint16_t st1[QO_STEPS];
  if (fast) qo_viterbi_fast(lut0, lut1, R, -1, st1);
  else qo_viterbi(lut0, lut1, R, -1, st1);
  int overlap = st1[QO_SEQ / 4] >> QO_KV;
  double c = fast ? qo_viterbi_fast(lut0, lut1, X, overlap, states) : qo_viterbi(lut0, lut1, X, overlap, states);
  if (hatX) qo_decode_states(lut0, lut1, states, hatX);
  return c;
}
double qo_quantize_seq(const float* lut0, const float* lut1, const float* X, uint16_t* states, float* hatX) {
  return quantize_seq_impl(lut0, lut1, X, states, hatX, 0);
}
void qo_quantize_tiles(const float* lut0, const float* lut1, const float* X, long B, uint16_t* states, float* hatX,
                       int threads, int fast) {
  if (threads <= 0) threads = omp_get_max_threads();
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
  for (long b = 0; b < B; ++b)
    quantize_seq_impl(lut0, lut1, X + b * QO_SEQ, states + b * QO_STEPS, hatX ? hatX + b * QO_SEQ : 0, fast);
}

/* ------------------------------------------------------------------ packing, src/qtip_core.cpp:194-253 */
void qo_pack_trellis(const uint16_t* states, long B, uint16_t* packed) {
  for (long b = 0; b < B; ++b) {
    const uint16_t* st = states + b * QO_STEPS;
    uint16_t* out = packed + b * QO_WORDS;
    memset(out, 0, QO_WORDS * 2);
    /* bit stream, MSB first: 16 bits of state 0, then the 4 new bits of each later state; first 512 bits kept */
    int pos = 0;
    for (int i = QO_L - 1; i >= 0; --i, ++pos)
      if (pos < 512 && ((st[0] >> i) & 1)) out[pos >> 4] |= (uint16_t)(1u << (15 - (pos & 15)));
    for (int t = 1; t < QO_STEPS; ++t)
      for (int i = QO_KV - 1; i >= 0; --i, ++pos)
        if (pos < 512 && ((st[t] >> i) & 1)) out[pos >> 4] |= (uint16_t)(1u << (15 - (pos & 15)));
  }
}
void qo_unpack_trellis(const uint16_t* packed, long B, uint16_t* states) {
  for (long b = 0; b < B; ++b) {
    const uint16_t* in = packed + b * QO_WORDS;
    uint16_t* st = states + b * QO_STEPS;
    uint32_t s = 0;
    for (int i = 0; i < QO_L; ++i) s = (s << 1) | ((in[i >> 4] >> (15 - (i & 15))) & 1u);
    st[0] = (uint16_t)s;
    for (int t = 1; t < QO_STEPS; ++t) {
      uint32_t e = 0;
      for (int i = 0; i < QO_KV; ++i) {
        int pos = (QO_L + (t - 1) * QO_KV + i) % 512; /* the stream wraps: tail-biting */
        e = (e << 1) | ((in[pos >> 4] >> (15 - (pos & 15))) & 1u);
      }
      s = ((s << QO_KV) & (QO_STATES - 1)) | e;
      st[t] = (uint16_t)s;
    }
  }
}
int qo_swizzle_for_kernel(const uint16_t* packed, int m, int n, uint16_t* out) { /* :233-243 */
  if (m % 32 || n % 32) return -1;
  long nb = n / 16, M2 = m / 32, N2 = n / 32;
  for (long i0 = 0; i0 < M2; ++i0)
    for (long j0 = 0; j0 < N2; ++j0)
      for (int c = 0; c < 32; ++c)
        for (int j1 = 0; j1 < 2; ++j1)
          for (int i1 = 0; i1 < 2; ++i1)
            out[(((i0 * N2 + j0) * 32 + c) * 2 + j1) * 2 + i1] = packed[((2 * i0 + i1) * nb + 2 * j0 + j1) * 32 + c];
  return 0;
}
int qo_unswizzle_for_kernel(const uint16_t* in, int m, int n, uint16_t* packed) { /* :244-253 */
  if (m % 32 || n % 32) return -1;
  long nb = n / 16, M2 = m / 32, N2 = n / 32;
  for (long i0 = 0; i0 < M2; ++i0)
    for (long j0 = 0; j0 < N2; ++j0)
      for (int c = 0; c < 32; ++c)
        for (int j1 = 0; j1 < 2; ++j1)
          for (int i1 = 0; i1 < 2; ++i1)
            packed[((2 * i0 + i1) * nb + 2 * j0 + j1) * 32 + c] = in[(((i0 * N2 + j0) * 32 + c) * 2 + j1) * 2 + i1];
  return 0;
}

/* ------------------------------------------------------------------ Cholesky / block LDL */
/* Right-looking blocked lower Cholesky in fp64, src/qtip_core.cpp:321-442, with every element formed by the
 * reference's own sequence of operations (its build contracts a * b + c into one fused operation), so that the
 * factor equals the compiled reference's bit for bit; checked against it live and through committed rows of L.
 * Per 256-column panel:
 *   diagonal block, unblocked (:329-343): s = a_ij minus the products l_ip * l_jp, p ascending inside the block;
 *     l_jj = sqrt(s_jj); l_ij = s_ij / l_jj.  The reference's build (GCC -O3) vectorizes these two sums as
 *     in-order reductions, which decides what is fused: over the full groups of four p the products are rounded
 *     on their own and subtracted one after the other; of the len mod 4 terms left, an element below the
 *     diagonal subtracts two as rounded products (if there are two or three) and the last odd one as a fused
 *     multiply-add, the diagonal element takes all of them as fused multiply-adds;
 *   rows below (:376-394): four partial sums, s0 from the element and s1..s3 from zero; the full groups of four
 *     p < j feed s_(p mod 4) = fma(-l_jp, x_p, s_(p mod 4)), leftover p feed s0;
 *     x_j = ((s0 + s1) + (s2 + s3)) * (1 / l_jj);
 *   trailing update (:267-317, :409-427): acc = fma(x_ip, x_jp, acc) for p ascending over the panel from zero, then
 *     c_ij -= acc.
 * Lower triangle in, lower triangle out. */
int qo_cholesky(double* A, int n) {
  enum { NB = 256 };
  double* Lkk = (double*)malloc(sizeof(double) * NB * NB);
  for (int k = 0; k < n; k += NB) {
    const int kb = n - k < NB ? n - k : NB;
    for (int j = k; j < k + kb; ++j) {
      double* aj = A + (long)j * n;
      const int full = k + ((j - k) & ~3), rem = (j - k) & 3;
      double d = aj[j];
      for (int p = k; p < full; p += 4) {
        const double t0 = aj[p] * aj[p], t1 = aj[p + 1] * aj[p + 1], t2 = aj[p + 2] * aj[p + 2],
                     t3 = aj[p + 3] * aj[p + 3];
        d = (((d - t0) - t1) - t2) - t3;
      }
      for (int p = full; p < j; ++p) d = fma(-aj[p], aj[p], d);
      if (!(d > 0)) {
        free(Lkk);
        return 0;
      }
      d = sqrt(d);
      aj[j] = d;
      for (int i = j + 1; i < k + kb; ++i) {
        double* ai = A + (long)i * n;
        double s = ai[j];
        const int unfused = full + (rem >= 2 ? 2 : 0);
        for (int p = k; p < unfused; ++p) {
          const double t = ai[p] * aj[p];
          s -= t;
        }
        if (rem & 1) s = fma(-ai[j - 1], aj[j - 1], s);
        ai[j] = s / d;
      }
    }
    const int r0 = k + kb;
    if (r0 >= n) break;
    for (int j = 0; j < kb; ++j)
      for (int p = 0; p <= j; ++p) Lkk[j * NB + p] = A[(long)(k + j) * n + k + p];
#pragma omp parallel for schedule(dynamic, 8)
    for (int i = r0; i < n; ++i) {
      double* x = A + (long)i * n + k;
      for (int j = 0; j < kb; ++j) {
        const double* lj = Lkk + j * NB;
        double s0 = x[j], s1 = 0, s2 = 0, s3 = 0;
        int p = 0;
        for (; p + 4 <= j; p += 4) {
          s0 = fma(-lj[p], x[p], s0);
          s1 = fma(-lj[p + 1], x[p + 1], s1);
          s2 = fma(-lj[p + 2], x[p + 2], s2);
          s3 = fma(-lj[p + 3], x[p + 3], s3);
        }
        for (; p < j; ++p) s0 = fma(-lj[p], x[p], s0);
        x[j] = ((s0 + s1) + (s2 + s3)) * (1.0 / lj[j]);
      }
    }
#pragma omp parallel for schedule(dynamic, 8)
    for (int i = n - 1; i >= r0; --i) {
      const double* xi = A + (long)i * n + k;
      for (int j = r0; j <= i; ++j) {
        const double* xj = A + (long)j * n + k;
        double acc = 0;
        for (int p = 0; p < kb; ++p) acc = fma(xi[p], xj[p], acc);
        A[(long)i * n + j] -= acc;
      }
    }
  }
  free(Lkk);
  return 1;
}

/* block_LDL(H, 16) followed by zeroing the diagonal blocks, src/qtip_core.cpp:444-487:
 * L = C * blockdiag(C_bb^-1), strictly block-lower, fp32. A (fp64, lower triangle used) is destroyed.
 * The sums are chains of fused multiply-adds, as the reference's build makes them. */
int qo_block_ldl_to_L(double* A, int n, float* L) {
  if (n % 16) return 0;
  if (!qo_cholesky(A, n)) return 0;
  int nb = n / 16;
  double* inv = (double*)malloc(sizeof(double) * (size_t)nb * 256);
  for (int bi = 0; bi < nb; ++bi) {
    double D[16][16], Iv[16][16];
    for (int i = 0; i < 16; ++i)
      for (int j = 0; j < 16; ++j) D[i][j] = j <= i ? A[(long)(bi * 16 + i) * n + bi * 16 + j] : 0.0;
    for (int c = 0; c < 16; ++c)
      for (int i = 0; i < 16; ++i) {
        double s = (i == c) ? 1.0 : 0.0;
        for (int p = 0; p < i; ++p) s = fma(-D[i][p], Iv[p][c], s);
        Iv[i][c] = s / D[i][i];
      }
    for (int i = 0; i < 16; ++i)
      for (int j = 0; j < 16; ++j) inv[(size_t)bi * 256 + i * 16 + j] = Iv[i][j];
  }
  int finite = 1;
  for (int r = 0; r < n; ++r) {
    const double* ar = A + (long)r * n;
    float* lr = L + (long)r * n;
    int rb = r / 16;
    for (int bj = 0; bj < nb; ++bj) {
      float* o = lr + bj * 16;
      if (bj >= rb) {
        memset(o, 0, 16 * sizeof(float));
        continue;
      }
      const double* a = ar + bj * 16;
      const double* iv = inv + (size_t)bj * 256;
      for (int j = 0; j < 16; ++j) {
        double s = 0;
        for (int p = j; p < 16; ++p) s = fma(a[p], iv[p * 16 + j], s);
        o[j] = (float)s;
        if (!isfinite(s)) finite = 0;
      }
    }
  }
  free(inv);
  return finite;
}

/* ------------------------------------------------------------------ LDLQ, tests/test_gpu.cpp:180-225 */
/* WT: n x mt fp64 (already scaled); L: n x n fp32.  hT: n x mt fp64 out; Q[(mt/16)*(n/16)][128]. */
static void quantize_block(const float* lut0, const float* lut1, const double* WX /*16 x mt*/, int mt, int n,
                           int col0, double* hT, uint16_t* Q, int threads) {
  int perm[256];
  qo_perm256(perm, 0);
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
  for (int b = 0; b < mt / 16; ++b) {
    float x[256], h[256];
    uint16_t st[128];
    for (int p = 0; p < 256; ++p) {
      int q = perm[p], r = q >> 4, c = q & 15;
      x[p] = qo_round_fp16((float)WX[(size_t)c * mt + 16 * b + r]);
    }
    quantize_seq_impl(lut0, lut1, x, st, h, 1);
    for (int p = 0; p < 256; ++p) {
      int q = perm[p], r = q >> 4, c = q & 15;
      hT[(size_t)(col0 + c) * mt + 16 * b + r] = h[p];
    }
    memcpy(Q + ((size_t)b * (n / 16) + col0 / 16) * 128, st, 128 * sizeof(uint16_t));
  }
}

static int ldlq_core(const float* lut0, const float* lut1, const double* WT, const float* L, int mt, int n, double* hT,
                     uint16_t* Q, int threads) {
  if (n % 128 || mt % 16) return -1;
  if (threads <= 0) threads = omp_get_max_threads();
  double* prod = (double*)calloc((size_t)n * mt, sizeof(double));
  double* WX = (double*)malloc(sizeof(double) * 16 * (size_t)mt);
  memset(hT, 0, sizeof(double) * (size_t)n * mt);
  for (int cur = n / 16; cur > 0; cur -= 8) {
    int bufend = 16 * cur, c0 = bufend - 128;
    for (int bi = 7; bi >= 0; --bi) {
      int col0 = c0 + 16 * bi;
#pragma omp parallel for schedule(static) num_threads(threads)
      for (int c = 0; c < 16; ++c)
        for (int j = 0; j < mt; ++j) {
          double v = WT[(size_t)(col0 + c) * mt + j] + prod[(size_t)(col0 + c) * mt + j];
          for (int k = col0 + 16; k < bufend; ++k)
            v += (double)L[(size_t)k * n + col0 + c] * (WT[(size_t)k * mt + j] - hT[(size_t)k * mt + j]);
          WX[(size_t)c * mt + j] = v;
        }
      quantize_block(lut0, lut1, WX, mt, n, col0, hT, Q, threads);
    }
#pragma omp parallel for schedule(static) num_threads(threads)
    for (int r = 0; r < c0; ++r)
      for (int k = c0; k < bufend; ++k) {
        double l = L[(size_t)k * n + r];
        if (l == 0) continue;
        for (int j = 0; j < mt; ++j) prod[(size_t)r * mt + j] += l * (WT[(size_t)k * mt + j] - hT[(size_t)k * mt + j]);
      }
  }
  free(prod);
  free(WX);
  return 0;
}

int qo_ldlq(const float* lut0, const float* lut1, const float* Wr, const float* L, int m, int n, float* hatWr,
            uint16_t* Q, int threads) {
  if (m <= 0 || n <= 0) return -1;
  double* WT = (double*)calloc((size_t)n * m, sizeof(double));
  double* hT = (double*)malloc(sizeof(double) * (size_t)n * m);
  if (!WT || !hT) {
    free(WT);
    free(hT);
    return -1;
  }
  for (int i = 0; i < m; ++i)
    for (int j = 0; j < n; ++j) WT[(size_t)j * m + i] = Wr[(size_t)i * n + j];
  int rc = ldlq_core(lut0, lut1, WT, L, m, n, hT, Q, threads);
  if (rc == 0)
    for (int i = 0; i < m; ++i)
      for (int j = 0; j < n; ++j) hatWr[(size_t)i * n + j] = (float)hT[(size_t)j * m + i];
  free(WT);
  free(hT);
  return rc;
}

int qo_ldlq_naive(const float* lut0, const float* lut1, const float* Wr, const float* L, int m, int n, float* hatWr,
                  uint16_t* Q, int threads) {
  if (n % 16 || m % 16) return -1;
  if (threads <= 0) threads = omp_get_max_threads();
  double* WT = (double*)malloc(sizeof(double) * (size_t)n * m);
  double* hT = (double*)calloc((size_t)n * m, sizeof(double));
  double* WX = (double*)malloc(sizeof(double) * 16 * (size_t)m);
  for (int i = 0; i < m; ++i)
    for (int j = 0; j < n; ++j) WT[(size_t)j * m + i] = Wr[(size_t)i * n + j];
  for (int col0 = n - 16; col0 >= 0; col0 -= 16) {
    for (int c = 0; c < 16; ++c)
      for (int j = 0; j < m; ++j) {
        double v = WT[(size_t)(col0 + c) * m + j];
        for (int k = col0 + 16; k < n; ++k)
          v += (double)L[(size_t)k * n + col0 + c] * (WT[(size_t)k * m + j] - hT[(size_t)k * m + j]);
        WX[(size_t)c * m + j] = v;
      }
    quantize_block(lut0, lut1, WX, m, n, col0, hT, Q, threads);
  }
  for (int i = 0; i < m; ++i)
    for (int j = 0; j < n; ++j) hatWr[(size_t)i * n + j] = (float)hT[(size_t)j * m + i];
  free(WT);
  free(hT);
  free(WX);
  return 0;
}

/* ------------------------------------------------------------------ Hessian, src/quantizer.cpp:124-165 */
static void transpose_f32(const float* in, long rows, long cols, long ld_in, float* out, long ld_out) {
  for (long r = 0; r < rows; ++r)
    for (long c = 0; c < cols; ++c) out[c * ld_out + r] = in[r * ld_in + c];
}

int qo_rotate_hessian(const float* H, int n, uint64_t seed, double sigma_reg, float* su, double* creg, float* HRr) {
  qo_rng_t rng;
  rng_init(&rng, seed);
  for (int i = 0; i < n; ++i) su[i] = rng_sign(&rng);
  float* Ht = (float*)malloc(sizeof(float) * (size_t)n * n);
  memcpy(Ht, H, sizeof(float) * (size_t)n * n);
  double dsum = 0;
  for (long i = 0; i < n; ++i) dsum += Ht[i * n + i];
  *creg = sigma_reg * dsum / n;
  for (long i = 0; i < n; ++i) Ht[i * n + i] += (float)*creg;
  for (long r = 0; r < n; ++r)
    for (long c = 0; c < n; ++c) {
      float v = Ht[r * n + c];
      v *= su[r];
      v *= su[c];
      Ht[r * n + c] = v;
    }
  int rc = qo_hadamard_rows_f32(Ht, n, n, n, 1);
  if (rc) {
    free(Ht);
    return rc;
  }
  transpose_f32(Ht, n, n, n, HRr, n);
  rc = qo_hadamard_rows_f32(HRr, n, n, n, 1);
  free(Ht);
  return rc;
}

int qo_ldl_hessian(const float* HRr, int n, float* L) {
  double* A = (double*)malloc(sizeof(double) * (size_t)n * n);
  for (long i = 0; i < n; ++i)
    for (long j = 0; j <= i; ++j) A[i * n + j] = 0.5 * ((double)HRr[i * n + j] + HRr[j * n + i]);
  int ok = qo_block_ldl_to_L(A, n, L);
  free(A);
  return ok ? 0 : -1;
}

/* ------------------------------------------------------------------ proxy */
/* sum_j x_j^T H x_j over the mt columns x_j of X (n x mt, fp64), H n x n fp32 */
static double quad_trace(const double* X, const float* H, int n, int mt, int c0, int mc, int ld, int threads) {
  double tot = 0;
#pragma omp parallel for schedule(static) reduction(+ : tot) num_threads(threads)
  for (int a = 0; a < n; ++a) {
    double* y = (double*)calloc((size_t)mc, sizeof(double));
    for (int b = 0; b < n; ++b) {
      double h = H[(size_t)a * n + b];
      const double* xb = X + (size_t)b * ld + c0;
      for (int j = 0; j < mc; ++j) y[j] += h * xb[j];
    }
    const double* xa = X + (size_t)a * ld + c0;
    double s = 0;
    for (int j = 0; j < mc; ++j) s += xa[j] * y[j];
    tot += s;
    free(y);
  }
  (void)mt;
  return tot;
}

double qo_proxy(const float* W, const float* hatW, const float* H, int m, int n, int threads) {
  if (threads <= 0) threads = omp_get_max_threads();
  double* WT = (double*)malloc(sizeof(double) * (size_t)n * m);
  double* DT = (double*)malloc(sizeof(double) * (size_t)n * m);
  for (int i = 0; i < m; ++i)
    for (int j = 0; j < n; ++j) {
      WT[(size_t)j * m + i] = W[(size_t)i * n + j];
      DT[(size_t)j * m + i] = (double)W[(size_t)i * n + j] - hatW[(size_t)i * n + j];
    }
  double num = quad_trace(DT, H, n, m, 0, m, m, threads), den = quad_trace(WT, H, n, m, 0, m, m, threads);
  free(WT);
  free(DT);
  return num / den;
}

/* ------------------------------------------------------------------ whole group, src/quantizer.cpp:176-346 */
int qo_quantize_group(const float* tlut, int nlin, const float* const* W, const int* m, int n, const float* H,
                      uint64_t seed, double sigma_reg, double scale_override, uint16_t* trellis, uint16_t* su_bf16,
                      float* sv, float* wscale, double* proxy, double* proxy_rot_reg, uint16_t* Q_out, float* WT_out,
                      float* hatWT_out, int threads) {
  if (threads <= 0) threads = omp_get_max_threads();
  if (n % 128) return -1;
  long mt = 0;
  for (int i = 0; i < nlin; ++i) {
    if (m[i] % 32 || n % 32) return -1;
    mt += m[i];
  }
  float* lut0 = (float*)malloc(sizeof(float) * QO_STATES);
  float* lut1 = (float*)malloc(sizeof(float) * QO_STATES);
  double lut_rms = 0;
  qo_build_codebook(tlut, lut0, lut1, 0, &lut_rms);

  float* su = (float*)malloc(sizeof(float) * (size_t)n);
  float* HRr = (float*)malloc(sizeof(float) * (size_t)n * n);
  float* L = (float*)malloc(sizeof(float) * (size_t)n * n);
  double creg = 0;
  int rc = qo_rotate_hessian(H, n, seed, sigma_reg, su, &creg, HRr);
  if (rc == 0) rc = qo_ldl_hessian(HRr, n, L);
  if (rc) {
    free(lut0), free(lut1), free(su), free(HRr), free(L);
    return rc;
  }
  for (int i = 0; i < n; ++i) su_bf16[i] = qo_f32_to_bf16(su[i]);

  float* WT = (float*)malloc(sizeof(float) * (size_t)n * mt);
  long off = 0;
  for (int li = 0; li < nlin; ++li) {
    int ml = m[li];
    qo_rng_t r2;
    rng_init(&r2, seed * 1000003ull + (uint64_t)li + 1);
    for (int i = 0; i < ml; ++i) sv[off + i] = rng_sign(&r2);
    float* Wt = (float*)malloc(sizeof(float) * (size_t)ml * n);
    for (long r = 0; r < ml; ++r)
      for (long c = 0; c < n; ++c) {
        float v = W[li][r * n + c];
        v *= sv[off + r];
        v *= su[c];
        Wt[r * n + c] = v;
      }
    qo_hadamard_rows_f32(Wt, ml, n, n, 1);
    transpose_f32(Wt, ml, n, n, WT + off, mt);
    qo_hadamard_rows_f32(WT + off, n, ml, mt, 1);
    free(Wt);
    double ss = 0;
    for (long r = 0; r < n; ++r)
      for (long c = 0; c < ml; ++c) {
        double v = WT[r * mt + off + c];
        ss += v * v;
      }
    double rms = sqrt(ss / ((double)n * ml));
    wscale[li] = (float)(rms / ((double)(float)lut_rms * scale_override));
    float a = 1.0f / wscale[li];
    for (long r = 0; r < n; ++r)
      for (long c = 0; c < ml; ++c) WT[r * mt + off + c] *= a;
    off += ml;
  }

  double* WTd = (double*)malloc(sizeof(double) * (size_t)n * mt);
  double* hT = (double*)malloc(sizeof(double) * (size_t)n * mt);
  uint16_t* Q = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)(mt / 16) * (n / 16) * 128);
  for (size_t i = 0; i < (size_t)n * mt; ++i) WTd[i] = WT[i];
  rc = ldlq_core(lut0, lut1, WTd, L, (int)mt, n, hT, Q, threads);

  /* proxy in the rotated, scaled domain (Wscale cancels), src/quantizer.cpp:272-301 */
  double* DT = (double*)malloc(sizeof(double) * (size_t)n * mt);
  for (size_t i = 0; i < (size_t)n * mt; ++i) DT[i] = WTd[i] - hT[i];
  off = 0;
  for (int li = 0; li < nlin && rc == 0; ++li) {
    int ml = m[li];
    double den = quad_trace(WTd, HRr, n, (int)mt, (int)off, ml, (int)mt, threads);
    double num = quad_trace(DT, HRr, n, (int)mt, (int)off, ml, (int)mt, threads);
    double wn2 = 0, dn2 = 0;
    for (long r = 0; r < n; ++r)
      for (long c = 0; c < ml; ++c) {
        double w = WTd[r * mt + off + c], d = DT[r * mt + off + c];
        wn2 += w * w;
        dn2 += d * d;
      }
    proxy_rot_reg[li] = num / den;
    proxy[li] = (num - creg * dn2) / (den - creg * wn2);
    /* states -> packed trellis in kernel layout, src/quantizer.cpp:307-320 */
    long nblk = n / 16, ntr = (ml / 16) * nblk;
    const uint16_t* q = Q + (size_t)(off / 16) * nblk * 128;
    uint16_t* packed = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)ntr * QO_WORDS);
    qo_pack_trellis(q, ntr, packed);
    qo_swizzle_for_kernel(packed, ml, n, trellis + (size_t)(off / 16) * nblk * QO_WORDS);
    free(packed);
    off += ml;
  }
  if (Q_out) memcpy(Q_out, Q, sizeof(uint16_t) * (size_t)(mt / 16) * (n / 16) * 128);
  if (WT_out) memcpy(WT_out, WT, sizeof(float) * (size_t)n * mt);
  if (hatWT_out)
    for (size_t i = 0; i < (size_t)n * mt; ++i) hatWT_out[i] = (float)hT[i];
  free(lut0), free(lut1), free(su), free(HRr), free(L), free(WT), free(WTd), free(hT), free(Q), free(DT);
  return rc;
}

/* ================================================================== NVFP4 fallback quantizer */
static unsigned nv_round_even(float v) { /* src/nvfp4.hpp:19-23 */
  const float f = floorf(v), r = v - f;
  unsigned n = (unsigned)f;
  return n + (unsigned)(r > .5f || (r == .5f && (n & 1u)));
}
uint8_t qo_f32_to_fp8e4m3(float x) { /* src/nvfp4.hpp:15-33 */
  const uint8_t sign = signbit(x) ? 128 : 0;
  if (isnan(x)) return (uint8_t)(sign | 127);
  x = fminf(fabsf(x), 448.f);
  if (x < ldexpf(1.f, -6)) return (uint8_t)(sign | nv_round_even(x * 512.f));
  int e;
  const float frac = frexpf(x, &e) * 2;
  unsigned mant = nv_round_even((frac - 1) * 8);
  int ee = e + 6;
  if (mant == 8) {
    mant = 0;
    ++ee;
  }
  unsigned c = ((unsigned)ee << 3) | mant;
  return (uint8_t)(sign | (c < 126u ? c : 126u));
}
float qo_fp8e4m3_to_f32(uint8_t b) { /* src/common.hpp:81-88 */
  const uint32_t s = b >> 7, e = (b >> 3) & 0xf, m = b & 7;
  float v;
  if (e == 0) v = ldexpf((float)m, -9);
  else if (e == 15 && m == 7) v = NAN;
  else v = ldexpf((float)(m | 8), (int)e - 10);
  return s ? -v : v;
}
static const float kNvLevels[8] = {0, .5f, 1, 1.5f, 2, 3, 4, 6};
/* nearest E2M1 magnitude code, ties to the even code (src/nvfp4.cpp:27-38, src/nvfp4_gpu.hip:47-60) */
static int nv_fp4_mag(float a) {
  float best = INFINITY;
  int code = 0;
  for (int i = 0; i < 8; ++i) {
    const float e = fabsf(a - kNvLevels[i]);
    if (e < best || (e == best && (i % 2 == 0))) {
      best = e;
      code = i;
    }
  }
  return code;
}
int qo_nvfp4_quantize(const float* w, int m, int n, uint8_t* packed, uint8_t* scales, float* global) {
  if (m <= 0 || n <= 0 || n % 16) return -1;
  const size_t numel = (size_t)m * n;
  float maximum = 0;
  for (size_t i = 0; i < numel; ++i) maximum = fmaxf(maximum, fabsf(w[i]));
  const float g = maximum ? maximum / (448.f * 6) : 1.f;
  *global = g;
  for (size_t b = 0; b < numel / 16; ++b) {
    float mx = 0;
    for (int j = 0; j < 16; ++j) mx = fmaxf(mx, fabsf(w[b * 16 + j]));
    const uint8_t sc = qo_f32_to_fp8e4m3(mx / (6 * g));
    scales[b] = sc;
    const float scale = qo_fp8e4m3_to_f32(sc) * g;
    for (int j = 0; j < 16; j += 2) {
      const float x0 = scale ? w[b * 16 + j] / scale : 0, x1 = scale ? w[b * 16 + j + 1] / scale : 0;
      const uint8_t c0 = (uint8_t)(nv_fp4_mag(fabsf(x0)) | (signbit(x0) ? 8 : 0));
      const uint8_t c1 = (uint8_t)(nv_fp4_mag(fabsf(x1)) | (signbit(x1) ? 8 : 0));
      packed[b * 8 + j / 2] = (uint8_t)(c0 | (c1 << 4));
    }
  }
  return 0;
}
void qo_nvfp4_dequantize(const uint8_t* packed, const uint8_t* scales, float global, int m, int n, float* out) {
  const size_t numel = (size_t)m * n;
  for (size_t i = 0; i < numel; ++i) {
    const uint8_t code = (packed[i / 2] >> (i % 2 * 4)) & 15;
    const float s = qo_fp8e4m3_to_f32(scales[i / 16]);
    const float v = (code & 8 ? -1.f : 1.f) * kNvLevels[code & 7];
    out[i] = qo_bf16_to_f32(qo_f32_to_bf16(v * s * global));
  }
}
double qo_nvfp4_proxy_error(const float* w, const float* what, int m, int n, const float* H) {
  double total = 0;
#pragma omp parallel for reduction(+ : total) schedule(static)
  for (int r = 0; r < m; ++r) {
    double* e = (double*)malloc(sizeof(double) * (size_t)n);
    for (int j = 0; j < n; ++j) e[j] = (double)w[(size_t)r * n + j] - what[(size_t)r * n + j];
    if (!H) {
      for (int j = 0; j < n; ++j) total += e[j] * e[j];
    } else {
      for (int i = 0; i < n; ++i) {
        double acc = 0;
        for (int j = 0; j < n; ++j) acc += (double)H[(size_t)i * n + j] * e[j];
        total += e[i] * acc;
      }
    }
    free(e);
  }
  return total / m;
}
int qo_nvfp4_prepare(const float* H, int n, double sigma_reg, int calibrate, float* L, float* dw) {
  double dsum = 0;
  for (int i = 0; i < n; ++i) dsum += H[(size_t)i * n + i];
  const double creg = sigma_reg * dsum / n;
  if (!calibrate) {
    for (int i = 0; i < n; ++i) dw[i] = (float)(H[(size_t)i * n + i] + creg);
    return 0;
  }
  double* A = (double*)malloc(sizeof(double) * (size_t)n * n);
  for (long i = 0; i < n; ++i)
    for (long j = 0; j <= i; ++j)
      A[(size_t)i * n + j] = 0.5 * ((double)H[(size_t)i * n + j] + H[(size_t)j * n + i]) + (i == j ? creg : 0.0);
  if (!qo_cholesky(A, n)) {
    free(A);
    return -1;
  }
  memset(L, 0, sizeof(float) * (size_t)n * n);
  for (long j = 0; j < n; ++j) {
    const double d = A[(size_t)j * n + j];
    dw[j] = (float)(d * d);
    for (long i = j + 1; i < n; ++i) L[(size_t)i * n + j] = (float)(A[(size_t)i * n + j] / d);
  }
  free(A);
  return 0;
}
/* one row of one 16-column block: nv_block_kernel, src/nvfp4_gpu.hip:66-158 */
static void nv_block_row(const float* w16, const float* f16, const float Lb[16][16], const float* Dw, float global,
                         int calibrate, int search, uint8_t* nib, uint8_t* scale_out, float* err_out) {
  float w[16], base[16], amax = 0;
  for (int k = 0; k < 16; ++k) {
    w[k] = w16[k];
    base[k] = w[k] + (calibrate ? f16[k] : 0.f);
    amax = fmaxf(amax, fabsf(calibrate ? base[k] : w[k]));
  }
  unsigned cand[11];
  int nc = 0;
  const unsigned c1 = qo_f32_to_fp8e4m3(amax / (6.f * global)) & 127u;
  cand[nc++] = c1;
  if (search) {
    static const float g[8] = {0.70f, 0.75f, 0.80f, 0.85f, 0.90f, 0.95f, 1.00f, 1.05f};
    for (int i = 0; i < 8; ++i) cand[nc++] = qo_f32_to_fp8e4m3(amax * g[i] / (6.f * global)) & 127u;
    cand[nc++] = c1 > 0 ? c1 - 1 : 0;
    cand[nc++] = c1 < 126 ? c1 + 1 : 126;
  }
  float best_cost = INFINITY;
  unsigned best = c1;
  for (int ci = 0; ci < nc; ++ci) {
    const float sd = qo_fp8e4m3_to_f32((uint8_t)cand[ci]), scale = sd * global;
    float err[16], cost = 0;
    for (int k = 15; k >= 0; --k) {
      float t = base[k];
      if (calibrate)
        for (int j = k + 1; j < 16; ++j) t = fmaf(err[j], Lb[j][k], t);
      const float x = scale != 0.f ? t / scale : 0.f;
      const int code = nv_fp4_mag(fabsf(x));
      const float q = qo_bf16_to_f32(qo_f32_to_bf16((x < 0 ? -1.f : 1.f) * kNvLevels[code] * sd * global));
      cost = fmaf(Dw[k] * (t - q), t - q, cost);
      err[k] = w[k] - q;
    }
    if (cost < best_cost) {
      best_cost = cost;
      best = cand[ci];
    }
  }
  const float sd = qo_fp8e4m3_to_f32((uint8_t)best), scale = sd * global;
  for (int k = 15; k >= 0; --k) {
    float t = base[k];
    if (calibrate)
      for (int j = k + 1; j < 16; ++j) t = fmaf(err_out[j], Lb[j][k], t);
    const float x = scale != 0.f ? t / scale : 0.f;
    const int code = nv_fp4_mag(fabsf(x));
    const float q = qo_bf16_to_f32(qo_f32_to_bf16((x < 0 ? -1.f : 1.f) * kNvLevels[code] * sd * global));
    err_out[k] = w[k] - q;
    nib[k] = (uint8_t)(code | (signbit(x) ? 8 : 0));
  }
  *scale_out = (uint8_t)best;
}
void qo_nvfp4_blocks(const float* w, int m, int n, const float* L, const float* dw, float global, int calibrate,
                     int search, uint8_t* packed, uint8_t* scales) {
  const int cal = calibrate && L != NULL;
  float* F = cal ? (float*)calloc((size_t)m * n, sizeof(float)) : NULL;
  float* E = (float*)malloc(sizeof(float) * (size_t)m * 16);
  for (int c0 = n - 16; c0 >= 0; c0 -= 16) {
    float Lb[16][16], Dw[16];
    for (int a = 0; a < 16; ++a) {
      Dw[a] = dw ? dw[c0 + a] : 1.f;
      for (int b = 0; b < 16; ++b) Lb[a][b] = cal ? L[(size_t)(c0 + a) * n + c0 + b] : 0.f;
    }
#pragma omp parallel for schedule(static)
    for (int r = 0; r < m; ++r) {
      uint8_t nib[16], sc;
      nv_block_row(w + (size_t)r * n + c0, cal ? F + (size_t)r * n + c0 : NULL, Lb, Dw, global, cal, search, nib, &sc,
                   E + (size_t)r * 16);
      for (int k = 0; k < 16; k += 2) packed[(size_t)r * (n / 2) + (c0 + k) / 2] = (uint8_t)(nib[k] | (nib[k + 1] << 4));
      scales[(size_t)r * (n / 16) + c0 / 16] = sc;
    }
    if (cal && c0 > 0) { /* nv_feedback_kernel: F[r][col] += sum_j E[r][j] * L[c0 + j][col], col < c0 */
#pragma omp parallel for schedule(static)
      for (int r = 0; r < m; ++r)
        for (int col = 0; col < c0; ++col) {
          float acc = 0;
          for (int j = 0; j < 16; ++j) acc = fmaf(E[(size_t)r * 16 + j], L[(size_t)(c0 + j) * n + col], acc);
          F[(size_t)r * n + col] += acc;
        }
    }
  }
  free(E);
  free(F);
}
