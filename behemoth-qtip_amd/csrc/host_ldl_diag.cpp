// Diagonal block of the host fp64 Cholesky, in the order of operations of the reference's unblocked loop
// (src/qtip_core.cpp:329-343) AS ITS BUILD EVALUATES IT.  GCC -O3 vectorizes the two inner sums of that loop as
// in-order reductions, which splits every chain s -= l_ip * l_jp (p ascending, len = j terms inside the block) into
//   * the full groups of four p: the four products are rounded on their own, then subtracted one after the other;
//   * what is left (len mod 4 terms), for an element below the diagonal: two terms -> both rounded products, three
//     -> two rounded products then one fused multiply-add, one -> one fused multiply-add;
//   * what is left, for the diagonal element: every term a fused multiply-add.
// The factor only equals the compiled reference's bit for bit if the same operations are fused here, so this file is
// built with -ffp-contract=off and says which ones are.  The chains of the rows i > j of a column run 8 (or 4) rows
// to a vector on a transposed copy of the block; all rows of a column have the same length of chain, so the pattern
// is uniform over the lanes.
#include <immintrin.h>

#include <cmath>
#include <cstddef>

namespace qtipmi {

// T: scratch of kb * ldt doubles, ldt >= kb rounded up to 32; T[p * ldt + i] = l_ip.  The lanes of rows i <= j carry
// values that no later column reads.  false if the block is not positive definite.
#define QTIP_FACTOR_DIAG(NAME, VW, VT, LOADU, STOREU, SET1, MUL, SUB, FNMADD)                                  \
  bool NAME(double* __restrict__ A, long ld, int kb, double* __restrict__ T, int ldt) {                        \
    for (int p = 0; p < kb; ++p) {                                                                             \
      for (int i = 0; i < p; ++i) T[size_t(p) * ldt + i] = 0.0;                                                \
      for (int i = p; i < kb; ++i) T[size_t(p) * ldt + i] = A[long(i) * ld + p];                               \
      for (int i = kb; i < ldt; ++i) T[size_t(p) * ldt + i] = 0.0;                                             \
    }                                                                                                          \
    for (int j = 0; j < kb; ++j) {                                                                             \
      double* tj = T + size_t(j) * ldt;                                                                        \
      const int full = j & ~3, rem = j & 3;                                                                    \
      /* the diagonal element */                                                                               \
      double d = tj[j];                                                                                        \
      for (int p = 0; p < full; p += 4) {                                                                      \
        const double l0 = T[size_t(p) * ldt + j], l1 = T[size_t(p + 1) * ldt + j],                             \
                     l2 = T[size_t(p + 2) * ldt + j], l3 = T[size_t(p + 3) * ldt + j];                         \
        const double t0 = l0 * l0, t1 = l1 * l1, t2 = l2 * l2, t3 = l3 * l3;                                   \
        d = (((d - t0) - t1) - t2) - t3;                                                                       \
      }                                                                                                        \
      for (int p = full; p < j; ++p) {                                                                         \
        const double l = T[size_t(p) * ldt + j];                                                               \
        d = __builtin_fma(-l, l, d);                                                                           \
      }                                                                                                        \
      if (!(d > 0) || !std::isfinite(d)) return false;                                                         \
      d = std::sqrt(d);                                                                                        \
      /* the rows below it, four vectors of rows in flight */                                                  \
      for (int i0 = ((j + 1) / (4 * VW)) * (4 * VW); i0 < kb; i0 += 4 * VW) {                                  \
        VT a0 = LOADU(tj + i0), a1 = LOADU(tj + i0 + VW), a2 = LOADU(tj + i0 + 2 * VW),                        \
           a3 = LOADU(tj + i0 + 3 * VW);                                                                       \
        const int unfused = full + (rem >= 2 ? 2 : 0);                                                         \
        for (int p = 0; p < unfused; ++p) {                                                                    \
          const double* tp = T + size_t(p) * ldt;                                                              \
          const VT l = SET1(tp[j]);                                                                            \
          a0 = SUB(a0, MUL(l, LOADU(tp + i0)));                                                                \
          a1 = SUB(a1, MUL(l, LOADU(tp + i0 + VW)));                                                           \
          a2 = SUB(a2, MUL(l, LOADU(tp + i0 + 2 * VW)));                                                       \
          a3 = SUB(a3, MUL(l, LOADU(tp + i0 + 3 * VW)));                                                       \
        }                                                                                                      \
        if (rem & 1) {                                                                                         \
          const double* tp = T + size_t(j - 1) * ldt;                                                          \
          const VT l = SET1(tp[j]);                                                                            \
          a0 = FNMADD(l, LOADU(tp + i0), a0);                                                                  \
          a1 = FNMADD(l, LOADU(tp + i0 + VW), a1);                                                             \
          a2 = FNMADD(l, LOADU(tp + i0 + 2 * VW), a2);                                                         \
          a3 = FNMADD(l, LOADU(tp + i0 + 3 * VW), a3);                                                         \
        }                                                                                                      \
        STOREU(tj + i0, a0);                                                                                   \
        STOREU(tj + i0 + VW, a1);                                                                              \
        STOREU(tj + i0 + 2 * VW, a2);                                                                          \
        STOREU(tj + i0 + 3 * VW, a3);                                                                          \
      }                                                                                                        \
      tj[j] = d;                                                                                               \
      for (int i = j + 1; i < kb; ++i) tj[i] = tj[i] / d;                                                      \
    }                                                                                                          \
    for (int p = 0; p < kb; ++p)                                                                               \
      for (int i = p; i < kb; ++i) A[long(i) * ld + p] = T[size_t(p) * ldt + i];                               \
    return true;                                                                                               \
  }

__attribute__((target("avx512f")))
QTIP_FACTOR_DIAG(factor_diag_avx512, 8, __m512d, _mm512_loadu_pd, _mm512_storeu_pd, _mm512_set1_pd, _mm512_mul_pd,
                 _mm512_sub_pd, _mm512_fnmadd_pd)
QTIP_FACTOR_DIAG(factor_diag_avx2, 4, __m256d, _mm256_loadu_pd, _mm256_storeu_pd, _mm256_set1_pd, _mm256_mul_pd,
                 _mm256_sub_pd, _mm256_fnmadd_pd)
#undef QTIP_FACTOR_DIAG

}  // namespace qtipmi
