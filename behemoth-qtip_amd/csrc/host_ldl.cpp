// Host-side fp64 block LDL of the rotated Hessian (the reference keeps this step in fp64 on the CPU:
// ldl_hessian, src/quantizer.cpp:154-165; block_ldl_to_L / cholesky_inplace, src/qtip_core.cpp:321-487).
//
//   A = C C^T (lower Cholesky, fp64)  ->  L = C * blockdiag(C_bb^-1) with the 16x16 diagonal blocks and the
//   upper triangle zeroed, stored as fp32.
//
// The factor is the reference's bit for bit, which fixes the order of operations of every element (the schedule,
// the register blocking and the data layout are this file's own):
//   * right-looking panels of width NB = 256;
//   * diagonal block: left-looking, s = a_ij minus the products l_ip * l_jp for p ascending inside the block, fused
//     or not as the reference's build has them (host_ldl_diag.cpp), sqrt, division by the square root
//     (src/qtip_core.cpp:329-343);
//   * rows below the block: x_j = ((s0 + s1) + (s2 + s3)) * (1 / l_jj), where s0 starts at the element, s1..s3 at zero,
//     s_(p mod 4) = fma(-l_jp, x_p, s_(p mod 4)) over the full groups of four p < j and the leftover p go to s0
//     (src/qtip_core.cpp:376-394);
//   * trailing update: c -= acc with acc one chain fma(x_ip, x_jp, acc), p ascending over the panel from zero
//     (src/qtip_core.cpp:267-317).
// Here the rows
// below are solved in chunks of NR rows held transposed, and the trailing symmetric update runs as a packed
// register-blocked rank-NB kernel over lower-triangular tiles handed out dynamically to a team of host threads
// (host_team.hpp).  The kernels are written with GCC vector extensions and compiled twice (AVX2 baseline, AVX-512
// clone); the clone is picked at run time so one binary serves any x86-64-v3 host.  Built with -ffp-contract=fast:
// every a * b + c below is one fused operation.
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstring>
#include <memory>
#include <thread>
#include <vector>

#include "host_team.hpp"
#include "qtip_internal.hpp"

namespace qtipmi {
namespace {


// The team belongs to the calling thread (the factorization may run on a side thread while another thread does
// other work with a team of its own) and lives until that thread ends or asks for another size.
HostTeam& team_of_this_thread(int threads) {
  if (threads <= 0) threads = int(std::thread::hardware_concurrency());
  if (threads <= 0) threads = 1;
  static thread_local std::unique_ptr<HostTeam> team;
  if (!team || team->size() != threads) team.reset(new HostTeam(threads));
  return *team;
}

typedef double v8d __attribute__((vector_size(64), aligned(8)));
typedef double v4d __attribute__((vector_size(32), aligned(8)));

#ifndef QTIP_LDL_NB
#define QTIP_LDL_NB 256  // the reference's panel width: part of the factor's bits
#endif
#ifndef QTIP_LDL_TILE
#define QTIP_LDL_TILE 384
#endif
constexpr int NB = QTIP_LDL_NB;      // panel width
constexpr int TILE = QTIP_LDL_TILE;  // rows / columns of one trailing-update task (multiple of every MR and NR below)

// ---- rank-kc update of an MR x NR tile: Cij -= sum_p a[p][i] * b[p][j], a packed [kc][MR], b packed [kc][NR]
// AVX-512: 8 x 24 (24 accumulators of 8 doubles, named so that they stay in registers)
#define QTIP_ROWS8(X) X(0) X(1) X(2) X(3) X(4) X(5) X(6) X(7)
#define QTIP_ROWS4(X) X(0) X(1) X(2) X(3)
__attribute__((target("avx512f"))) static void micro_8x24(int kc, const double* __restrict__ a,
                                                          const double* __restrict__ b, double* __restrict__ C,
                                                          long ldc, int mr, int nr) {
  const v8d z = {0, 0, 0, 0, 0, 0, 0, 0};
#define QTIP_DECL(i) v8d c##i##0 = z, c##i##1 = z, c##i##2 = z;
  QTIP_ROWS8(QTIP_DECL)
#undef QTIP_DECL
  for (int p = 0; p < kc; ++p) {
    const v8d b0 = *reinterpret_cast<const v8d*>(b + p * 24), b1 = *reinterpret_cast<const v8d*>(b + p * 24 + 8),
              b2 = *reinterpret_cast<const v8d*>(b + p * 24 + 16);
#define QTIP_FMA(i)                   \
  {                                   \
    const double ai = a[p * 8 + i];   \
    c##i##0 += ai * b0;               \
    c##i##1 += ai * b1;               \
    c##i##2 += ai * b2;               \
  }
    QTIP_ROWS8(QTIP_FMA)
#undef QTIP_FMA
  }
  if (mr == 8 && nr == 24) {
#define QTIP_STORE(i)                                   \
  {                                                     \
    double* ci = C + i * ldc;                           \
    *reinterpret_cast<v8d*>(ci) -= c##i##0;             \
    *reinterpret_cast<v8d*>(ci + 8) -= c##i##1;         \
    *reinterpret_cast<v8d*>(ci + 16) -= c##i##2;        \
  }
    QTIP_ROWS8(QTIP_STORE)
#undef QTIP_STORE
  } else {
    v8d t[8][3];
#define QTIP_SPILL(i) t[i][0] = c##i##0, t[i][1] = c##i##1, t[i][2] = c##i##2;
    QTIP_ROWS8(QTIP_SPILL)
#undef QTIP_SPILL
    for (int i = 0; i < mr; ++i)
      for (int j = 0; j < nr; ++j) C[i * ldc + j] -= t[i][j >> 3][j & 7];
  }
}
// AVX2: 4 x 12
static void micro_4x12(int kc, const double* __restrict__ a, const double* __restrict__ b, double* __restrict__ C,
                       long ldc, int mr, int nr) {
  const v4d z = {0, 0, 0, 0};
#define QTIP_DECL(i) v4d c##i##0 = z, c##i##1 = z, c##i##2 = z;
  QTIP_ROWS4(QTIP_DECL)
#undef QTIP_DECL
  for (int p = 0; p < kc; ++p) {
    const v4d b0 = *reinterpret_cast<const v4d*>(b + p * 12), b1 = *reinterpret_cast<const v4d*>(b + p * 12 + 4),
              b2 = *reinterpret_cast<const v4d*>(b + p * 12 + 8);
#define QTIP_FMA(i)                   \
  {                                   \
    const double ai = a[p * 4 + i];   \
    c##i##0 += ai * b0;               \
    c##i##1 += ai * b1;               \
    c##i##2 += ai * b2;               \
  }
    QTIP_ROWS4(QTIP_FMA)
#undef QTIP_FMA
  }
  v4d t[4][3];
#define QTIP_SPILL(i) t[i][0] = c##i##0, t[i][1] = c##i##1, t[i][2] = c##i##2;
  QTIP_ROWS4(QTIP_SPILL)
#undef QTIP_SPILL
  for (int i = 0; i < mr; ++i)
    for (int j = 0; j < nr; ++j) C[i * ldc + j] -= t[i][j >> 2][j & 3];
}

// ---- panel solve  X * L11^T = A21 on a chunk of NRC rows held transposed, x[p][NRC] (the layout of one packed
// B micro-panel), in the order given at the top of the file: four partial sums per element, the lanes are rows.
#define QTIP_TRI_SOLVE(NAME, VT, VW, NRC)                                                                      \
  static void NAME(int nb, const double* __restrict__ L11, int ldl, const double* __restrict__ rdiag,          \
                   double* __restrict__ x) {                                                                   \
    constexpr int NV = NRC / VW;                                                                               \
    for (int j = 0; j < nb; ++j) {                                                                             \
      VT s0[NV], s1[NV], s2[NV], s3[NV];                                                                       \
      VT* xj = reinterpret_cast<VT*>(x + size_t(j) * NRC);                                                     \
      for (int v = 0; v < NV; ++v) s0[v] = xj[v], s1[v] = s2[v] = s3[v] = VT{};                                \
      const double* lj = L11 + size_t(j) * ldl;                                                                \
      int p = 0;                                                                                               \
      for (; p + 4 <= j; p += 4) {                                                                             \
        const VT* xp = reinterpret_cast<const VT*>(x + size_t(p) * NRC);                                       \
        const double l0 = lj[p], l1 = lj[p + 1], l2 = lj[p + 2], l3 = lj[p + 3];                               \
        for (int v = 0; v < NV; ++v) {                                                                         \
          s0[v] -= l0 * xp[v];                                                                                 \
          s1[v] -= l1 * xp[NV + v];                                                                            \
          s2[v] -= l2 * xp[2 * NV + v];                                                                        \
          s3[v] -= l3 * xp[3 * NV + v];                                                                        \
        }                                                                                                      \
      }                                                                                                        \
      for (; p < j; ++p) {                                                                                     \
        const VT* xp = reinterpret_cast<const VT*>(x + size_t(p) * NRC);                                       \
        const double l0 = lj[p];                                                                               \
        for (int v = 0; v < NV; ++v) s0[v] -= l0 * xp[v];                                                      \
      }                                                                                                        \
      const double rd = rdiag[j];                                                                              \
      for (int v = 0; v < NV; ++v) xj[v] = ((s0[v] + s1[v]) + (s2[v] + s3[v])) * rd;                           \
    }                                                                                                          \
  }
__attribute__((target("avx512f"))) QTIP_TRI_SOLVE(tri_solve_24, v8d, 8, 24)
QTIP_TRI_SOLVE(tri_solve_12, v4d, 4, 12)
#undef QTIP_TRI_SOLVE

// ---- one row of L over nblk 16-column blocks: out[16 b + j] = float(sum_p a[16 b + p] * inv_b[p][j]), p = j .. 15,
// every sum one fused chain over ascending p from zero (src/qtip_core.cpp:473-483).  The lanes are the 16 values of
// j: inv_b is lower triangular with +0 above the diagonal, so a lane j > p adds a zero product to its zero and its
// chain is the scalar one.  false if a sum is not finite.
typedef float v8f __attribute__((vector_size(32), aligned(4)));
typedef float v4f __attribute__((vector_size(16), aligned(4)));
#define QTIP_ASSEMBLE_ROW(NAME, VT, FT, VW)                                                                    \
  static bool NAME(const double* __restrict__ a, const double* __restrict__ inv, int nblk, float* __restrict__ out) { \
    constexpr int NV = 16 / VW;                                                                                \
    VT chk[NV];                                                                                                \
    for (int v = 0; v < NV; ++v) chk[v] = VT{};                                                                \
    for (int b = 0; b < nblk; ++b) {                                                                           \
      const double* ab = a + b * 16;                                                                           \
      const double* iv = inv + size_t(b) * 256;                                                                \
      VT s[NV];                                                                                                \
      for (int v = 0; v < NV; ++v) s[v] = VT{};                                                                \
      for (int p = 0; p < 16; ++p) {                                                                           \
        const double ap = ab[p];                                                                               \
        for (int v = 0; v < NV; ++v) s[v] += ap * *reinterpret_cast<const VT*>(iv + p * 16 + v * VW);          \
      }                                                                                                        \
      for (int v = 0; v < NV; ++v) {                                                                           \
        *reinterpret_cast<FT*>(out + b * 16 + v * VW) = __builtin_convertvector(s[v], FT);                     \
        chk[v] += s[v] * 0.0; /* NaN as soon as a sum is infinite or NaN */                                    \
      }                                                                                                        \
    }                                                                                                          \
    double c = 0;                                                                                              \
    for (int v = 0; v < NV; ++v)                                                                               \
      for (int l = 0; l < VW; ++l) c += chk[v][l];                                                             \
    return std::isfinite(c);                                                                                   \
  }
__attribute__((target("avx512f"))) QTIP_ASSEMBLE_ROW(assemble_row_avx512, v8d, v8f, 8)
QTIP_ASSEMBLE_ROW(assemble_row_avx2, v4d, v4f, 4)
#undef QTIP_ASSEMBLE_ROW

}  // namespace
// lower Cholesky of the kb x kb diagonal block at A (row stride ld) (host_ldl_diag.cpp, built without contraction: it
// has to say which of its operations are fused); T: scratch of kb * ldt doubles, ldt >= kb rounded up to 32
bool factor_diag_avx512(double* A, long ld, int kb, double* T, int ldt);
bool factor_diag_avx2(double* A, long ld, int kb, double* T, int ldt);
namespace {

struct Kernels {
  int MR, NR;
  void (*micro)(int, const double*, const double*, double*, long, int, int);
  void (*tri_solve)(int, const double*, int, const double*, double*);
  bool (*factor_diag)(double*, long, int, double*, int);
  bool (*assemble_row)(const double*, const double*, int, float*);
};
static Kernels pick_kernels() {
  __builtin_cpu_init();
  if (__builtin_cpu_supports("avx512f")) return Kernels{8, 24, micro_8x24, tri_solve_24, factor_diag_avx512, assemble_row_avx512};
  return Kernels{4, 12, micro_4x12, tri_solve_12, factor_diag_avx2, assemble_row_avx2};
}

// Lower Cholesky of the n x n matrix at A (row stride ld) by right-looking panels of width NBT, shared out over the
// team.
// assist: the trailing matrix lives elsewhere.  Before a panel is factored its columns, rows k .. n-1, are fetched
// into a buffer of row stride kb; after the solve the buffer holds the final columns of C and is handed back, and
// whoever holds the trailing matrix applies the rank-kb update (every element one chain
// acc = fma(x_ip, x_jp, acc), p ascending from zero, then c -= acc, as the micro-kernels here do).
template <int NBT, int TILET>
bool cholesky_panels(double* A, long ld, int n, HostTeam* team, PanelAssist* assist = nullptr) {
  const Kernels kn = pick_kernels();
  const int MR = kn.MR, NR = kn.NR;
  constexpr int LDT = (NBT + 31) / 32 * 32;
  std::vector<double> L11(static_cast<size_t>(NBT) * NBT, 0.0), rdiag(static_cast<size_t>(NBT), 0.0),
      diagT(static_cast<size_t>(NBT) * LDT);
  // packed copies of the solved panel (A side: MR-row micro-panels, B side: NR-row micro-panels), first panel largest
  const size_t capA = size_t((n + MR - 1) / MR) * MR * NBT, capB = size_t((n + NR - 1) / NR) * NR * NBT;
  HostScratch packs((capA + capB) * sizeof(double));
  double* const packA = static_cast<double*>(packs.get());
  double* const packB = packA + capA;
  for (int k = 0; k < n; k += NBT) {
    const int kb = std::min(NBT, n - k);
    // the panel: diagonal block at Ap, the rows below follow with stride ldp
    double* Ap = assist ? assist->fetch(k, kb) : A + long(k) * ld + k;
    const long ldp = assist ? kb : ld;
    if (!kn.factor_diag(Ap, ldp, kb, diagT.data(), LDT)) return false;
    if (assist) assist->factored(k, kb, Ap, ldp);
    const int r0 = k + kb, nr = n - r0;
    if (nr <= 0) {
      if (assist) assist->solved(k, kb, Ap);
      break;
    }
    for (int j = 0; j < kb; ++j) {
      for (int p = 0; p < kb; ++p) L11[size_t(j) * kb + p] = p <= j ? Ap[long(j) * ldp + p] : 0.0;
      rdiag[j] = 1.0 / L11[size_t(j) * kb + j];
    }
    const int nPA = (nr + MR - 1) / MR, nPB = (nr + NR - 1) / NR;
    // only the padding rows of the last micro-panels need zeroing
    for (int i = nr; i < nPA * MR; ++i)
      for (int p = 0; p < kb; ++p) packA[size_t(i / MR) * MR * kb + size_t(p) * MR + (i % MR)] = 0.0;
    for (int i = nr; i < nPB * NR; ++i)
      for (int p = 0; p < kb; ++p) packB[size_t(i / NR) * NR * kb + size_t(p) * NR + (i % NR)] = 0.0;
    // panel solve in place in the packed B micro-panels (one chunk = NR rows), then write back and pack the A side
    auto solve_chunk = [&](long gl) {
      const int g = int(gl);
      const int rb = g * NR, rows = std::min(NR, nr - rb);
      double* x = packB + size_t(g) * NR * kb;  // [p][NR], rows beyond `rows` stay zero
      for (int r = 0; r < rows; ++r) {
        const double* src = Ap + long(kb + rb + r) * ldp;
        for (int p = 0; p < kb; ++p) x[size_t(p) * NR + r] = src[p];
      }
      kn.tri_solve(kb, L11.data(), kb, rdiag.data(), x);
      for (int r = 0; r < rows; ++r) {
        const int i = rb + r;
        double* dst = Ap + long(kb + i) * ldp;
        if (assist) {  // the update runs elsewhere: no A-side pack
          for (int p = 0; p < kb; ++p) dst[p] = x[size_t(p) * NR + r];
          continue;
        }
        double* pa = packA + size_t(i / MR) * MR * kb + (i % MR);
        for (int p = 0; p < kb; ++p) {
          const double v = x[size_t(p) * NR + r];
          dst[p] = v;
          pa[size_t(p) * MR] = v;
        }
      }
    };
    auto solve_and_hand_over = [&](long gl) {
      solve_chunk(gl);
      const int rb = int(gl) * NR;
      assist->rows_solved(k, kb, r0 + rb, std::min(NR, nr - rb), Ap + long(kb + rb) * ldp, ldp);
    };
    if (team && assist) team->parallel_for(nPB, 2, solve_and_hand_over);
    else if (team) team->parallel_for(nPB, 2, solve_chunk);
    else
      for (long gl = 0; gl < nPB; ++gl) assist ? solve_and_hand_over(gl) : solve_chunk(gl);
    if (assist) {
      assist->solved(k, kb, Ap);
      continue;
    }
    // trailing update of the lower triangle, tiles (bi, bj <= bi) largest rows first
    const int nT = (nr + TILET - 1) / TILET;
    const long ntask = long(nT) * (nT + 1) / 2;
    auto update_tile = [&](long task) {
      // enumerate from the bottom row block upwards: row block bi has bi+1 tiles
      long rem = task;
      int bi = nT - 1;
      while (rem > bi) {
        rem -= bi + 1;
        --bi;
      }
      const int bj = int(rem);
      const int i0 = bi * TILET, i1 = std::min(nr, i0 + TILET), j0 = bj * TILET, j1 = std::min(nr, j0 + TILET);
      for (int jj = j0; jj < j1; jj += NR) {
        const double* pb = packB + size_t(jj / NR) * NR * kb;
        const int nrr = std::min(NR, nr - jj);
        for (int ii = i0; ii < i1; ii += MR) {
          if (jj > ii + MR - 1) continue;  // micro tile entirely above the diagonal
          const int mrr = std::min(MR, nr - ii);
          kn.micro(kb, packA + size_t(ii / MR) * MR * kb, pb, A + long(r0 + ii) * ld + r0 + jj, ld, mrr, nrr);
        }
      }
    };
    if (team) team->parallel_for(ntask, 1, update_tile);
    else
      for (long task = 0; task < ntask; ++task) update_tile(task);
  }
  return true;
}

}  // namespace

bool cholesky_lower_host(double* A, int n, int threads) {
  HostTeam& team = team_of_this_thread(threads);
  return cholesky_panels<NB, TILE>(A, n, n, &team);
}

// inverse of every 16 x 16 lower-triangular diagonal block b of C (column by column, forward substitution): Cp holds
// the rows of the first diagonal block onwards, inv receives nbp blocks of 256 values
static void invert_diag_blocks(const double* Cp, long ldc, int nbp, double* inv, HostTeam& team) {
  team.parallel_for(nbp, (nbp + team.size() - 1) / team.size(), [&](long bl) {
    const int b = int(bl);
    double D[16][16], V[16][16];
    for (int i = 0; i < 16; ++i)
      for (int j = 0; j < 16; ++j) D[i][j] = j <= i ? Cp[long(b * 16 + i) * ldc + b * 16 + j] : 0.0;
    for (int c = 0; c < 16; ++c)
      for (int i = 0; i < 16; ++i) {
        double s = i == c ? 1.0 : 0.0;
        for (int p = 0; p < i; ++p) s -= D[i][p] * V[p][c];
        V[i][c] = s / D[i][i];
      }
    std::memcpy(inv + size_t(b) * 256, V, sizeof V);
  });
}

// L columns c0 .. c0 + nc - 1 from the same columns of C, rows 0 .. row_end - 1: Cp holds rows c0 .. of those columns
// (row stride ldc), inv the inverses of their diagonal blocks.  L = C * blockdiag(C_bb^-1), 16x16 diagonal blocks
// and everything above them zero.  false if a value is not finite.
static bool assemble_L_columns(const double* Cp, long ldc, const double* inv, int c0, int nc, int n, int row_end,
                               float* L_out, HostTeam& team) {
  const Kernels kn = pick_kernels();
  const int nbp = nc / 16;
  std::atomic<int> finite{1};
  team.parallel_for(row_end, 16, [&](long rl) {
    const int r = int(rl);
    float* lr = L_out + long(r) * n + c0;
    if (r < c0) {  // above the diagonal blocks of these columns
      std::memset(lr, 0, sizeof(float) * size_t(nc));
      return;
    }
    const int rb = std::min(nbp, (r - c0) / 16);  // column blocks strictly left of this row's diagonal block
    const bool ok = kn.assemble_row(Cp + long(r - c0) * ldc, inv, rb, lr);
    if (rb < nbp) std::memset(lr + long(rb) * 16, 0, sizeof(float) * size_t(nc - rb * 16));  // diagonal block and right of it
    if (!ok) finite.store(0, std::memory_order_relaxed);
  });
  return finite.load() != 0;
}

bool block_ldl_host(double* A, int n, float* L_out, int threads) {
  if (n % 16 != 0) fail(QTIP_E_ARG, "block LDL needs n %% 16 == 0 (n = %d)", n);
  HostTeam& team = team_of_this_thread(threads);
  if (!cholesky_panels<NB, TILE>(A, n, n, &team)) return false;
  std::vector<double> inv(size_t(n / 16) * 256);
  invert_diag_blocks(A, n, n / 16, inv.data(), team);
  return assemble_L_columns(A, n, inv.data(), 0, n, n, n, L_out, team);
}

int ldl_panel_width() { return NB; }

bool block_ldl_assisted(int n, float* L_out, int threads, PanelAssist& assist) {
  if (n % 16 != 0) fail(QTIP_E_ARG, "block LDL needs n %% 16 == 0 (n = %d)", n);
  HostTeam& team = team_of_this_thread(threads);
  // L is assembled panel by panel from the solved columns as they pass through the host: the rows below a panel by
  // the thread that solved them, while they are in its cache; the rows above (zeros) and those of the diagonal
  // block after the update has been queued
  struct Wrap : PanelAssist {
    PanelAssist& inner;
    int n;
    float* L;
    HostTeam& team;
    const Kernels kn = pick_kernels();
    std::vector<double> inv;
    std::atomic<int> finite{1};
    Wrap(PanelAssist& i, int n_, float* L_, HostTeam& t) : inner(i), n(n_), L(L_), team(t) {}
    double* fetch(int k, int kb) override { return inner.fetch(k, kb); }
    void factored(int k, int kb, const double* diag, long ld) override {
      inv.resize(size_t(kb / 16) * 256);
      invert_diag_blocks(diag, ld, kb / 16, inv.data(), team);
    }
    void rows_solved(int k, int kb, int row0, int count, const double* rows, long ld) override {
      bool ok = true;
      for (int i = 0; i < count; ++i)
        ok = kn.assemble_row(rows + long(i) * ld, inv.data(), kb / 16, L + long(row0 + i) * n + k) && ok;
      if (!ok) finite.store(0, std::memory_order_relaxed);
    }
    void solved(int k, int kb, const double* panel) override {
      inner.solved(k, kb, panel);  // the update is queued first and runs while the rest of L's columns is written
      if (!assemble_L_columns(panel, kb, inv.data(), k, kb, n, k + kb, L, team)) finite.store(0, std::memory_order_relaxed);
      inner.assembled(k, kb);
    }
  } wrap(assist, n, L_out, team);
  if (!cholesky_panels<NB, TILE>(nullptr, 0, n, &team, &wrap)) return false;
  return wrap.finite.load() != 0;
}

// The scalar LDL of the NVFP4 calibration (nvfp4_quantize_group, src/nvfp4_gpu.hip:181-207: H = L D L^T from the
// Cholesky factor C, L_ij = C_ij / C_jj unit lower, dw_j = C_jj^2) from the same panel factorization, written as the
// panels pass through the host: the rows below a panel by the thread that solved them, the rows of the diagonal
// block, with the zeros on and right of the diagonal, once the update is queued.
bool scalar_ldl_assisted(int n, float* L_out, float* dw, int threads, PanelAssist& assist) {
  if (n % 16 != 0) fail(QTIP_E_ARG, "NVFP4 calibration needs n %% 16 == 0 (n = %d)", n);
  HostTeam& team = team_of_this_thread(threads);
  struct Wrap : PanelAssist {
    PanelAssist& inner;
    int n;
    float* L;
    float* dw;
    std::vector<double> diag;
    Wrap(PanelAssist& i, int n_, float* L_, float* dw_) : inner(i), n(n_), L(L_), dw(dw_) {}
    double* fetch(int k, int kb) override { return inner.fetch(k, kb); }
    void factored(int k, int kb, const double* d, long ld) override {
      diag.resize(size_t(kb));
      for (int j = 0; j < kb; ++j) {
        diag[size_t(j)] = d[long(j) * ld + j];
        dw[k + j] = float(diag[size_t(j)] * diag[size_t(j)]);
      }
    }
    void rows_solved(int k, int kb, int row0, int count, const double* rows, long ld) override {
      for (int i = 0; i < count; ++i) {
        float* li = L + long(row0 + i) * n + k;
        const double* r = rows + long(i) * ld;
        for (int j = 0; j < kb; ++j) li[j] = float(r[j] / diag[size_t(j)]);
      }
    }
    void solved(int k, int kb, const double* panel) override {
      inner.solved(k, kb, panel);  // the update is queued first
      for (int i = 0; i < kb; ++i) {
        float* li = L + long(k + i) * n;
        for (int j = 0; j < i; ++j) li[k + j] = float(panel[long(i) * kb + j] / diag[size_t(j)]);
        std::memset(li + k + i, 0, sizeof(float) * size_t(n - k - i));
      }
      inner.assembled(k, kb);
    }
  } wrap(assist, n, L_out, dw);
  return cholesky_panels<NB, TILE>(nullptr, 0, n, &team, &wrap);
}

// block_ldl_assisted with the trailing matrix held and updated by plain host code (one fma chain per element over the
// panel, from zero, then one subtraction): exercises the panel hand-over without a device.  L must come out as
// block_ldl_host's.
bool block_ldl_assisted_on_host(const float* HRr, int n, float* L_out, int threads) {
  struct HostTrailing final : PanelAssist {
    long n;
    std::vector<double> A, buf[2];
    int turn = 0;
    double* fetch(int k, int kb) override {
      std::vector<double>& b = buf[turn ^= 1];  // alternate, as the device form's two page-locked buffers do
      b.resize(size_t(n - k) * kb);
      for (long i = k; i < n; ++i)
        for (int p = 0; p < kb; ++p) b[size_t(i - k) * kb + p] = A[size_t(i) * n + k + p];
      return b.data();
    }
    void solved(int k, int kb, const double* panel) override {
      const long r0 = k + kb;
      const double* X = panel + size_t(kb) * kb;
      for (long i = r0; i < n; ++i)
        for (long j = r0; j <= i; ++j) {
          double acc = 0;
          for (int p = 0; p < kb; ++p) acc = __builtin_fma(X[size_t(i - r0) * kb + p], X[size_t(j - r0) * kb + p], acc);
          A[size_t(i) * n + j] -= acc;
        }
    }
  } host;
  host.n = n;
  host.A.assign(size_t(n) * n, 0.0);
  symmetrize_lower_host(HRr, n, host.A.data(), threads);
  return block_ldl_assisted(n, L_out, threads, host);
}

// A[i][j] = (HRr[i][j] + HRr[j][i]) / 2 in fp64, lower triangle (tiled so both reads stay in cache)
void symmetrize_lower_host(const float* HRr, int n, double* A, int threads) {
  HostTeam& team = team_of_this_thread(threads);
  constexpr int T = 64;
  const int nt = (n + T - 1) / T;
  team.parallel_for(nt, 1, [&](long bil) {
    const int bi = int(bil);
    for (int bj = 0; bj <= bi; ++bj) {
      const int i1 = std::min(n, (bi + 1) * T), j1 = std::min(n, (bj + 1) * T);
      for (int i = bi * T; i < i1; ++i)
        for (int j = bj * T; j < j1 && j <= i; ++j)
          A[size_t(i) * n + j] = 0.5 * (double(HRr[size_t(i) * n + j]) + double(HRr[size_t(j) * n + i]));
    }
  });
}

}  // namespace qtipmi
