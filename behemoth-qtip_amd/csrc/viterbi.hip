// Two-pass tail-biting Viterbi over the L=16, K=2, V=2 bitshift trellis for gfx950 (wave64).
//
// One 256-thread workgroup (4 waves) quantizes one 256-weight sequence (128 steps, 2^16 states) at a time and
// walks over its share of the tiles.  Path metrics are fp64 and every add/compare is the one the CPU
// algorithm performs (reference: viterbi_ref / quantize_seq_ref, src/qtip_core.cpp:123-191), so the
// selected path is identical, not merely close.
//
// Recursion.  With M_i[g] the best metric over the 16 states of group g (states sharing their low 12 bits)
// and E_i[e] the squared error of codebook entry e against the two inputs of step i,
//     M_{i+1}[j] = min_d ( E_i[entry((d << 12) | j)] + M_i[(d << 8) | (j >> 4)] ),   first minimum in d.
// The codebook has 1024 distinct entries, entry(s) = bits 6..15 of s*(s+1).  For s = (d << 12) | j the low
// 6 bits of the entry depend on j only ("row" of j) and the high 4 bits are (b4(j) + d*(2*(j&7)+1)) mod 16,
// a bijection in d.  Groups j and 4095-j have the same row, and their 16 entries are the same 16 values read
// in opposite order.  A lane therefore owns 8 groups of one metric column c (one for each value m of the low
// three bits, so that the stride 2m+1 is a compile-time constant) and their mirrors in column 255-c: per step it
// keeps the two metric columns (2 x 16 fp64) in registers and streams 8 rows of E (16 fp64 each) from LDS, i.e.
// 128 + 16 LDS reads for 256 add-compare-selects.
//
// LDS layout: free of bank conflicts.  An 8-byte LDS access is served 16 lanes at a time, and a 16-lane quarter
// takes as many cycles as the largest number of distinct addresses that fall on one of the 16 bank pairs.
//   * Lane t runs metric column c = 4u + r + 64b with u = t & 15, r = (t >> 4) & 3, b = (t >> 6) & 1 and owns the
//     groups j = 16c + 8h + m (h = t >> 7, m = 0..7) and their mirrors.  Bits 6..9 of j(j+1) are then
//     (u (2t'+1) + const) mod 16 over the 16 lanes of a quarter (t' = 8h + m): 16 different values for every m.
//   * The error table is stored entry position by row, E[q][row] (q = high 4 bits of the entry, 64 rows of 8 bytes),
//     so the bank pair of a read is row mod 16 = those bits, whatever the rotation b4; the 16 positions are stored
//     twice (q = 0..31) so that the rotation is a per-lane base address and the stride d*(2m+1) mod 16 a
//     compile-time offset.
//   * The metric of (column c, digit d) sits at pos(c)*16 + (d ^ swz(c)): pos(c) is c with bits 0 and 2 exchanged and
//     swz(c) = 2 ((c >> 3 & 7) ^ 2 (c >> 6)) is even, so the digits 2k and 2k+1 of a column are one 16-byte piece, in
//     that order for every lane: a column comes in as eight 16-byte reads whose addresses are one XOR of a per-lane
//     base with 16k.  A 16-byte LDS access is served 16 lanes at a time as well, but in the turns {0-3, 12-15, 20-27}
//     and {4-11, 16-19, 28-31} of each half-wave, at full rate when the 16 lanes of a turn touch 16 different 16-byte
//     bank groups: bits 4..6 of the address are (k ^ u >> 1) and bit 7 is u & 1 here, a different value for each of
//     the 16 values u of a turn.  The 16 lanes of a quarter write 16 different bank pairs for every slot (their
//     digits differ in the low two bits, their target columns in bits 6 and 7, which swz moves to slot bits 2 and 3),
//     and the mirror group's slot is the group's XOR 0xffd.
// LDS per workgroup ~50 KB, three workgroups per CU; metrics single-buffered (the columns are read into registers
// before the step's results are written).
// No back-pointers.  A step's 16-way search keeps the minimum only (add + min per candidate); which digit won
// matters for the 127 groups on the surviving path alone, so the metrics entering every second step (32 KB, written
// value-major: one contiguous 512-byte store per wave and value) are kept in HBM and the trace-back redoes the
// add-compare-selects of the path it walks, two steps per round trip, with the forward pass's own fp64 operations
// and tie rule.  Only the last step tracks its digits (in registers), which the final state needs.
//
// The above is the fp64 form.  By default every pass first runs on unsigned 32-bit metrics in units of 2^-26
// (forward_pass32 / trace_back32 further down: 4-byte table and metrics in the same LDS footprint, double-buffered,
// one barrier per step; the free pass computes the groups below 2048 only, since complementary states decode alike),
// its trace-back checks that every decision it takes was won by more than the rounding can move two candidates
// against each other, and a pass that fails the check is run again through the fp64 form in the same launch: the
// states are the fp64 form's, bit for bit.  A launch that cannot fill the chip uses the kernel's wide form, 512
// threads per tile.
#include <hip/hip_ext.h>

#include <cstddef>
#include <mutex>
#include <type_traits>

#include "bf16_split.hpp"
#include "qtip_internal.hpp"

namespace qtipmi {
namespace {

constexpr int kThreads = 256;
constexpr int kESlots = 32 * 64;                 // E[q][row]: 16 entry positions stored twice x 64 rows
constexpr int kMSlots = 4096;                    // metric of (column c, digit d) at m_slot(c, d)
constexpr int kHistSteps = 63;                           // the metrics entering the odd steps 1, 3 .. 125 are kept
constexpr int kHistWordsPerTile = kHistSteps * kGroups;  // fp64 words
enum StepKind { kPlain = 0, kStore = 1, kDigits = 2 };

// Kept-metrics slots for callers that may not allocate (qtip_viterbi_tiles_dev_noalloc): part of the code object, so
// every device that loads the library holds its own copy (63 MiB) until the process ends.  Host code must not use
// this name as an address; the per-device address comes from hipGetSymbolAddress (static_scratch_of below).
constexpr int kStaticSlots = 32;
static __device__ __align__(256) double scratch[size_t(kStaticSlots) * kHistWordsPerTile];
constexpr int kMaxDevices = 64;
double* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

// metric array: column `col` lives at position m_pos(col) (bits 0 and 2 of the column exchanged), digit d in slot
// d ^ m_swz(col) of its 16; m_swz is even, so the digits 2k and 2k + 1 are the halves of one 16-byte piece
__device__ __forceinline__ int m_pos(int col) { return (col & ~5) | ((col & 1) << 2) | ((col >> 2) & 1); }
__device__ __forceinline__ int m_swz(int col) { return (((col >> 3) & 7) ^ (((col >> 6) & 3) << 1)) << 1; }
__device__ __forceinline__ int m_slot(int col, int d) { return m_pos(col) * 16 + (d ^ m_swz(col)); }

// threadIdx.x through a barrier for the optimizer: what a pass derives from it (table rows, metric slots, read
// addresses: some twenty registers per kind of pass) is then formed where the pass starts instead of once at the top
// of the kernel, where the three kinds together would sit in registers for the whole launch and push the passes' own
// values out to scratch memory
// The wide form of the kernel runs 512 threads per tile: its 32-bit forward passes share the groups out over all of
// them (opaque_tid_wide), everything else is done twice, by the threads t and t + 256 alike (same reads, same
// values written to the same places), so that every wave meets every barrier.
__device__ __forceinline__ int opaque_tid() {
  int t = threadIdx.x & (kThreads - 1);
  asm volatile("" : "+v"(t));
  return t;
}
__device__ __forceinline__ int opaque_tid_wide() {
  int t = threadIdx.x;
  asm volatile("" : "+v"(t));
  return t;
}

struct Smem {
  double E[kESlots];  // first: its reads use 8-bit immediate offsets from a per-lane base
  double M[kMSlots];
  float x[kSeq];
  uint16_t st[kSteps];
  double red_c[4];
  uint32_t red_s[4];
  double tr_c[2][4];    // trace-back: the four waves' best candidates of a round (cost; d | d1 << 8), two sets
  uint32_t tr_d[2][4];
  alignas(16) uint32_t tr32[2][4][4];  // the same for the 32-bit passes: best, second best, d | d1 << 8, gap inside the best's row
  uint32_t red32[8][3];    // end of the free 32-bit pass: per wave the best group's metric, the second best, the group
  int overlap;
  uint32_t final_state;
  float final_metric;  // the free fp64 pass's best final metric (what later 32-bit passes of the tile row may expect)
};

__device__ __forceinline__ int perm_fwd(int p) {  // sequence position -> tile index 16*r + c
  const int e = p & 1, a = (p >> 1) & 1, c = (p >> 2) & 1, d = (p >> 3) & 3, b = (p >> 5) & 7;
  return a * 128 + b * 16 + c * 8 + d * 2 + e;
}

// thread that owns group jj < 2048 (slot m = jj & 7): column c = jj >> 4 = 4u + r + 64b, half h = bit 3 of jj
__device__ __forceinline__ uint32_t owner_thread(uint32_t jj) {
  const uint32_t c = jj >> 4, h = (jj >> 3) & 1u;
  return ((c & 63u) >> 2) | ((c & 3u) << 4) | ((c >> 6) << 6) | (h << 7);
}
// place of group g in one kept step of metrics: value (jj & 7) (+ 8 for a mirror group) of the owning thread, stored
// value-major so that a wave's 64 values are one contiguous 512-byte store
__device__ __forceinline__ uint32_t hist_index(uint32_t g) {
  const uint32_t jj = g < 2048u ? g : 4095u - g;
  return ((jj & 7u) + (g < 2048u ? 0u : 8u)) * kThreads + owner_thread(jj);
}

// One forward pass over the 128 steps.  roll: input rotation (128 for the first pass).  ov < 0: free start and
// end; otherwise start in states with (s >> 4) == ov and end in the state of group ov.
// The even steps first_kept .. 124 also write their results, the metrics entering the next (odd) step, to hist.
// Returns nothing; the final state is left in sm.final_state.
__device__ __forceinline__ void forward_pass(Smem& sm, const double* __restrict__ entry_d, int roll, int ov,
                                             double* __restrict__ hist, int first_kept) {
  const int tid = opaque_tid();
  const int colA = 4 * (tid & 15) + ((tid >> 4) & 3) + 64 * ((tid >> 6) & 1), colB = 255 - colA;
  const int half = tid >> 7;  // owns 16c + 8 half + m, m = 0..7
  const double INF = __builtin_inf();

  // this thread's 4 codebook entries for the per-step error table: e = tid + 256*q -> row tid & 63, position
  // (tid >> 6) + 4q (re-read from the 16 KB global table every step: it stays in the CU's vector L1 and the registers
  // are needed)
  const double2* __restrict__ entries = reinterpret_cast<const double2*>(entry_d) + tid;
  const int e_wr = (tid >> 6) * 64 + (tid & 63);

  // per slot: E base (b4 * 64 + row) and the metric slot written for the group; the mirror group's is that ^ kMirror
  int ebase[8], wslot[8];
  constexpr int kMirror = 0xffd;
#pragma unroll
  for (int m = 0; m < 8; ++m) {
    const uint32_t j = 16u * colA + 8u * uint32_t(half) + m, p = j * (j + 1u);
    ebase[m] = int((p >> 12) & 15u) * 64 + int((p >> 6) & 63u);
    wslot[m] = m_slot(int(j & 255u), int(j >> 8));
  }
  // byte offsets of digit 0 of the two metric columns; the pair of digits (2k, 2k + 1) is at that ^ 16 k
  int xA = m_pos(colA) * 128 + m_swz(colA) * 8, xB = m_pos(colB) * 128 + m_swz(colB) * 8;
  const char* const Mb = reinterpret_cast<const char*>(sm.M);

  // initial metrics: M_0[g] = 0, or +inf outside group ov
  for (int g = tid; g < kGroups; g += kThreads) {
    sm.M[m_slot(g & 255, g >> 8)] = (ov < 0 || g == ov) ? 0.0 : INF;
  }
  __syncthreads();

  unsigned long long word = 0;
  // one trellis step; kDigits: the winning digits are wanted (without them a candidate costs an add and a min);
  // kStore: the results also go to hist
  auto step = [&](int it, auto kind_tag) __attribute__((always_inline)) {
    constexpr int kind = decltype(kind_tag)::value;
    constexpr bool digits = kind == kDigits;
    double* hs = nullptr;
    if constexpr (kind == kStore) hs = hist + size_t(it >> 1) * kGroups + tid;
    // ---- phase R: metric columns -> registers, error table of this step -> LDS
    double MA[16], MB[16];
    // 16-byte reads, two digits each; the 16 read addresses are recomputed in every step (one XOR each): kept
    // across the loop they would take 16 registers the accumulators need
    asm volatile("" : "+v"(xA), "+v"(xB));
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const double2 a = *reinterpret_cast<const double2*>(Mb + (xA ^ (16 * k)));
      const double2 b = *reinterpret_cast<const double2*>(Mb + (xB ^ (16 * k)));
      MA[2 * k] = a.x, MA[2 * k + 1] = a.y;
      MB[2 * k] = b.x, MB[2 * k + 1] = b.y;
    }
    {
      const int t = (2 * it + roll) & 255;
      const double x0 = double(sm.x[t]), x1 = double(sm.x[t + 1]);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const double2 l = entries[256 * q];
        const double a = l.x - x0, b = l.y - x1;
        const double err = __builtin_fma(a, a, b * b);
        sm.E[e_wr + 256 * q] = err;
        sm.E[e_wr + 256 * q + 1024] = err;
      }
    }
    __syncthreads();
    // ---- phase C: 16 groups x 16 candidates.  The 16 error values of a slot are consumed as two halves of 8
    // (software-pipelined: the next half is in flight while this one is used).  The group scans its digits
    // upwards with "<", its mirror scans downwards with "<=" over the same values; both keep the smallest
    // digit among equal minima, as the ascending first-minimum rule of the CPU algorithm does.
    word = 0;
    double cur[8], nxt[8];
    {
      const double* er = sm.E + ebase[0];
#pragma unroll
      for (int k = 0; k < 8; ++k) cur[k] = er[(k & 15) * 64];  // slot 0: stride 1
    }
#pragma unroll
    for (int m = 0; m < 8; ++m) {
      const int g = 2 * m + 1;
      {
        const double* er = sm.E + ebase[m];
#pragma unroll
        for (int k = 0; k < 8; ++k) nxt[k] = er[(((8 + k) * g) & 15) * 64];
      }
      double ba = cur[0] + MA[0], bb = cur[0] + MB[15], ca, cb;
      uint32_t da = 0, db = 15;
      unsigned long long mka, mkb;
      // one candidate of the group (digit KA, strict <) and one of its mirror (digit KB, <=) from the same table
      // value: add, compare, min, select -- written out so that the two chains stay interleaved
#define QTIP_ACS2(KA, KB, EV, MAV, MBV)                                                                      \
  asm volatile(                                                                                             \
      "v_add_f64 %[ca], %[e], %[ma]\n\t"                                                                    \
      "v_add_f64 %[cb], %[e], %[mb]\n\t"                                                                    \
      "v_cmp_lt_f64_e64 %[ka], %[ca], %[ba]\n\t"                                                            \
      "v_cmp_le_f64_e64 %[kb], %[cb], %[bb]\n\t"                                                            \
      "v_min_f64 %[ba], %[ba], %[ca]\n\t"                                                                   \
      "v_min_f64 %[bb], %[bb], %[cb]\n\t"                                                                   \
      "v_cndmask_b32_e64 %[da], %[da], " #KA ", %[ka]\n\t"                                                  \
      "v_cndmask_b32_e64 %[db], %[db], " #KB ", %[kb]"                                                       \
      : [ca] "=&v"(ca), [cb] "=&v"(cb), [ka] "=&s"(mka), [kb] "=&s"(mkb), [ba] "+v"(ba), [bb] "+v"(bb),     \
        [da] "+v"(da), [db] "+v"(db)                                                                        \
      : [e] "v"(EV), [ma] "v"(MAV), [mb] "v"(MBV))
      // the same without the digit
#define QTIP_AM2(EV, MAV, MBV)                                       \
  asm volatile(                                                      \
      "v_add_f64 %[ca], %[e], %[ma]\n\t"                             \
      "v_add_f64 %[cb], %[e], %[mb]\n\t"                             \
      "v_min_f64 %[ba], %[ba], %[ca]\n\t"                            \
      "v_min_f64 %[bb], %[bb], %[cb]"                                \
      : [ca] "=&v"(ca), [cb] "=&v"(cb), [ba] "+v"(ba), [bb] "+v"(bb) \
      : [e] "v"(EV), [ma] "v"(MAV), [mb] "v"(MBV))
      if constexpr (digits) {
        QTIP_ACS2(1, 14, cur[1], MA[1], MB[14]);
        QTIP_ACS2(2, 13, cur[2], MA[2], MB[13]);
        QTIP_ACS2(3, 12, cur[3], MA[3], MB[12]);
        QTIP_ACS2(4, 11, cur[4], MA[4], MB[11]);
        QTIP_ACS2(5, 10, cur[5], MA[5], MB[10]);
        QTIP_ACS2(6, 9, cur[6], MA[6], MB[9]);
        QTIP_ACS2(7, 8, cur[7], MA[7], MB[8]);
      } else {
        QTIP_AM2(cur[1], MA[1], MB[14]);
        QTIP_AM2(cur[2], MA[2], MB[13]);
        QTIP_AM2(cur[3], MA[3], MB[12]);
        QTIP_AM2(cur[4], MA[4], MB[11]);
        QTIP_AM2(cur[5], MA[5], MB[10]);
        QTIP_AM2(cur[6], MA[6], MB[9]);
        QTIP_AM2(cur[7], MA[7], MB[8]);
      }
      if (m < 7) {
        const int gn = 2 * (m + 1) + 1;
        const double* er = sm.E + ebase[m < 7 ? m + 1 : 7];
#pragma unroll
        for (int k = 0; k < 8; ++k) cur[k] = er[((k * gn) & 15) * 64];
      }
      if constexpr (digits) {
        QTIP_ACS2(8, 7, nxt[0], MA[8], MB[7]);
        QTIP_ACS2(9, 6, nxt[1], MA[9], MB[6]);
        QTIP_ACS2(10, 5, nxt[2], MA[10], MB[5]);
        QTIP_ACS2(11, 4, nxt[3], MA[11], MB[4]);
        QTIP_ACS2(12, 3, nxt[4], MA[12], MB[3]);
        QTIP_ACS2(13, 2, nxt[5], MA[13], MB[2]);
        QTIP_ACS2(14, 1, nxt[6], MA[14], MB[1]);
        QTIP_ACS2(15, 0, nxt[7], MA[15], MB[0]);
      } else {
        QTIP_AM2(nxt[0], MA[8], MB[7]);
        QTIP_AM2(nxt[1], MA[9], MB[6]);
        QTIP_AM2(nxt[2], MA[10], MB[5]);
        QTIP_AM2(nxt[3], MA[11], MB[4]);
        QTIP_AM2(nxt[4], MA[12], MB[3]);
        QTIP_AM2(nxt[5], MA[13], MB[2]);
        QTIP_AM2(nxt[6], MA[14], MB[1]);
        QTIP_AM2(nxt[7], MA[15], MB[0]);
      }
#undef QTIP_ACS2
#undef QTIP_AM2
      sm.M[wslot[m]] = ba;
      sm.M[wslot[m] ^ kMirror] = bb;
      if constexpr (kind == kStore) {
        hs[m * kThreads] = ba;
        hs[(8 + m) * kThreads] = bb;
      }
      if constexpr (digits) {
        word |= (unsigned long long)(da) << (4 * m);
        word |= (unsigned long long)(db) << (32 + 4 * m);
      }
    }
    __syncthreads();
  };
  using Plain = std::integral_constant<int, kPlain>;
  using Store = std::integral_constant<int, kStore>;
  using Digits = std::integral_constant<int, kDigits>;
#pragma nounroll
  for (int it = 0; it < kSteps - 1; ++it) {
    if (!(it & 1) && it >= first_kept && it < kSteps - 2) step(it, Store{});
    else step(it, Plain{});
  }
  step(kSteps - 1, Digits{});
  // final state: smallest metric, then smallest state, over the metrics of the last step (each lane re-reads the
  // 16 values it has just written; their predecessor digits are the nibbles of the last step's digit word)
  if (ov < 0) {
    double bestc = INF;
    uint32_t bests = 0xffffffffu;
#pragma unroll
    for (int m = 0; m < 8; ++m) {
      const uint32_t ja = 16u * colA + 8u * uint32_t(half) + m, jb = 4095u - ja;
      const uint32_t sa = (uint32_t(word >> (4 * m)) & 15u) << 12 | ja;
      const uint32_t sb = (uint32_t(word >> (32 + 4 * m)) & 15u) << 12 | jb;
      const double ca = sm.M[wslot[m]], cb = sm.M[wslot[m] ^ kMirror];
      if (ca < bestc || (ca == bestc && sa < bests)) bestc = ca, bests = sa;
      if (cb < bestc || (cb == bestc && sb < bests)) bestc = cb, bests = sb;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const double oc = __shfl_xor(bestc, off, 64);
      const uint32_t os = __shfl_xor(bests, off, 64);
      if (oc < bestc || (oc == bestc && os < bests)) bestc = oc, bests = os;
    }
    if ((tid & 63) == 0) sm.red_c[tid >> 6] = bestc, sm.red_s[tid >> 6] = bests;
    __syncthreads();
    if (tid == 0) {
      double c = sm.red_c[0];
      uint32_t s = sm.red_s[0];
      for (int w = 1; w < 4; ++w)
        if (sm.red_c[w] < c || (sm.red_c[w] == c && sm.red_s[w] < s)) c = sm.red_c[w], s = sm.red_s[w];
      sm.final_state = s & 0xffffu;  // (no comparison succeeds on NaN metrics; the walk needs a 16-bit state anyway)
      sm.final_metric = float(c);
    }
  } else {
    const uint32_t j = uint32_t(ov), jj = j < 2048u ? j : 4095u - j;
    if (owner_thread(jj) == uint32_t(tid)) {
      const uint32_t shift = (jj & 7u) * 4u + (j < 2048u ? 0u : 32u);
      sm.final_state = (uint32_t(word >> shift) & 15u) << 12 | j;
    }
  }
  __syncthreads();
}

// The Viterbi input of one tile inside LDLQ: W plus the error feedback of the columns already quantized (the formula
// at TileJob), which the reference computes in a kernel of its own (ldlq_prep_kernel, src/viterbi.hip:241-267; CPU
// form tests/test_gpu.cpp:196-207).  The (<= 112) x 16 blocks of L, WT and hatWT the tile needs are staged in the
// metric array, which is idle between tiles; thread u then owns the sequence position u.
template <typename Acc>
__device__ __forceinline__ void tile_targets(Smem& sm, const TileJob& job, long col0, long tile,
                                             const Acc* __restrict__ prod) {
  const int u = opaque_tid();
  const int k0 = int(col0) + 16, nk = job.bufend - k0;
  float* Ls = reinterpret_cast<float*>(sm.M);
  float* Ws = Ls + 112 * 16;
  float* Hs = Ws + 112 * 16;
  const long row0 = tile * 16;
  for (int idx = u; idx < nk * 16; idx += kThreads) {
    const long k = k0 + (idx >> 4);
    const int e = idx & 15;
    Ls[idx] = job.L[k * job.ldl + col0 + e];
    Ws[idx] = job.WT[k * job.ldw + row0 + e];
    Hs[idx] = job.hatWT[k * job.ldw + row0 + e];
  }
  __syncthreads();
  const int q = perm_fwd(u), r = q >> 4, c = q & 15;
  const long col = col0 + c;
  const Acc* pp = prod + (col - job.prod_row0) * (job.ldp ? job.ldp : job.ldw) + row0 + r;
  Acc gathered = pp[0];
  for (int sp = 1; sp < job.prod_splits; ++sp) gathered += pp[long(sp) * job.prod_split_stride];
  Acc acc = Acc(job.WT[col * job.ldw + row0 + r]) + gathered;
  for (int kk = 0; kk < nk; ++kk) acc += Acc(Ls[kk * 16 + c]) * (Acc(Ws[kk * 16 + r]) - Acc(Hs[kk * 16 + r]));
  sm.x[u] = float(_Float16(float(acc)));
}

// smallest value over the 16 lanes of a row (lanes 16 r .. 16 r + 15), in each of them: four cross-lane moves inside
// the vector pipe (neighbour, pair, mirrored half row, mirrored row).  No NaNs reach it.
__device__ __forceinline__ double row_min16(double c) {
#define QTIP_ROW_STEP(CTRL)                                                                       \
  {                                                                                               \
    const int lo = __builtin_amdgcn_update_dpp(0, __double2loint(c), CTRL, 0xf, 0xf, false);      \
    const int hi = __builtin_amdgcn_update_dpp(0, __double2hiint(c), CTRL, 0xf, 0xf, false);      \
    const double o = __hiloint2double(hi, lo);                                                    \
    asm volatile("v_min_f64 %0, %1, %2" : "=v"(c) : "v"(c), "v"(o));                              \
  }
  QTIP_ROW_STEP(0xB1)   // quad_perm [1, 0, 3, 2]
  QTIP_ROW_STEP(0x4E)   // quad_perm [2, 3, 0, 1]
  QTIP_ROW_STEP(0x141)  // row_half_mirror
  QTIP_ROW_STEP(0x140)  // row_mirror
#undef QTIP_ROW_STEP
  return c;
}

__device__ __forceinline__ double read_lane_f64(double v, int lane) {
  return __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(v), lane),
                          __builtin_amdgcn_readlane(__double2loint(v), lane));
}

// Trace-back, run by all four waves: walks two steps per round trip to HBM.  s is the state of step it + 1;
// for every digit d of step it the metric M_it[g_d] of the group g_d = (d << 8) | (j >> 4), j = s >> 4, is rebuilt
// from the kept metrics of step it - 1 as the forward pass built it (the 16 lanes of a row, one per digit of step
// it - 1, same fp64 operations, smallest digit among equal minima), then the 16 candidates of step it are compared
// the same way: wave w takes the digits 4w .. 4w+3 (one per row), picks among its four, and the four waves' picks
// meet in LDS (two alternating sets of slots, one barrier per round).
// Returns the state of step it_min - 1; record: the states of the steps walked are written to sm.st.
__device__ __forceinline__ uint32_t trace_back(Smem& sm, const double* __restrict__ entry_d,
                                               const double* __restrict__ hist, int roll, uint32_t s, int it_min,
                                               bool record) {
  const uint32_t tid = uint32_t(opaque_tid());
  const uint32_t lane = tid & 63u, wave = tid >> 6, dp = lane & 15u, d = 4u * wave + (lane >> 4);
  int set = 0;
#pragma nounroll
  for (int it = kSteps - 2; it >= it_min; it -= 2, set ^= 1) {
    const uint32_t j = s >> 4;
    const int ta = (2 * (it - 1) + roll) & 255, tb = (2 * it + roll) & 255;
    const double xa0 = double(sm.x[ta]), xa1 = double(sm.x[ta + 1]);
    const double xb0 = double(sm.x[tb]), xb1 = double(sm.x[tb + 1]);
    const unsigned long long* row =
        reinterpret_cast<const unsigned long long*>(hist + size_t(it / 2 - 1) * kGroups);
    const uint32_t p = (dp << 8) | (d << 4) | (j >> 8);
    // written by this workgroup's own waves before the barrier that ended the forward pass: workgroup scope suffices
    const double mv = __longlong_as_double((long long)__hip_atomic_load(row + hist_index(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP));
    const uint32_t g = (d << 8) | (j >> 4);
    const uint32_t s1 = (dp << 12) | g, e1 = ((s1 * (s1 + 1u)) >> 6) & 1023u;
    const double a1 = entry_d[2 * e1] - xa0, b1 = entry_d[2 * e1 + 1] - xa1;
    const uint32_t s0 = (d << 12) | j, e0 = ((s0 * (s0 + 1u)) >> 6) & 1023u;
    const double a0 = entry_d[2 * e0] - xb0, b0 = entry_d[2 * e0 + 1] - xb1;
    const double c1 = __builtin_fma(a1, a1, b1 * b1) + mv;
    const double m1 = row_min16(c1);  // M_it[g_d]
    // its digit: the first lane of the row that holds the minimum (no lane at all if the inputs held a NaN: any
    // digit will do then, but it must stay a digit)
    const unsigned long long at_min = __builtin_amdgcn_ballot_w64(c1 == m1);
    const uint32_t row_bits = uint32_t(at_min >> (lane & 48u)) & 0xffffu;
    const uint32_t k1 = row_bits ? uint32_t(__builtin_ctz(row_bits)) : 0u;
    const double c0 = __builtin_fma(a0, a0, b0 * b0) + m1;
    // every lane of row r holds that row's (cost, d1) for d = 4 wave + r; pick across the four rows, smallest d on ties
    double bc = read_lane_f64(c0, 0);
    uint32_t bd = 4u * wave, bd1 = uint32_t(__builtin_amdgcn_readlane(int(k1), 0));
#pragma unroll
    for (int r = 1; r < 4; ++r) {
      const double oc = read_lane_f64(c0, 16 * r);
      const uint32_t od1 = uint32_t(__builtin_amdgcn_readlane(int(k1), 16 * r));
      const bool take = oc < bc;  // rows ascend in d: the first minimum stays
      bc = take ? oc : bc;
      bd = take ? 4u * wave + uint32_t(r) : bd;
      bd1 = take ? od1 : bd1;
    }
    if (lane == 0) {
      sm.tr_c[set][wave] = bc;
      sm.tr_d[set][wave] = bd | (bd1 << 8);
    }
    __syncthreads();
    bc = sm.tr_c[set][0];
    uint32_t bdd = sm.tr_d[set][0];
#pragma unroll
    for (int w = 1; w < 4; ++w) {
      const double oc = sm.tr_c[set][w];
      const uint32_t od = sm.tr_d[set][w];
      const bool take = oc < bc;  // waves ascend in d
      bc = take ? oc : bc;
      bdd = take ? od : bdd;
    }
    const uint32_t s_it = ((bdd & 15u) << 12) | j;
    s = (((bdd >> 8) & 15u) << 12) | (s_it >> 4);
    if (record && threadIdx.x == 0) {
      sm.st[it] = uint16_t(s_it);
      sm.st[it - 1] = uint16_t(s);
    }
  }
  return s;
}

// ================================================================= the same two passes on 32-bit metrics
// The fp64 passes above are bound by the issue rate of fp64 vector instructions and, behind it, by 8-byte LDS reads.
// Both passes are therefore first run on unsigned 32-bit metrics in units of 2^-26 (or another even power of two,
// unit_log2_for below): the squared error of a codebook entry is formed in fp64 (the sum of the two squared
// differences, as above, on operands scaled by a power of two) and brought to the nearest unit once (|error| <= 1/2
// unit + 2^-20); errors and metrics are held to 2^32 - 1 (= 64.0 at 2^-26, which also stands for +inf: every chain of
// minima starts from it; the adds are the integer add with its clamp bit set, which stops there instead of
// wrapping), and a path metric of n terms differs from the fp64 one by at most n/2 units (and a little), whatever
// the path.  Only the decisions on the surviving path matter: the
// trace-back redoes them from the kept metrics as above and also looks at the runner-up.  If every decision it takes
// (the final state, and the 16-way choice of each step it walks) is won by at least `thr` > 128 units and the winner is
// below 2^32 - 2^20 (nothing on its path was cut off), the fp64 recursion takes the same decisions and the
// pass's result is the fp64 result.  (thr is what the last step needs, whose candidates are sums of 128 terms; a
// decision of step t compares sums of t + 1 terms and is held to thr - (127 - t).)  Otherwise the
// workgroup runs that pass again through the fp64 code above (a fraction of a percent of the passes: near-ties of
// 5e-6, and the exact ties between states that share predecessor and codebook entry).
// Integer adds issue at twice the rate of fp64 adds on this chip and a three-way minimum covers two candidates, so an
// add-compare-select costs 1.5 instructions of 4.5 ns per pair instead of 2 of 8.2 ns; the table and the metrics are
// 4 bytes, half the LDS traffic, and the kept metrics half the HBM traffic.
//
// Free ends (first pass): state s and its complement 65535 - s decode to the same values and the complement of a
// predecessor is a predecessor of the complement, so with equal initial metrics the metric of group 4095 - j equals
// that of group j at every step, exactly.  The pass computes the groups below 2048 only (half of the candidates) and
// copies them to their mirrors; of the two best final states, complements of each other, the smaller one is taken,
// which is what the first-minimum rule of the CPU algorithm does.
//
// LDS layout for 4-byte values (32 banks of 4 bytes, a 4-byte access served 32 lanes at a time): lane t runs metric
// column c = 4 (t & 31) + (t >> 5 & 3) and owns the groups j = 16 c + 8 (t >> 7) + m, m = 0..7, and their mirrors.
// Bits 6..10 of j(j+1) then run through all 32 values over the 32 lanes of a half wave, so the table E32[q][row]
// (64 rows of 4 bytes per entry position q, positions stored twice for the rotation as above) is read without
// conflicts.  The metric of (column, digit d) sits at pos(column) * 16 + (d ^ swz(column)) with swz a multiple of 4,
// so a column comes in as four 16-byte reads; pos and swz are chosen so that those reads, the 4-byte writes of a
// group's result (32 lanes: 4 columns x 8 digits) and of its mirror (slot ^ 0xfeb) are free of bank conflicts.
constexpr uint32_t kSat = 0xffffffffu;      // the largest metric (64.0 in units of 2^-26), and +inf
// A decision's winner must be below this: nothing on its path was then cut off at kSat (a path's metric only grows).
// A candidate that was cut off is truly larger than it reads, so a margin seen against it is a margin there.
constexpr uint32_t kWinnerMax = kSat - (1u << 20);
// The unit of a pass is 2^-k, k even and chosen per pass so that the winner expected, with room to spare, still
// fits: the finer the unit, the narrower in value the margin a decision must be won by, the fewer passes repeated -
// and inputs of another scale than normalized weights (winners near 20 to 25: k = 26) still run on 32-bit metrics.
// The tail-biting pass expects the winner of its block's free pass, which ran on the same values (room: an eighth);
// the free pass that of the tile row's previous column block (room: as much again).  k = 26 (winners up to 64.0)
// when nothing is known yet.  A winner that does not fit after all repeats the pass on fp64 metrics.
constexpr int kUnitLog2Default = 26, kUnitLog2Min = 12, kUnitLog2Max = 30;
__device__ __forceinline__ int unit_log2_for(float expected_winner, float room) {
  if (!(expected_winner > 0.f)) return kUnitLog2Default;
  // largest even k with room x winner x 2^k <= 2^32
  int k = (32 - int(__builtin_ceilf(__builtin_log2f(room * expected_winner)))) & ~1;
  return k < kUnitLog2Min ? kUnitLog2Min : k > kUnitLog2Max ? kUnitLog2Max : k;
}
// The unit 2^-k as the table's arithmetic wants it (k is even): codebook values and inputs are multiplied by pre =
// 2^(k/2), which is exact and scales the differences, their squares and the sum of the squares exactly as a
// multiplication of the sum by 2^k would, so the sum comes out in units.
struct Unit {
  double pre;
};
__device__ __forceinline__ Unit unit_of(int k) { return Unit{__builtin_bit_cast(double, uint64_t(1023 + k / 2) << 52)}; }
constexpr int kMirror32 = 0xfeb;
static_assert(64 * kGroups <= 2 * kHistWordsPerTile, "the 32-bit kept metrics (64 steps) must fit the fp64 slot");

__device__ __forceinline__ int m32_pos(int col) {  // bits 7..0: b7 b6 b5 b4 b1 b0 b3 (b2 ^ b6)
  return (col & 0xf0) | ((col & 3) << 2) | (((col >> 3) & 1) << 1) | (((col >> 2) ^ (col >> 6)) & 1);
}
__device__ __forceinline__ int m32_swz(int col) { return (((col >> 4) & 1) << 2) | ((((col >> 5) ^ (col >> 7)) & 1) << 3); }
__device__ __forceinline__ int m32_slot(int col, int d) { return m32_pos(col) * 16 + (d ^ m32_swz(col)); }
// The free pass keeps the groups below 2048 only (column c, digits 0..7) in a compact array: 8 slots per column,
// column c at position [b7 b6 b5 b1 b0 b4 b3^b7 b2^b6], digit d in slot d ^ 4 b5.  The two 16-byte pieces of a
// column are read by the 16 lanes of a turn from 16 different bank groups, for a thread's own column and for its
// mirror 255 - c alike (digits 8..15 of column c are digits 7..0 of the mirror), and the 32 lanes of a half-wave
// write 32 different banks.
__device__ __forceinline__ int m32c_pos(int col) {
  return (col & 0xe0) | (((col >> 1) & 1) << 4) | ((col & 1) << 3) | (((col >> 4) & 1) << 2) |
         ((((col >> 3) ^ (col >> 7)) & 1) << 1) | (((col >> 2) ^ (col >> 6)) & 1);
}
__device__ __forceinline__ int m32c_swz(int col) { return ((col >> 5) & 1) << 2; }
__device__ __forceinline__ int m32c_slot(int col, int d) { return m32c_pos(col) * 8 + (d ^ m32c_swz(col)); }
// thread that owns group jj < 2048 in the 32-bit passes
__device__ __forceinline__ uint32_t owner32(uint32_t jj) {
  const uint32_t c = jj >> 4;
  return (c >> 2) | ((c & 3u) << 5) | (((jj >> 3) & 1u) << 7);
}
// place of group g in one kept step (value-major: a wave's store is 256 contiguous bytes); kSym: the mirror groups
// are not kept, their metrics are those of the groups they mirror
template <bool kSym>
__device__ __forceinline__ uint32_t hist32_index(uint32_t g) {
  const uint32_t jj = g < 2048u ? g : 4095u - g;
  return ((jj & 7u) + ((kSym || g < 2048u) ? 0u : 8u)) * kThreads + owner32(jj);
}
// metrics and errors are at most kSat = 2^32 - 1 and the add stops there (v_add_u32 with clamp); every chain of
// minima starts from kSat
__device__ __forceinline__ uint32_t sat_add(uint32_t a, uint32_t b) { return __builtin_elementwise_add_sat(a, b); }
__device__ __forceinline__ uint32_t min3u(uint32_t a, uint32_t b, uint32_t c) {
  uint32_t r;  // written out: the compiler forms the three-way minimum for only half of the chains
  asm("v_min3_u32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
// Squared error of a codebook entry against the two inputs of a step in units: the fp64 value of the passes above,
// times 2^k, to the nearest integer (the half is added in fp64 and the conversion cuts off: within 1/2 + 2^-20 of
// the scaled value); 2^32 - 1 and more (and NaN) become 2^32 - 1.  l and x come multiplied by Unit::pre.
__device__ __forceinline__ uint32_t err_units(double l0, double l1, double x0, double x1) {
  const double a = l0 - x0, b = l1 - x1;
  const double v = __builtin_fma(a, a, __builtin_fma(b, b, 0.5));
  return uint32_t(__builtin_fmin(v, 4294967295.0));
}

// One forward pass on 32-bit metrics.  kSym: free ends, the groups below 2048 only (a mirror group's metric is read
// from the group it mirrors), all 128 steps, and the best final group, its metric and the gap to the runner-up are left in sm.red32[0]; otherwise:
// start in group ov, steps 0 .. 126 (the last step's decision is taken by the trace-back from the metrics entering
// it).  The results of the even steps first_kept .. 126 (the metrics entering the next, odd step) go to hist.
// Metrics and error table are double-buffered in LDS (2 x 16 KB, 2 x 8 KB: the footprint of the fp64 arrays): a step
// reads the present buffers and writes the next metrics and the next step's table, so one barrier per step suffices;
// a thread keeps its four codebook entries in registers.
// kWide: 512 threads; the threads t and t + 256 share the eight groups of a column half, four each (slots 0..3 and
// 4..7), and the table's 1024 entries two each instead of four.
template <bool kSym, bool kWide>
__device__ __forceinline__ void forward_pass32(Smem& sm, const double* __restrict__ entry_d, int roll, int ov,
                                               uint32_t* __restrict__ hist, int first_kept, const Unit unit) {
  constexpr int kT = kWide ? 2 * kThreads : kThreads, kSlotsOwn = kWide ? 4 : 8, kEnt = 1024 / kT;
  const int tfull = kWide ? opaque_tid_wide() : opaque_tid();
  const int tid = tfull & (kThreads - 1), upper = kWide ? tfull >> 8 : 0;
  const int colA = 4 * (tid & 31) + ((tid >> 5) & 3), colB = 255 - colA;
  const int half = tid >> 7;
  // Tail-biting pass: table [2][32 positions][64 rows] in sm.E, metrics [2][4096] in sm.M.  Free pass: the same 48 KB
  // hold the table as pairs of neighbouring positions, [2][2 parities][16 pairs][64 rows] x 8 bytes (a lane reads its
  // 16 positions as eight 8-byte pieces, 333 against 250 B/ns for two-dword reads; parity 0 pairs the positions
  // (2p, 2p + 1), parity 1 (2p + 1, 2p + 2), the 8 pairs stored twice for the wrap-around), then the compact
  // metrics [2][2048].
  constexpr int kEPairWords = 2 * 16 * 64 * 2, kMcSlots = kGroups / 2;
  uint32_t* const E32 = reinterpret_cast<uint32_t*>(sm.E);
  uint32_t* const M32 = kSym ? E32 + 2 * kEPairWords : reinterpret_cast<uint32_t*>(sm.M);
  static_assert(sizeof(sm.E) >= 2 * kESlots * sizeof(uint32_t) && sizeof(sm.M) >= 2 * kMSlots * sizeof(uint32_t));
  static_assert(offsetof(Smem, M) == sizeof(sm.E) &&
                sizeof(sm.E) + sizeof(sm.M) >= (2 * kEPairWords + 2 * kMcSlots) * sizeof(uint32_t));
  // The table entries (position, row) = entry index position * 64 + row a thread forms each step.  Tail-biting
  // pass: entry t + kT q.  Free pass: row (t % 16) + 16 (t / 32 % 4), positions 2 (t / 128 + (kT / 128) q) + (t / 16
  // % 2): the 32 lanes of a half-wave then hold both halves of 16 rows' pairs and write 32 different banks.
  const int e_row = (tfull & 15) | (((tfull >> 5) & 3) << 4), e_h = (tfull >> 4) & 1, e_a = tfull >> 7;
  const int e_wr = kSym ? (2 * e_a + e_h) * 64 + e_row : tfull;
  double2 ent[kEnt];
  const double2* __restrict__ entries = reinterpret_cast<const double2*>(entry_d) + e_wr;
#pragma unroll
  for (int q = 0; q < kEnt; ++q) ent[q] = entries[kT * q], ent[q].x *= unit.pre, ent[q].y *= unit.pre;
  // free pass, words: parity 0 holds position 2a + h in pair a, half h; parity 1 in pair a - 1 + h, the other half
  const int e_wr0 = (e_a * 64 + e_row) * 2 + e_h;
  const int e_wr1 = ((16 + e_a - 1 + e_h) * 64 + e_row) * 2 + (e_h ^ 1);
  int ebase[kSlotsOwn], wslot[kSlotsOwn];  // of the slots m0 .. m0 + kSlotsOwn - 1, m0 = 4 upper
#pragma unroll
  for (int i = 0; i < kSlotsOwn; ++i) {
    const uint32_t j = 16u * colA + 8u * uint32_t(half) + uint32_t(i + 4 * upper), p = j * (j + 1u);
    const int pos0 = int((p >> 12) & 15u), row = int((p >> 6) & 63u);
    if constexpr (kSym) {
      ebase[i] = (((pos0 & 1) * 16 + (pos0 >> 1)) * 64 + row) * 2;  // words: parity, first pair, row
      wslot[i] = m32c_slot(int(j & 255u), int(j >> 8));
    } else {
      ebase[i] = pos0 * 64 + row;
      wslot[i] = m32_slot(int(j & 255u), int(j >> 8));
    }
  }
  // bytes
  int xA = kSym ? m32c_pos(colA) * 32 + m32c_swz(colA) * 4 : m32_pos(colA) * 64 + m32_swz(colA) * 4;
  int xB = kSym ? m32c_pos(colB) * 32 + m32c_swz(colB) * 4 : m32_pos(colB) * 64 + m32_swz(colB) * 4;
  // the error table of step `it` into table buffer it & 1 (given as a constant: the buffers' offsets then are part
  // of the instructions)
  auto table = [&](int it, auto par_tag) __attribute__((always_inline)) {
    constexpr int tpar = decltype(par_tag)::value;
    const int t = (2 * it + roll) & 255;
    const double x0 = double(sm.x[t]) * unit.pre, x1 = double(sm.x[t + 1]) * unit.pre;

    if constexpr (kSym) {
      // Parity 0: pair position / 2, half position % 2; parity 1: pair floor((position - 1) / 2), the other half;
      // pair -1, which position 0 asks for, is pair 15 of parity 0, which like itself nobody reads.  Every pair a
      // second time 8 further on.  Both addresses advance by kT words per q (kT / 128 pairs).
      uint32_t* const Ew0 = E32 + tpar * kEPairWords + e_wr0;
      uint32_t* const Ew1 = E32 + tpar * kEPairWords + e_wr1;
#pragma unroll
      for (int q = 0; q < kEnt; ++q) {
        const double2 l = ent[q];
        const uint32_t v = err_units(l.x, l.y, x0, x1);
        Ew0[kT * q] = v;
        Ew0[kT * q + 8 * 128] = v;
        Ew1[kT * q] = v;
        Ew1[kT * q + 8 * 128] = v;
      }
    } else {
      uint32_t* const Ew = E32 + tpar * kESlots + e_wr;
#pragma unroll
      for (int q = 0; q < kEnt; ++q) {
        const double2 l = ent[q];
        const uint32_t v = err_units(l.x, l.y, x0, x1);
        Ew[kT * q] = v;
        Ew[kT * q + 1024] = v;
      }
    }
  };
  if constexpr (kSym) {
    for (int g = tfull; g < kMcSlots; g += kT) M32[g] = 0u;
  } else {
    for (int g = tfull; g < kGroups; g += kT) M32[m32_slot(g & 255, g >> 8)] = (ov < 0 || g == ov) ? 0u : kSat;
  }
  table(0, std::integral_constant<int, 0>{});
  __syncthreads();

  uint32_t fin[kSlotsOwn];
  // step `it`: metrics of buffer it & 1 and table buffer it & 1 -> metrics of buffer (it + 1) & 1; par = it & 1
  auto step = [&](int it, auto kind_tag, auto par_tag) __attribute__((always_inline)) {
    constexpr int kind = decltype(kind_tag)::value;  // kDigits: the free pass's last step, results to fin only
    constexpr int par = decltype(par_tag)::value;
    uint32_t* hs = nullptr;
    if constexpr (kind == kStore) hs = hist + size_t(it >> 1) * kGroups + tid;
    constexpr int kMBuf = kSym ? kMcSlots : kMSlots, kEBuf = kSym ? kEPairWords : kESlots;
    const char* const Mb = reinterpret_cast<const char*>(M32 + par * kMBuf);
    uint32_t* const Mw = M32 + (par ^ 1) * kMBuf;
    const uint32_t* const Er = E32 + par * kEBuf;
    uint32_t MA[16], MB[16];
    asm volatile("" : "+v"(xA), "+v"(xB));
    if constexpr (kSym) {
      // digits 0..7 of the own column, and digits 8..15 as digits 7..0 of the mirror column
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        const uint4 a = *reinterpret_cast<const uint4*>(Mb + (xA ^ (16 * k)));
        MA[4 * k] = a.x, MA[4 * k + 1] = a.y, MA[4 * k + 2] = a.z, MA[4 * k + 3] = a.w;
        const uint4 b = *reinterpret_cast<const uint4*>(Mb + (xB ^ (16 * k)));
        MA[15 - 4 * k] = b.x, MA[14 - 4 * k] = b.y, MA[13 - 4 * k] = b.z, MA[12 - 4 * k] = b.w;
      }
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const uint4 a = *reinterpret_cast<const uint4*>(Mb + (xA ^ (16 * k)));
        MA[4 * k] = a.x, MA[4 * k + 1] = a.y, MA[4 * k + 2] = a.z, MA[4 * k + 3] = a.w;
        const uint4 b = *reinterpret_cast<const uint4*>(Mb + (xB ^ (16 * k)));
        MB[4 * k] = b.x, MB[4 * k + 1] = b.y, MB[4 * k + 2] = b.z, MB[4 * k + 3] = b.w;
      }
    }
    if constexpr (kind != kDigits) table(it + 1, std::integral_constant<int, par ^ 1>{});
    // The 16 table values of a slot are fetched while the slot before it is worked on; the value of digit k of slot
    // m lies (k (2 m + 1)) % 16 positions after the slot's first.  m0: the first slot of this thread, a constant in
    // each of the two copies of the loop that the wide form needs.  Tail-biting pass: evb[.][k] is the value of digit
    // k (the offsets of the reads are permuted); free pass: evb[.][t] is the value t positions after the first
    // (eight 8-byte reads, kept apart: the paired form of the read is the slower one), digit k reads it at
    // (k (2 m + 1)) % 16.
    auto slots = [&](auto m0_tag) __attribute__((always_inline)) {
    constexpr int m0 = decltype(m0_tag)::value;
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    uint32_t evb[2][kSym ? 1 : 16];  // tail-biting pass: 16 values
    u32x2 evp[2][kSym ? 8 : 1];      // free pass: 8 pieces of two neighbouring positions
    auto fetch = [&](int own, int gn, int buf) __attribute__((always_inline)) {
      const uint32_t* er = Er + ebase[own];
      if constexpr (kSym) {
        // written out, so that the eight reads stay eight: the compiler would pair them (ds_read2st64_b64), and the
        // paired read moves fewer bytes per cycle than two single ones.  It does not know of their latency either:
        // the wait below is what the uses of the values depend on.
        const uint32_t a = uint32_t(reinterpret_cast<size_t>(er));
#define QTIP_READ_PAIR(I) asm volatile("ds_read_b64 %0, %1 offset:" #I "*512" : "=v"(evp[buf][I]) : "v"(a));
        QTIP_READ_PAIR(0) QTIP_READ_PAIR(1) QTIP_READ_PAIR(2) QTIP_READ_PAIR(3)
        QTIP_READ_PAIR(4) QTIP_READ_PAIR(5) QTIP_READ_PAIR(6) QTIP_READ_PAIR(7)
#undef QTIP_READ_PAIR
      } else {
#pragma unroll
        for (int k = 0; k < 16; ++k) evb[buf][k] = er[((k * gn) & 15) * 64];
      }
    };
    fetch(0, 2 * m0 + 1, 0);
#pragma unroll
    for (int i = 0; i < kSlotsOwn; ++i) {
      constexpr int kLast = kSlotsOwn - 1;
      const int m = i;  // index into this thread's own slots
      if (i < kLast) fetch(i < kLast ? i + 1 : kLast, 2 * (m0 + i + 1) + 1, (i + 1) & 1);
      const uint32_t* ev = evb[i & 1];
      u32x2* ep = evp[i & 1];
      if constexpr (kSym) {
        // the reads of this slot's values are done when at most the eight issued after them (the next slot's) are
        // outstanding: LDS operations complete in order
#define QTIP_EP8 "+v"(ep[0]), "+v"(ep[1]), "+v"(ep[2]), "+v"(ep[3]), "+v"(ep[4]), "+v"(ep[5]), "+v"(ep[6]), "+v"(ep[7])
        if (i < kLast) asm volatile("s_waitcnt lgkmcnt(8)" : QTIP_EP8);
        else asm volatile("s_waitcnt lgkmcnt(0)" : QTIP_EP8);
#undef QTIP_EP8
      }
      const int g = 2 * (m0 + i) + 1;
      // the table value of digit k
      auto at = [&](int k) -> uint32_t {
        if constexpr (kSym) {
          const int t = (k * g) & 15;
          return (t & 1) ? ep[t >> 1].y : ep[t >> 1].x;
        } else {
          return ev[k];
        }
      };
      // the table value of digit k is the candidate of digit k of the group and of digit 15 - k of its mirror
      uint32_t ba = kSat;
#pragma unroll
      for (int k = 0; k < 8; ++k) ba = min3u(ba, sat_add(at(2 * k), MA[2 * k]), sat_add(at(2 * k + 1), MA[2 * k + 1]));
      uint32_t bb = ba;
      if constexpr (!kSym) {
        bb = kSat;
#pragma unroll
        for (int k = 0; k < 8; ++k)
          bb = min3u(bb, sat_add(ev[2 * k], MB[15 - 2 * k]), sat_add(ev[2 * k + 1], MB[14 - 2 * k]));
      }
      if constexpr (kind == kDigits) {
        fin[m] = ba;
      } else {
        Mw[wslot[m]] = ba;
        if constexpr (!kSym) Mw[wslot[m] ^ kMirror32] = bb;
      }
      if constexpr (kind == kStore) {
        hs[(m0 + m) * kThreads] = ba;
        if constexpr (!kSym) hs[(8 + m0 + m) * kThreads] = bb;
      }
    }
    };
    if constexpr (!kWide) {
      slots(std::integral_constant<int, 0>{});
    } else {
      if (upper) slots(std::integral_constant<int, 4>{});
      else slots(std::integral_constant<int, 0>{});
    }
    __syncthreads();
  };
  using Plain = std::integral_constant<int, kPlain>;
  using Store = std::integral_constant<int, kStore>;
  using Last = std::integral_constant<int, kDigits>;
  using Even = std::integral_constant<int, 0>;
  using Odd = std::integral_constant<int, 1>;
  static_assert((kSteps - 1) % 2 == 1, "steps 0 .. kSteps - 2 are pairs and one more even step");
  // two steps per turn, so that a step's parity is a constant (first_kept is even: the kept steps are even ones)
#pragma nounroll
  for (int it = 0; it < kSteps - 2; it += 2) {
    if (it >= first_kept) step(it, Store{}, Even{});
    else step(it, Plain{}, Even{});
    step(it + 1, Plain{}, Odd{});
  }
  step(kSteps - 2, Store{}, Even{});
  if constexpr (kSym) {
    step(kSteps - 1, Last{}, Odd{});
    // Best final group among the groups below 2048 (each stands for a pair of complementary states), and the best
    // among the groups of other columns (j >> 4): the 16 groups of a column end in final states that differ in their
    // last digit only where they come from the same predecessor, and which of those wins changes nothing that is
    // traced back; the trace-back looks at the winner's column itself.  A partial result is (best value, its
    // smallest group, best value outside that group's column); a thread's own groups are one column.
    uint32_t b1 = kSat, b2 = kSat, bj = 0;
#pragma unroll
    for (int m = 0; m < kSlotsOwn; ++m) {
      const uint32_t v = fin[m], j = 16u * colA + 8u * uint32_t(half) + uint32_t(m + 4 * upper);
      const bool take = v < b1;
      bj = take ? j : bj;
      b1 = take ? v : b1;
    }
    auto merge = [&](uint32_t o1, uint32_t o2, uint32_t oj) {
      const bool same = (oj >> 4) == (bj >> 4);
      const bool take = o1 < b1 || (o1 == b1 && oj < bj);  // equal metrics: same choice in both lanes
      const uint32_t out = take ? min(o2, b1) : min(b2, o1);
      b2 = same ? min(b2, o2) : out;
      bj = take ? oj : bj;
      b1 = take ? o1 : b1;
    };
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) merge(__shfl_xor(b1, off, 64), __shfl_xor(b2, off, 64), __shfl_xor(bj, off, 64));
    if ((tfull & 63) == 0) sm.red32[tfull >> 6][0] = b1, sm.red32[tfull >> 6][1] = b2, sm.red32[tfull >> 6][2] = bj;
    __syncthreads();
    b1 = sm.red32[0][0], b2 = sm.red32[0][1], bj = sm.red32[0][2];
#pragma unroll
    for (int w = 1; w < kT / 64; ++w) merge(sm.red32[w][0], sm.red32[w][1], sm.red32[w][2]);
    __syncthreads();
    if (tfull == 0) sm.red32[0][0] = b1, sm.red32[0][1] = b2 - b1, sm.red32[0][2] = bj;
    __syncthreads();
  }
}

__device__ __forceinline__ uint32_t row_min16_u32(uint32_t c) {
#define QTIP_ROW_STEP32(CTRL) c = min(c, uint32_t(__builtin_amdgcn_update_dpp(0, int(c), CTRL, 0xf, 0xf, false)));
  QTIP_ROW_STEP32(0xB1)   // quad_perm [1, 0, 3, 2]
  QTIP_ROW_STEP32(0x4E)   // quad_perm [2, 3, 0, 1]
  QTIP_ROW_STEP32(0x141)  // row_half_mirror
  QTIP_ROW_STEP32(0x140)  // row_mirror
#undef QTIP_ROW_STEP32
  return c;
}

// Trace-back of a 32-bit pass, the scheme of trace_back above with the runner-up of every decision looked at as well.
// j_last: low 12 bits of the final state (the group the pass ends in; for a free pass the best group, of which the
// column counts).  The decision of step 127 is taken from the metrics entering it (kept slot 63), then two steps
// per round trip.  flag is raised (in every thread alike) when a
// decision is won by less than thr units or the winner is not below kWinnerMax.
// Returns the state of step it_min - 1; record: the states of the steps walked are written to sm.st.
// kStream (the 512-thread form, whose workgroup has its compute unit to itself): which 256 of a kept step's values a
// round reads is known only when the round before it is decided, so fetched on demand every round waits for HBM.
// Whole kept steps are streamed into LDS ahead of the rounds instead (the metric and table arrays are idle now:
// 48 KB, three steps of 4096 values or six of the 2048 a free pass keeps; direct-to-LDS loads, every wave a share of
// a step, as many steps in flight as there are buffers beside the one in use), and the codebook is read from a
// 2 KB table of fp16 pairs in LDS (tl), so that no other vector-memory load waits in line behind the streamed ones.
// Beside other workgroups the streamed form loses more in their forward passes than it gains (measured), so the
// 256-thread form fetches on demand.
template <bool kSym, bool kStream>
__device__ __forceinline__ uint32_t trace_back32(Smem& sm, const double* __restrict__ entry_d,
                                                 const uint32_t* __restrict__ hist, int roll, uint32_t j_last,
                                                 int it_min, bool record, uint32_t thr, uint32_t& flag,
                                                 const uint32_t* tl, const Unit unit) {
  const uint32_t tid = uint32_t(opaque_tid());
  const uint32_t lane = tid & 63u, wave = tid >> 6, dp = lane & 15u, d = 4u * wave + (lane >> 4);
  // streamed form: kept steps 63, 62, ..., it_min / 2 - 1 are the rows q = 0, 1, ... of a ring of kBufs buffers
  constexpr int kRowWords = kSym ? kGroups / 2 : kGroups, kBufs = kSym ? 6 : 3;
  constexpr int kLoads = kStream ? kRowWords / (4 * 2 * kThreads) : 1;  // 16-byte loads per thread and row, 512 threads
  static_assert(sizeof(sm.E) + sizeof(sm.M) >= size_t(kBufs) * kRowWords * 4 && offsetof(Smem, M) == sizeof(sm.E));
  static_assert((kBufs - 2) * kLoads <= 15, "the count of outstanding loads must fit the low four bits of the wait");
  uint32_t* const rows = reinterpret_cast<uint32_t*>(sm.E);
  const int count = 65 - it_min / 2;
  int issued = 0, q = 0;  // rows requested so far; the row in use
  typedef __attribute__((address_space(3))) void* lds_ptr;
  auto issue = [&](int row) {
    const uint32_t wave8 = threadIdx.x >> 6;  // all eight waves bring a share
    const uint32_t* g = hist + size_t(63 - row) * kGroups + 4u * lane;
    uint32_t* l = rows + (row % kBufs) * kRowWords;
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const uint32_t w0 = (uint32_t(i) * 8u + wave8) * 256u;  // first word of this wave's 1 KB piece
      __builtin_amdgcn_global_load_lds(g + w0, (lds_ptr)(l + w0), 16, 0, 0);
    }
  };
  // this wave's loads of the rows up to the one wanted have landed: at most `later` rows requested after it are out
  auto landed = [&](int later) {
    if (kBufs >= 6 && later >= 4) __builtin_amdgcn_s_waitcnt(0x0F70 | (kBufs >= 6 ? 4 * kLoads : 0));
    else if (kBufs >= 5 && later == 3) __builtin_amdgcn_s_waitcnt(0x0F70 | (kBufs >= 5 ? 3 * kLoads : 0));
    else if (kBufs >= 4 && later == 2) __builtin_amdgcn_s_waitcnt(0x0F70 | (kBufs >= 4 ? 2 * kLoads : 0));
    else if (later >= 1) __builtin_amdgcn_s_waitcnt(0x0F70 | kLoads);
    else __builtin_amdgcn_s_waitcnt(0x0F70);
  };
  // The barrier of a round.  Streamed: one that orders LDS only (__syncthreads() would wait for the loads in flight);
  // before it this wave's share of the next row has landed, after it everyone's has, and the buffer of the row in
  // use, which nobody reads after the barrier, takes the row kBufs further on.
  auto round_barrier = [&]() {
    if constexpr (kStream) {
      const int later = issued - 2 - q;  // rows requested after the next one
      landed(later > 0 ? later : 0);
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      if (issued < count) issue(issued++);
      ++q;
    } else {
      __syncthreads();
    }
  };
  if constexpr (kStream) {
    for (; issued < kBufs && issued < count; ++issued) issue(issued);
    landed(issued - 1);
    __builtin_amdgcn_s_waitcnt(0xC07F);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  }
  // the metrics of kept step `slot` (the row in use, when streamed).  On demand: written by this workgroup's own waves
  // before the barrier that ended the forward pass, workgroup scope suffices
  auto kept = [&](int slot, uint32_t g) -> uint32_t {
    if constexpr (kStream) return rows[(q % kBufs) * kRowWords + hist32_index<kSym>(g)];
    else return __hip_atomic_load(hist + size_t(slot) * kGroups + hist32_index<kSym>(g), __ATOMIC_RELAXED,
                                  __HIP_MEMORY_SCOPE_WORKGROUP);
  };
  // (the forward pass's own arithmetic: the same products and sums on the same operands give the same integers)
  // the codebook entry of a state, and its error against two inputs
  auto entry_of = [&](uint32_t st, double& l0, double& l1) {
    const uint32_t e = ((st * (st + 1u)) >> 6) & 1023u;
    if constexpr (kStream) {
      const uint32_t w = tl[e & 511u];
      const uint16_t h0 = uint16_t((w & 0xffffu) ^ ((e >> 9) << 15)), h1 = uint16_t(w >> 16);
      l0 = double(float(__builtin_bit_cast(_Float16, h0))), l1 = double(float(__builtin_bit_cast(_Float16, h1)));
    } else {
      l0 = entry_d[2 * e], l1 = entry_d[2 * e + 1];
    }
  };
  auto err_at = [&](double l0, double l1, double x0, double x1) -> uint32_t {
    return err_units(l0 * unit.pre, l1 * unit.pre, x0 * unit.pre, x1 * unit.pre);
  };
  auto err_of = [&](uint32_t st, double x0, double x1) -> uint32_t {
    double l0, l1;
    entry_of(st, l0, l1);
    return err_at(l0, l1, x0, x1);
  };
  // over the 16 lanes of a row: the smallest value (returned), the first lane that holds it, the gap to the runner-up
  auto row_pick = [&](uint32_t c, uint32_t& first, uint32_t& gap) -> uint32_t {
    const uint32_t m = row_min16_u32(c);
    const unsigned long long at_min = __builtin_amdgcn_ballot_w64(c == m);
    const uint32_t bits = uint32_t(at_min >> (lane & 48u)) & 0xffffu;
    first = bits ? uint32_t(__builtin_ctz(bits)) : 0u;
    gap = row_min16_u32(dp == first ? kSat : c) - m;
    return m;
  };
  uint32_t s;
  if constexpr (!kSym) {  // step 127: the 16 states (digit << 12) | j_last, one per lane of a row; every row does the same
    const int t = (2 * (kSteps - 1) + roll) & 255;
    const double x0 = double(sm.x[t]), x1 = double(sm.x[t + 1]);
    const uint32_t st = (dp << 12) | j_last;
    const uint32_t c = sat_add(err_of(st, x0, x1), kept(63, st >> 4));
    uint32_t k, gap;
    const uint32_t m = row_pick(c, k, gap);
    flag |= uint32_t(gap < thr) | uint32_t(m >= kWinnerMax);
    s = (k << 12) | j_last;
    if (record && threadIdx.x == 0) sm.st[kSteps - 1] = uint16_t(s);
    if constexpr (kStream) round_barrier();
  } else {
    // Free pass: the final state is the best of all.  The forward pass has named the best group's column and
    // vouched for the distance to every other column; here the 256 final states of that column, (digit k << 12) |
    // column << 4 | last digit e, are weighed: row 4 wave + r of the workgroup takes k, its lanes the 16 e.  The
    // states of one k come from one predecessor, so only their best counts, and the decision to be won by thr units
    // is the one between the k: states that share k are traced back alike.
    const int t = (2 * (kSteps - 1) + roll) & 255;
    const double x0 = double(sm.x[t]), x1 = double(sm.x[t + 1]);
    const uint32_t col = j_last >> 4;
    const uint32_t st = (d << 12) | (col << 4) | dp;
    const uint32_t c = sat_add(err_of(st, x0, x1), kept(63, st >> 4));
    uint32_t e1, gap_unused;
    const uint32_t v = min(row_pick(c, e1, gap_unused), kSat);
    uint32_t bc = uint32_t(__builtin_amdgcn_readlane(int(v), 0)), sc = kSat, bk = 4u * wave;
    uint32_t be = uint32_t(__builtin_amdgcn_readlane(int(e1), 0));
#pragma unroll
    for (int r = 1; r < 4; ++r) {
      const uint32_t oc = uint32_t(__builtin_amdgcn_readlane(int(v), 16 * r));
      const uint32_t oe = uint32_t(__builtin_amdgcn_readlane(int(e1), 16 * r));
      const bool take = oc < bc;
      sc = take ? bc : min(sc, oc);
      bk = take ? 4u * wave + uint32_t(r) : bk;
      be = take ? oe : be;
      bc = take ? oc : bc;
    }
    if (lane == 0) {
      sm.tr32[1][wave][0] = bc;
      sm.tr32[1][wave][1] = sc;
      sm.tr32[1][wave][2] = bk | (be << 8);
    }
    round_barrier();
    bc = sm.tr32[1][0][0], sc = sm.tr32[1][0][1];
    uint32_t bke = sm.tr32[1][0][2];
#pragma unroll
    for (int w = 1; w < 4; ++w) {
      const uint32_t oc = sm.tr32[1][w][0], os = sm.tr32[1][w][1];
      const bool take = oc < bc;
      sc = take ? min(bc, os) : min(sc, oc);
      bke = take ? sm.tr32[1][w][2] : bke;
      bc = take ? oc : bc;
    }
    flag |= uint32_t(sc - bc < thr) | uint32_t(bc >= kWinnerMax);
    const uint32_t k = bke & 15u;
    s = (k << 12) | (col << 4) | ((bke >> 8) & 15u);
    if (k >= 8u) s = 65535u - s;  // the smaller state of the pair
    if (record && threadIdx.x == 0) sm.st[kSteps - 1] = uint16_t(s);
  }
  int set = 0;
#pragma nounroll
  for (int it = kSteps - 2; it >= it_min; it -= 2, set ^= 1) {
    const uint32_t j = s >> 4;
    const int ta = (2 * (it - 1) + roll) & 255, tb = (2 * it + roll) & 255;
    const double xa0 = double(sm.x[ta]), xa1 = double(sm.x[ta + 1]);
    const double xb0 = double(sm.x[tb]), xb1 = double(sm.x[tb + 1]);
    const uint32_t g = (d << 8) | (j >> 4);
    const uint32_t s1 = (dp << 12) | g;
    // A round's three loads all at once, the two codebook entries (cached) before the kept metric (from HBM): the
    // kept metric is read with an atomic load, which the compiler moves nothing across, so written in the order of
    // use a round would wait for one entry, then for the metric, then for the other entry.
    double la0, la1, lb0, lb1;
    entry_of(s1, la0, la1);
    entry_of((d << 12) | j, lb0, lb1);
    const uint32_t kv = kept(it / 2 - 1, s1 >> 4);
    const uint32_t c1 = sat_add(err_at(la0, la1, xa0, xa1), kv);
    uint32_t k1, gap1;
    // the metric of group g entering step it, as the forward pass had it
    const uint32_t m1 = min(row_pick(c1, k1, gap1), kSat);
    const uint32_t c0 = sat_add(err_at(lb0, lb1, xb0, xb1), m1);
    // every lane of row r holds that row's (c0, k1, gap1) for d = 4 wave + r: best and runner-up of the wave's four
    uint32_t bc = uint32_t(__builtin_amdgcn_readlane(int(c0), 0)), sc = kSat, bd = 4u * wave;
    uint32_t bd1 = uint32_t(__builtin_amdgcn_readlane(int(k1), 0)), bg = uint32_t(__builtin_amdgcn_readlane(int(gap1), 0));
#pragma unroll
    for (int r = 1; r < 4; ++r) {
      const uint32_t oc = uint32_t(__builtin_amdgcn_readlane(int(c0), 16 * r));
      const uint32_t od1 = uint32_t(__builtin_amdgcn_readlane(int(k1), 16 * r));
      const uint32_t og = uint32_t(__builtin_amdgcn_readlane(int(gap1), 16 * r));
      const bool take = oc < bc;
      sc = take ? bc : min(sc, oc);
      bd = take ? 4u * wave + uint32_t(r) : bd;
      bd1 = take ? od1 : bd1;
      bg = take ? og : bg;
      bc = take ? oc : bc;
    }
    if (lane == 0) {
      sm.tr32[set][wave][0] = bc;
      sm.tr32[set][wave][1] = sc;
      sm.tr32[set][wave][2] = bd | (bd1 << 8);
      sm.tr32[set][wave][3] = bg;
    }
    round_barrier();
    // The four waves' entries in four 16-byte reads, all asked for before the first is looked at: the values are the
    // same in every lane, and left to itself the compiler turns the choices below into branches around single
    // 4-byte reads, one LDS round trip after the other.
    uint4 q[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) q[w] = *reinterpret_cast<const uint4*>(sm.tr32[set][w]);
    asm volatile("" : "+v"(q[0].x), "+v"(q[0].y), "+v"(q[0].z), "+v"(q[0].w), "+v"(q[1].x), "+v"(q[1].y), "+v"(q[1].z),
                 "+v"(q[1].w), "+v"(q[2].x), "+v"(q[2].y), "+v"(q[2].z), "+v"(q[2].w), "+v"(q[3].x), "+v"(q[3].y),
                 "+v"(q[3].z), "+v"(q[3].w));
    bc = q[0].x, sc = q[0].y;
    uint32_t bdd = q[0].z;
    bg = q[0].w;
#pragma unroll
    for (int w = 1; w < 4; ++w) {
      const uint32_t oc = q[w].x, os = q[w].y;
      const bool take = oc < bc;
      sc = take ? min(bc, os) : min(sc, oc);
      bdd = take ? q[w].z : bdd;
      bg = take ? q[w].w : bg;
      bc = take ? oc : bc;
    }
    // (a candidate of step `it` is a sum of it + 1 rounded terms: what thr allows for 128 terms shrinks by one unit
    // per term less)
    const uint32_t fewer = uint32_t(kSteps - 1 - it), thr_it = thr - (fewer < thr ? fewer : thr);
    flag |= uint32_t(sc - bc < thr_it) | uint32_t(bg < thr_it) | uint32_t(bc >= kWinnerMax);
    const uint32_t s_it = ((bdd & 15u) << 12) | j;
    s = (((bdd >> 8) & 15u) << 12) | (s_it >> 4);
    if (record && threadIdx.x == 0) {
      sm.st[it] = uint16_t(s_it);
      sm.st[it - 1] = uint16_t(s);
    }
  }
  return s;
}

// kWide: 512 threads per tile, one workgroup per compute unit, for launches that cannot fill the chip anyway (a lone
// small group): a tile then takes about two thirds of the time.  Same results, bit for bit.
template <bool kWide>
__global__ __launch_bounds__(kWide ? 2 * kThreads : kThreads, kWide ? 1 : 3) void viterbi_tiles_kernel(
    TileJob job, const double* __restrict__ entry_d, const float* __restrict__ entry_f, double* __restrict__ hist_all) {
  __shared__ Smem sm;
  __shared__ uint32_t tl[kWide ? 512 : 1];  // wide form: the codebook's 512 value pairs as fp16 bits, for its trace-backs
  const int u = threadIdx.x & (kThreads - 1);
  const bool first_half = threadIdx.x < kThreads;  // global results are written once
  if constexpr (kWide) {  // the table's values are fp16 values (entry bit 9 is the sign of the first one)
    const int i = threadIdx.x;
    const uint32_t h0 = __builtin_bit_cast(uint16_t, _Float16(entry_f[2 * i]));
    const uint32_t h1 = __builtin_bit_cast(uint16_t, _Float16(entry_f[2 * i + 1]));
    tl[i] = h0 | (h1 << 16);
    __syncthreads();
  }
  double* hist = hist_all + size_t(blockIdx.x) * kHistWordsPerTile;
  for (long tile = blockIdx.x; tile < job.tiles; tile += gridDim.x) {
  float expected = 0.f;  // the free pass's winner of this tile row's previous column block (0: none yet)
  for (int blk = job.blocks - 1; blk >= 0; --blk) {
    // the column block of this turn; the hatWT values the previous turn wrote for this tile row are visible after
    // the barrier that ended it
    const long col0 = job.col0 + 16 * blk;
    if (job.X) sm.x[u] = job.X[tile * kSeq + u];
    else if (job.prod64) tile_targets<double>(sm, job, col0, tile, job.prod64);
    else tile_targets<float>(sm, job, col0, tile, job.prod32);
    __syncthreads();
    // pass 1 on the sequence rotated by half its length, free ends, traced back to step 64 for the overlap group;
    // pass 2 on the sequence itself, tail-biting through that group, traced back in full.  One loop, so that the
    // step bodies exist once in the instruction cache.
    int ov = -1;
#pragma nounroll
    for (int pass = 0; pass < 2; ++pass) {
      const int roll = pass == 0 ? kSeq / 2 : 0;
      bool done = false;
      if (job.mode == 0) {
        uint32_t* const hist32 = reinterpret_cast<uint32_t*>(hist);
        uint32_t flag = 0;
        // (the same in every thread; said so, so that it lives in scalar registers)
        const int unit_log2 = __builtin_amdgcn_readfirstlane(unit_log2_for(expected, pass == 0 ? 2.f : 1.125f));
        const Unit unit = unit_of(unit_log2);
        if (pass == 0) {
          forward_pass32<true, kWide>(sm, entry_d, roll, -1, hist32, 62, unit);
          const uint32_t winner = sm.red32[0][0];
          flag |= uint32_t(sm.red32[0][1] < job.margin) | uint32_t(winner >= kWinnerMax);
          const uint32_t s = trace_back32<true, kWide>(sm, entry_d, hist32, roll, sm.red32[0][2], 64, false, job.margin, flag, tl, unit);
          if (!flag && u == 0) sm.overlap = int(s & 0xfffu);  // s is the state of step 63
          // what the tail-biting pass of this block and the free pass of the next may expect (a winner that did
          // not fit is replaced by the true one when the pass is repeated on fp64 metrics)
          expected = __builtin_ldexpf(float(winner), -unit_log2);
        } else {
          forward_pass32<false, kWide>(sm, entry_d, roll, ov, hist32, 0, unit);
          const uint32_t s = trace_back32<false, kWide>(sm, entry_d, hist32, roll, uint32_t(ov), 2, true, job.margin, flag, tl, unit);
          // s is the state of step 1; at step 0 the one predecessor group with a finite initial metric is ov
          if (!flag && u == 0) sm.st[0] = uint16_t((s >> 4) | ((uint32_t(ov) >> 8) << 12));
        }
        done = !flag;
        if (flag && threadIdx.x == 0 && job.stats) atomicAdd(job.stats + pass, 1u);
      }
      if (!done) {
      forward_pass(sm, entry_d, roll, ov, hist, pass == 0 ? 62 : 0);
      if (pass == 0) expected = sm.final_metric;  // the true winner, also where a 32-bit pass could not hold it
      {
        const uint32_t s_last = sm.final_state;  // state of step 127
        const uint32_t s = trace_back(sm, entry_d, hist, roll, s_last, pass == 0 ? 64 : 2, pass == 1);
        if (u == 0) {
          if (pass == 0) {
            // s is the state of step 63: its low 12 bits are the high 12 bits of the state of step 64
            sm.overlap = int(s & 0xfffu);
          } else {
            // s is the state of step 1; at step 0 the one predecessor group with a finite initial metric is ov
            sm.st[kSteps - 1] = uint16_t(s_last);
            sm.st[0] = uint16_t((s >> 4) | ((uint32_t(ov) >> 8) << 12));
          }
        }
      }
      }
      __syncthreads();
      ov = sm.overlap;
    }
    // ---- outputs
    if (job.states && first_half && u < kSteps) job.states[(tile * job.q_tile_stride + job.q_offset + blk) * kSteps + u] = sm.st[u];
    if (job.packed && first_half && u < kWords) {
      uint32_t v;
      if (u == 0) v = sm.st[0];
      else {
        v = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) v = (v << 4) | (sm.st[4 * u + k - 3] & 15u);
      }
      job.packed[tile * kWords + u] = uint16_t(v);
    }
    if (job.hatWT && first_half) {
      const uint32_t s = sm.st[u >> 1];
      const uint32_t e = ((s * (s + 1u)) >> 6) & 1023u;
      const int q = perm_fwd(u), r = q >> 4, c = q & 15;
      const long wi = (col0 + c) * job.ldw + tile * 16 + r;
      const float hv = entry_f[2 * e + (u & 1)];
      job.hatWT[wi] = hv;
      if (job.dimg_h) {
        uint32_t hi, lo;
        bf16_split_bits(job.WT[wi] - hv, hi, lo);
        const long di = (tile * 16 + r) * job.ldd + col0 + c;
        job.dimg_h[di] = uint16_t(hi), job.dimg_l[di] = uint16_t(lo);
      }
    }
    __syncthreads();
  }
  }
}

// One wave that returns after `ticks` of the constant-rate clock (100 MHz), or after a bounded number of looks at it.
__global__ void delay_kernel(unsigned long long ticks) {
  const unsigned long long t0 = wall_clock64();
  for (int i = 0; i < (1 << 22) && wall_clock64() - t0 < ticks; ++i) __builtin_amdgcn_s_sleep(32);
}

__global__ void decode_states_kernel(const uint16_t* __restrict__ st, long count, float* __restrict__ hat,
                                     const float* __restrict__ entry_f) {
  const long i = long(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= count) return;
  const uint32_t s = st[i];
  const uint32_t e = ((s * (s + 1u)) >> 6) & 1023u;
  hat[2 * i] = entry_f[2 * e];
  hat[2 * i + 1] = entry_f[2 * e + 1];
}

}  // namespace

size_t viterbi_workspace_bytes(int slots) { return size_t(slots) * kHistWordsPerTile * sizeof(double); }

// workgroup slots of the 256-thread kernel on `device`, which must be current (found once per device)
int viterbi_max_slots(int device) {
  static std::mutex mu;
  static int cached[kMaxDevices] = {0};
  const bool tracked = device >= 0 && device < kMaxDevices;
  std::lock_guard<std::mutex> lock(mu);
  if (tracked && cached[device]) return cached[device];
  hipDeviceProp_t prop;
  QTIP_HIP(hipGetDeviceProperties(&prop, device));
  int per_cu = 0;
  QTIP_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, viterbi_tiles_kernel<false>, kThreads, 0));
  if (per_cu < 1) per_cu = 1;
  const int slots = per_cu * prop.multiProcessorCount;
  if (tracked) cached[device] = slots;
  return slots;
}

static int viterbi_device_slots() {
  int dev = 0;
  QTIP_HIP(hipGetDevice(&dev));
  return viterbi_max_slots(dev);
}

void launch_viterbi_tiles(const TileJob& job, const double* d_entry_d, const float* d_entry_f, void* workspace,
                          int slots, hipStream_t s, hipEvent_t start, hipEvent_t stop) {
  if (job.tiles <= 0) return;
  QTIP_REQUIRE(slots > 0 && workspace != nullptr, "viterbi: missing workspace");
  if (!job.X) {  // LDLQ block: the targets come from the feedback operands
    QTIP_REQUIRE(job.WT && job.L && job.hatWT && ((job.prod64 != nullptr) != (job.prod32 != nullptr)),
                 "viterbi: neither inputs nor complete LDLQ feedback operands");
    QTIP_REQUIRE((job.dimg_h != nullptr) == (job.dimg_l != nullptr) && (!job.dimg_h || job.ldd >= job.col0 + 16L * job.blocks),
                 "viterbi: residual images need both parts and rows that hold the block's columns");
    const long nk = job.bufend - job.col0 - 16;
    QTIP_REQUIRE(job.col0 >= 0 && nk >= 0 && nk <= 112 && job.blocks >= 1 && job.col0 + 16 * job.blocks <= job.bufend,
                 "viterbi: column blocks outside their 128-column buffer");
    QTIP_REQUIRE(job.col0 >= job.prod_row0 && job.ldw >= 16 * job.tiles && job.ldl >= job.bufend,
                 "viterbi: LDLQ operand geometry");
  }
  QTIP_REQUIRE(job.blocks == 1 || (!job.X && !job.packed), "viterbi: several blocks per tile row only for LDLQ launches");
  const unsigned grid = unsigned(job.tiles < slots ? job.tiles : slots);
  // the wide form where the launch leaves two thirds of the chip's workgroup slots empty anyway (and the 32-bit
  // passes, which are what it shares out over its 512 threads, are in use)
  const bool wide = job.mode == 0 && (job.wide > 0 || (job.wide < 0 && 3 * job.tiles <= viterbi_device_slots()));
  const auto kernel = wide ? viterbi_tiles_kernel<true> : viterbi_tiles_kernel<false>;
  const dim3 block(wide ? 2 * kThreads : kThreads);
  if (start || stop) {
    // the runtime stamps the two events at the kernel's own start and end: the time between them is the kernel's,
    // however late the host got round to queueing it
    hipExtLaunchKernelGGL(kernel, dim3(grid), block, 0, s, start, stop, 0, job, d_entry_d, d_entry_f,
                          static_cast<double*>(workspace));
  } else {
    kernel<<<dim3(grid), block, 0, s>>>(job, d_entry_d, d_entry_f, static_cast<double*>(workspace));
  }
  QTIP_HIP(hipGetLastError());
}

int viterbi_static_slots() { return kStaticSlots; }

void viterbi_static_scratch_init(int device) {
  QTIP_REQUIRE(device >= 0 && device < kMaxDevices, "device %d: the static Viterbi scratch is tracked for devices 0..%d",
               device, kMaxDevices - 1);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[device]) return;
  int cur = -1;
  QTIP_HIP(hipGetDevice(&cur));
  QTIP_REQUIRE(cur == device, "static scratch: device %d must be current (current: %d)", device, cur);
  void* p = nullptr;
  QTIP_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
  QTIP_REQUIRE(p != nullptr, "static scratch: no device address on device %d", device);
  g_scratch_ptr[device] = static_cast<double*>(p);
}

void* viterbi_static_scratch(int device) {
  if (device < 0 || device >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  return g_scratch_ptr[device];
}

void launch_delay(double microseconds, hipStream_t s) {
  if (microseconds <= 0) return;
  delay_kernel<<<dim3(1), dim3(64), 0, s>>>((unsigned long long)(microseconds * 100.0));
  QTIP_HIP(hipGetLastError());
}

void launch_decode_states(const uint16_t* states, long B, float* hat, const float* d_entry_f, hipStream_t s) {
  const long count = B * kSteps;
  if (count <= 0) return;
  decode_states_kernel<<<dim3(unsigned((count + 255) / 256)), dim3(256), 0, s>>>(states, count, hat, d_entry_f);
  QTIP_HIP(hipGetLastError());
}

}  // namespace qtipmi
