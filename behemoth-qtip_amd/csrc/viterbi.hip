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
// 160 LDS reads for 256 add-compare-selects.
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
//   * The metric of (column c, digit d) sits at c*16 + (pi(d) ^ ((c >> 2) & 15) ^ (c >> 6)) with
//     pi(d) = 4 (d & 3) + (d >> 2): the 16 lanes of a quarter read 16 different bank pairs for every d, write 16
//     different ones for every slot, a read address is one XOR of a per-lane base with a constant, and the mirror
//     group's slot is the group's XOR 0xff3.
// LDS per workgroup ~50 KB, three workgroups per CU; metrics single-buffered (the columns are read into registers
// before the step's results are written).
// Back-pointers (4 bits per group and step) go to HBM as one 64-bit word per thread and step, 2 KB per step,
// fully coalesced; the first pass only keeps the steps its half-length trace-back needs.
#include <hip/hip_ext.h>

#include <type_traits>

#include "qtip_internal.hpp"

namespace qtipmi {
namespace {

constexpr int kThreads = 256;
constexpr int kESlots = 32 * 64;                 // E[q][row]: 16 entry positions stored twice x 64 rows
constexpr int kMSlots = 4096;                    // metric of (column c, digit d) at m_slot(c, d)
constexpr int kBpWordsPerTile = 127 * kThreads;  // u64 words

__device__ __forceinline__ constexpr int pi16(int d) { return 4 * (d & 3) + (d >> 2); }
__device__ __forceinline__ int m_swz(int col) { return ((col >> 2) & 15) ^ (col >> 6); }
__device__ __forceinline__ int m_slot(int col, int d) { return col * 16 + (pi16(d) ^ m_swz(col)); }

struct Smem {
  double E[kESlots];  // first: its reads use 8-bit immediate offsets from a per-lane base
  double M[kMSlots];
  float x[kSeq];
  uint16_t st[kSteps];
  double red_c[4];
  uint32_t red_s[4];
  int overlap;
  uint32_t final_state;
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
// predecessor digit of group j from one step's 256 back-pointer words (word index = owning thread, so that a
// wave's 64 words are one contiguous 512-byte store; nibble m for the group itself, nibble 8 + m for a mirror
// group j >= 2048).  Read past the vector L1, which may still hold the previous tile's words.
__device__ __forceinline__ uint32_t bp_lookup(const unsigned long long* step_words, uint32_t j) {
  const uint32_t jj = j < 2048u ? j : 4095u - j;
  const uint32_t shift = (jj & 7u) * 4u + (j < 2048u ? 0u : 32u);
  const unsigned long long w = __hip_atomic_load(step_words + owner_thread(jj), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return uint32_t(w >> shift) & 15u;
}

// One forward pass over the 128 steps.  roll: input rotation (128 for the first pass).  ov < 0: free start and
// end; otherwise start in states with (s >> 4) == ov and end in the state of group ov.
// bp: this workgroup's back-pointer words; steps < bp_first are not stored.  Returns nothing; the final state
// is left in sm.final_state.
__device__ __forceinline__ void forward_pass(Smem& sm, const double* __restrict__ entry_d, int roll, int ov,
                                             unsigned long long* __restrict__ bp, int bp_first) {
  const int tid = threadIdx.x;
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
  constexpr int kMirror = 0xff3;
#pragma unroll
  for (int m = 0; m < 8; ++m) {
    const uint32_t j = 16u * colA + 8u * uint32_t(half) + m, p = j * (j + 1u);
    ebase[m] = int((p >> 12) & 15u) * 64 + int((p >> 6) & 63u);
    wslot[m] = m_slot(int(j & 255u), int(j >> 8));
  }
  // byte offsets of digit pi^-1(0) of the two metric columns; the other digits are XORs with 8 pi(d)
  int xA = colA * 128 + m_swz(colA) * 8, xB = colB * 128 + m_swz(colB) * 8;
  const char* const Mb = reinterpret_cast<const char*>(sm.M);

  // initial metrics: M_0[g] = 0, or +inf outside group ov
  for (int g = tid; g < kGroups; g += kThreads) {
    sm.M[m_slot(g & 255, g >> 8)] = (ov < 0 || g == ov) ? 0.0 : INF;
  }
  __syncthreads();

  unsigned long long word = 0;
  // one trellis step; DIGITS: the step's back-pointers are wanted (without them a candidate costs an add and a min)
  auto step = [&](int it, auto digits_tag) __attribute__((always_inline)) {
    constexpr bool digits = decltype(digits_tag)::value;
    // ---- phase R: metric columns -> registers, error table of this step -> LDS
    double MA[16], MB[16];
    // the 32 read addresses are recomputed in every step (one XOR each): kept across the loop they would take 32
    // registers the accumulators need
    asm volatile("" : "+v"(xA), "+v"(xB));
#pragma unroll
    for (int d = 0; d < 16; ++d) {
      MA[d] = *reinterpret_cast<const double*>(Mb + (xA ^ (8 * pi16(d))));
      MB[d] = *reinterpret_cast<const double*>(Mb + (xB ^ (8 * pi16(d))));
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
      // the same without the digit, for the steps whose back-pointers nobody reads (first half of the first pass)
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
      word |= (unsigned long long)(da) << (4 * m);
      word |= (unsigned long long)(db) << (32 + 4 * m);
    }
    if (digits && it < kSteps - 1) bp[size_t(it) * kThreads + tid] = word;
    __syncthreads();
  };
  for (int it = 0; it < bp_first; ++it) step(it, std::false_type{});
  for (int it = bp_first; it < kSteps; ++it) step(it, std::true_type{});
  // final state: smallest metric, then smallest state, over the metrics of the last step (each lane re-reads the
  // 16 values it has just written; their predecessor digits are the nibbles of the last back-pointer word)
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
      sm.final_state = s;
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
__device__ __forceinline__ void tile_targets(Smem& sm, const TileJob& job, long tile, const Acc* __restrict__ prod) {
  const int u = threadIdx.x;
  const int k0 = int(job.col0) + 16, nk = job.bufend - k0;
  float* Ls = reinterpret_cast<float*>(sm.M);
  float* Ws = Ls + 112 * 16;
  float* Hs = Ws + 112 * 16;
  const long row0 = tile * 16;
  for (int idx = u; idx < nk * 16; idx += kThreads) {
    const long k = k0 + (idx >> 4);
    const int e = idx & 15;
    Ls[idx] = job.L[k * job.ldl + job.col0 + e];
    Ws[idx] = job.WT[k * job.ldw + row0 + e];
    Hs[idx] = job.hatWT[k * job.ldw + row0 + e];
  }
  __syncthreads();
  const int q = perm_fwd(u), r = q >> 4, c = q & 15;
  const long col = job.col0 + c;
  Acc acc = Acc(job.WT[col * job.ldw + row0 + r]) + prod[(col - job.prod_row0) * job.ldw + row0 + r];
  for (int kk = 0; kk < nk; ++kk) acc += Acc(Ls[kk * 16 + c]) * (Acc(Ws[kk * 16 + r]) - Acc(Hs[kk * 16 + r]));
  sm.x[u] = float(_Float16(float(acc)));
}

__global__ __launch_bounds__(kThreads, 3) void viterbi_tiles_kernel(TileJob job, const double* __restrict__ entry_d,
                                                                 const float* __restrict__ entry_f,
                                                                 unsigned long long* __restrict__ bp_all) {
  __shared__ Smem sm;
  const int u = threadIdx.x;
  unsigned long long* bp = bp_all + size_t(blockIdx.x) * kBpWordsPerTile;
  for (long tile = blockIdx.x; tile < job.tiles; tile += gridDim.x) {
    if (job.X) sm.x[u] = job.X[tile * kSeq + u];
    else if (job.prod64) tile_targets<double>(sm, job, tile, job.prod64);
    else tile_targets<float>(sm, job, tile, job.prod32);
    __syncthreads();
    // pass 1 on the sequence rotated by half its length, free ends; only steps 64..126 are traced back
    forward_pass(sm, entry_d, 128, -1, bp, 64);
    if (u == 0) {
      uint32_t s = sm.final_state;  // state of step 127
      for (int i = 127; i > 64; --i) {
        const uint32_t j = s >> 4;
        s = j | (bp_lookup(bp + size_t(i - 1) * kThreads, j) << 12);
      }
      sm.overlap = int(s >> 4);  // state of step 64, high 12 bits
    }
    __syncthreads();
    const int ov = sm.overlap;
    // pass 2 on the sequence itself, tail-biting through group ov
    forward_pass(sm, entry_d, 0, ov, bp, 0);
    if (u == 0) {
      uint32_t s = sm.final_state;
      sm.st[127] = uint16_t(s);
      for (int i = 127; i > 0; --i) {
        const uint32_t j = s >> 4;
        s = j | (bp_lookup(bp + size_t(i - 1) * kThreads, j) << 12);
        sm.st[i - 1] = uint16_t(s);
      }
    }
    __syncthreads();
    // ---- outputs
    if (job.states && u < kSteps) job.states[(tile * job.q_tile_stride + job.q_offset) * kSteps + u] = sm.st[u];
    if (job.packed && u < kWords) {
      uint32_t v;
      if (u == 0) v = sm.st[0];
      else {
        v = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) v = (v << 4) | (sm.st[4 * u + k - 3] & 15u);
      }
      job.packed[tile * kWords + u] = uint16_t(v);
    }
    if (job.hatWT) {
      const uint32_t s = sm.st[u >> 1];
      const uint32_t e = ((s * (s + 1u)) >> 6) & 1023u;
      const int q = perm_fwd(u), r = q >> 4, c = q & 15;
      job.hatWT[(job.col0 + c) * job.ldw + tile * 16 + r] = entry_f[2 * e + (u & 1)];
    }
    __syncthreads();
  }
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

size_t viterbi_workspace_bytes(int slots) { return size_t(slots) * kBpWordsPerTile * sizeof(unsigned long long); }

int viterbi_max_slots(int device) {
  hipDeviceProp_t prop;
  QTIP_HIP(hipGetDeviceProperties(&prop, device));
  int per_cu = 0;
  QTIP_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, viterbi_tiles_kernel, kThreads, 0));
  if (per_cu < 1) per_cu = 1;
  return per_cu * prop.multiProcessorCount;
}

void launch_viterbi_tiles(const TileJob& job, const double* d_entry_d, const float* d_entry_f, void* workspace,
                          int slots, hipStream_t s, hipEvent_t start, hipEvent_t stop) {
  if (job.tiles <= 0) return;
  QTIP_REQUIRE(slots > 0 && workspace != nullptr, "viterbi: missing workspace");
  if (!job.X) {  // LDLQ block: the targets come from the feedback operands
    QTIP_REQUIRE(job.WT && job.L && job.hatWT && ((job.prod64 != nullptr) != (job.prod32 != nullptr)),
                 "viterbi: neither inputs nor complete LDLQ feedback operands");
    const long nk = job.bufend - job.col0 - 16;
    QTIP_REQUIRE(job.col0 >= 0 && nk >= 0 && nk <= 112, "viterbi: column block outside its 128-column buffer");
    QTIP_REQUIRE(job.col0 >= job.prod_row0 && job.ldw >= 16 * job.tiles && job.ldl >= job.bufend,
                 "viterbi: LDLQ operand geometry");
  }
  const unsigned grid = unsigned(job.tiles < slots ? job.tiles : slots);
  if (start || stop) {
    // the runtime stamps the two events at the kernel's own start and end: the time between them is the kernel's,
    // however late the host got round to queueing it
    hipExtLaunchKernelGGL(viterbi_tiles_kernel, dim3(grid), dim3(kThreads), 0, s, start, stop, 0, job, d_entry_d,
                          d_entry_f, static_cast<unsigned long long*>(workspace));
  } else {
    viterbi_tiles_kernel<<<dim3(grid), dim3(kThreads), 0, s>>>(job, d_entry_d, d_entry_f,
                                                               static_cast<unsigned long long*>(workspace));
  }
  QTIP_HIP(hipGetLastError());
}

void launch_decode_states(const uint16_t* states, long B, float* hat, const float* d_entry_f, hipStream_t s) {
  const long count = B * kSteps;
  if (count <= 0) return;
  decode_states_kernel<<<dim3(unsigned((count + 255) / 256)), dim3(256), 0, s>>>(states, count, hat, d_entry_f);
  QTIP_HIP(hipGetLastError());
}

}  // namespace qtipmi
