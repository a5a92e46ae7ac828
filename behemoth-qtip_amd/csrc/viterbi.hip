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
// in opposite order.  Thread u therefore owns the 8 groups 8u..8u+7 (all in metric column u>>1) and their
// mirrors 4095-8u-m (column 255-(u>>1)): per step it keeps the two metric columns (2 x 16 fp64) in registers
// and streams 8 rows of E (16 fp64 each) from LDS, i.e. 160 LDS reads for 256 add-compare-selects.
//
// LDS per workgroup (~51 KB, three workgroups per CU): E rows stored twice back to back so that the rotation
// by b4 is a per-lane base address and the stride d*(2m+1) a compile-time offset; metrics single-buffered
// (columns are read into registers before the step's results are written), padded by one slot per 8 columns.
// Back-pointers (4 bits per group and step) go to HBM as one 64-bit word per thread and step, 2 KB per step,
// fully coalesced; the first pass only keeps the steps its half-length trace-back needs.
#include "qtip_internal.hpp"

namespace qtipmi {
namespace {

constexpr int kThreads = 256;
constexpr int kRowStride = 33;                   // doubles per E row: 2 x 16 entries + 1 pad
constexpr int kESlots = 64 * kRowStride;         // 2112
constexpr int kMSlots = 256 * 16 + 32;           // 4128: column c at c*16 + (c >> 3)
constexpr int kBpWordsPerTile = 127 * kThreads;  // u64 words

struct Smem {
  double M[kMSlots];
  double E[kESlots];
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

// word index and nibble of group j inside one step's 256 back-pointer words
__device__ __forceinline__ uint32_t bp_lookup(const unsigned long long* step_words, uint32_t j) {
  const uint32_t jj = j < 2048u ? j : 4095u - j;
  const uint32_t shift = (jj & 7u) * 4u + (j < 2048u ? 0u : 32u);
  const unsigned long long w = __hip_atomic_load(step_words + (jj >> 3), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return uint32_t(w >> shift) & 15u;
}

// One forward pass over the 128 steps.  roll: input rotation (128 for the first pass).  ov < 0: free start and
// end; otherwise start in states with (s >> 4) == ov and end in the state of group ov.
// bp: this workgroup's back-pointer words; steps < bp_first are not stored.  Returns nothing; the final state
// is left in sm.final_state.
__device__ __forceinline__ void forward_pass(Smem& sm, const double* __restrict__ entry_d, int roll, int ov,
                                             unsigned long long* __restrict__ bp, int bp_first) {
  const int u = threadIdx.x;
  const double INF = __builtin_inf();

  // this thread's 4 codebook entries for the per-step error table: e = u + 256*q -> row u & 63, k = (u >> 6) + 4q
  double l0[4], l1[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    l0[q] = entry_d[2 * (u + 256 * q)];
    l1[q] = entry_d[2 * (u + 256 * q) + 1];
  }
  const int e_wr = (u & 63) * kRowStride + (u >> 6);

  // per-pair E row base (in doubles): row * stride + b4
  int ebase[8];
#pragma unroll
  for (int m = 0; m < 8; ++m) {
    const uint32_t j = 8u * u + m, p = j * (j + 1u);
    ebase[m] = int((p >> 6) & 63u) * kRowStride + int((p >> 12) & 15u);
  }
  const int colA = u >> 1, colB = 255 - colA;
  const int rA = colA * 16 + (colA >> 3), rB = colB * 16 + (colB >> 3);
  const int wA = 128 * (u & 31) + (u >> 5) + (u & 31);
  const int wB = (255 - 8 * (u & 31)) * 16 + 15 - (u >> 5) + 31 - (u & 31);

  // initial metrics: M_0[g] = 0, or +inf outside group ov
  for (int g = u; g < kGroups; g += kThreads) {
    const int col = g & 255, d = g >> 8;
    sm.M[col * 16 + d + (col >> 3)] = (ov < 0 || g == ov) ? 0.0 : INF;
  }
  __syncthreads();

  double bestc = INF;
  uint32_t bests = 0xffffffffu;
  for (int it = 0; it < kSteps; ++it) {
    // ---- phase R: metric columns -> registers, error table of this step -> LDS
    double MA[16], MB[16];
#pragma unroll
    for (int d = 0; d < 16; ++d) {
      MA[d] = sm.M[rA + d];
      MB[d] = sm.M[rB + d];
    }
    {
      const int t = (2 * it + roll) & 255;
      const double x0 = double(sm.x[t]), x1 = double(sm.x[t + 1]);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const double a = l0[q] - x0, b = l1[q] - x1;
        const double err = __builtin_fma(a, a, b * b);
        sm.E[e_wr + 4 * q] = err;
        sm.E[e_wr + 4 * q + 16] = err;
      }
    }
    __syncthreads();
    // ---- phase C: 16 groups x 16 candidates
    unsigned long long word = 0;
    const bool last = it == kSteps - 1;
#pragma unroll
    for (int m = 0; m < 8; ++m) {
      const int g = 2 * m + 1;
      const double* er = sm.E + ebase[m];
      double e[16];
#pragma unroll
      for (int d = 0; d < 16; ++d) e[d] = er[(d * g) & 15];
      double ba = e[0] + MA[0], bb = e[15] + MB[0];
      uint32_t da = 0, db = 0;
#pragma unroll
      for (int d = 1; d < 16; ++d) {
        const double ca = e[d] + MA[d];
        const double cb = e[15 - d] + MB[d];
        if (ca < ba) ba = ca, da = d;
        if (cb < bb) bb = cb, db = d;
      }
      sm.M[wA + 16 * m] = ba;
      sm.M[wB - 16 * m] = bb;
      word |= (unsigned long long)(da) << (4 * m);
      word |= (unsigned long long)(db) << (32 + 4 * m);
      if (last) {  // candidates for the final state: smallest metric, then smallest state
        const uint32_t ja = 8u * u + m, jb = 4095u - ja;
        const uint32_t sa = (da << 12) | ja, sb = (db << 12) | jb;
        if (ov < 0) {
          if (ba < bestc || (ba == bestc && sa < bests)) bestc = ba, bests = sa;
          if (bb < bestc || (bb == bestc && sb < bests)) bestc = bb, bests = sb;
        } else {
          if (int(ja) == ov) sm.final_state = sa;
          if (int(jb) == ov) sm.final_state = sb;
        }
      }
    }
    if (it >= bp_first && it < kSteps - 1)
      __hip_atomic_store(bp + size_t(it) * kThreads + u, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
  }
  if (ov < 0) {
    // lexicographic (metric, state) minimum over the workgroup
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const double oc = __shfl_xor(bestc, off, 64);
      const uint32_t os = __shfl_xor(bests, off, 64);
      if (oc < bestc || (oc == bestc && os < bests)) bestc = oc, bests = os;
    }
    if ((u & 63) == 0) sm.red_c[u >> 6] = bestc, sm.red_s[u >> 6] = bests;
    __syncthreads();
    if (u == 0) {
      double c = sm.red_c[0];
      uint32_t s = sm.red_s[0];
      for (int w = 1; w < 4; ++w)
        if (sm.red_c[w] < c || (sm.red_c[w] == c && sm.red_s[w] < s)) c = sm.red_c[w], s = sm.red_s[w];
      sm.final_state = s;
    }
  }
  __syncthreads();
}

__global__ __launch_bounds__(kThreads, 3) void viterbi_tiles_kernel(TileJob job, const double* __restrict__ entry_d,
                                                                 const float* __restrict__ entry_f,
                                                                 unsigned long long* __restrict__ bp_all) {
  __shared__ Smem sm;
  const int u = threadIdx.x;
  unsigned long long* bp = bp_all + size_t(blockIdx.x) * kBpWordsPerTile;
  for (long tile = blockIdx.x; tile < job.tiles; tile += gridDim.x) {
    sm.x[u] = job.X[tile * kSeq + u];
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
                          int slots, hipStream_t s) {
  if (job.tiles <= 0) return;
  QTIP_REQUIRE(job.X != nullptr && slots > 0 && workspace != nullptr, "viterbi: missing operand");
  const unsigned grid = unsigned(job.tiles < slots ? job.tiles : slots);
  viterbi_tiles_kernel<<<dim3(grid), dim3(kThreads), 0, s>>>(job, d_entry_d, d_entry_f,
                                                             static_cast<unsigned long long*>(workspace));
  QTIP_HIP(hipGetLastError());
}

void launch_decode_states(const uint16_t* states, long B, float* hat, const float* d_entry_f, hipStream_t s) {
  const long count = B * kSteps;
  if (count <= 0) return;
  decode_states_kernel<<<dim3(unsigned((count + 255) / 256)), dim3(256), 0, s>>>(states, count, hat, d_entry_f);
  QTIP_HIP(hipGetLastError());
}

}  // namespace qtipmi
