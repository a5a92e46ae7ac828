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

#include "data/viterbi_layout.h"

constexpr int kThreads = 256;
constexpr int kRowStride = QTIP_VIT_ROW_STRIDE;  // doubles per E row: 2 x 16 entries + padding
constexpr int kESlots = 64 * kRowStride + (kRowStride - 32);
constexpr int kMSlots = 256 * 17;                // metric of (column c, digit d) at c*17 + d
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
  const int tid = threadIdx.x;
  const int u = kOctetOfLane[tid];  // which octet of groups this lane owns (placement tuned against LDS bank conflicts)
  const double INF = __builtin_inf();

  // this thread's 4 codebook entries for the per-step error table: e = tid + 256*q -> row tid & 63, k = (tid >> 6) + 4q
  // (re-read from the 16 KB global table every step: it stays in the CU's vector L1 and the registers are needed)
  const double2* __restrict__ entries = reinterpret_cast<const double2*>(entry_d) + tid;
  const int e_wr = (tid & 63) * kRowStride + kRowPad[tid & 63] + (tid >> 6);

  // per-pair E row base (in doubles): row * stride + b4
  int ebase[8];
#pragma unroll
  for (int m = 0; m < 8; ++m) {
    const uint32_t j = 8u * u + m, p = j * (j + 1u);
    const int row = int((p >> 6) & 63u);
    ebase[m] = row * kRowStride + kRowPad[row] + int((p >> 12) & 15u);
  }
  const int colA = u >> 1, colB = 255 - colA;
  const int rA = colA * 17, rB = colB * 17;
  const int wA = 136 * (u & 31) + (u >> 5);                    // slot of group 8u + m: wA + 17 m
  const int wB = (255 - 8 * (u & 31)) * 17 + 15 - (u >> 5);    // slot of group 4095 - 8u - m: wB - 17 m

  // initial metrics: M_0[g] = 0, or +inf outside group ov
  for (int g = tid; g < kGroups; g += kThreads) {
    const int col = g & 255, d = g >> 8;
    sm.M[col * 17 + d] = (ov < 0 || g == ov) ? 0.0 : INF;
  }
  __syncthreads();

  unsigned long long word = 0;
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
        const double2 l = entries[256 * q];
        const double a = l.x - x0, b = l.y - x1;
        const double err = __builtin_fma(a, a, b * b);
        sm.E[e_wr + 4 * q] = err;
        sm.E[e_wr + 4 * q + 16] = err;
      }
    }
    __syncthreads();
    // ---- phase C: 16 groups x 16 candidates
    word = 0;
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
        da = ca < ba ? uint32_t(d) : da;  // strict: the first minimum in ascending d wins ties
        db = cb < bb ? uint32_t(d) : db;
        ba = __builtin_fmin(ba, ca);
        bb = __builtin_fmin(bb, cb);
      }
      sm.M[wA + 17 * m] = ba;
      sm.M[wB - 17 * m] = bb;
      word |= (unsigned long long)(da) << (4 * m);
      word |= (unsigned long long)(db) << (32 + 4 * m);
      __builtin_amdgcn_sched_barrier(0);  // keep one row of the error table in flight at a time (register budget)
    }
    if (it >= bp_first && it < kSteps - 1)
      __hip_atomic_store(bp + size_t(it) * kThreads + u, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
  }
  // final state: smallest metric, then smallest state, over the metrics of the last step (each lane re-reads the
  // 16 values it has just written; their predecessor digits are the nibbles of the last back-pointer word)
  if (ov < 0) {
    double bestc = INF;
    uint32_t bests = 0xffffffffu;
#pragma unroll
    for (int m = 0; m < 8; ++m) {
      const uint32_t ja = 8u * u + m, jb = 4095u - ja;
      const uint32_t sa = (uint32_t(word >> (4 * m)) & 15u) << 12 | ja;
      const uint32_t sb = (uint32_t(word >> (32 + 4 * m)) & 15u) << 12 | jb;
      const double ca = sm.M[wA + 17 * m], cb = sm.M[wB - 17 * m];
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
    if (jj >> 3 == uint32_t(u)) {
      const uint32_t shift = (jj & 7u) * 4u + (j < 2048u ? 0u : 32u);
      sm.final_state = (uint32_t(word >> shift) & 15u) << 12 | j;
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
