// Internal declarations shared by the host side and the HIP translation units of libqtip_mi355.so.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/qtip_mi355.h"

namespace qtipmi {

constexpr int kSeq = 256;      // weights per trellis (one 16x16 tile)
constexpr int kSteps = 128;    // trellis steps, 2 weights each
constexpr int kStates = 65536; // L = 16
constexpr int kGroups = 4096;  // states sharing a successor group
constexpr int kWords = 32;     // packed u16 words per trellis
constexpr int kLutEntries = 1024;  // distinct codebook entries: bits 6..15 of s*(s+1)
// A decision of a 32-bit Viterbi pass stands when it is won by this many units of 2^-26: a metric of at most 128
// rounded terms is within 64 units of the fp64 one, so two candidates 129 units apart are ordered alike in fp64.
// (The bound of the last step; a step whose candidates have fewer terms is held to as many units less.)
constexpr uint32_t kViterbiMargin = 160;

struct Error : std::runtime_error {
  int code;
  Error(int c, const std::string& m) : std::runtime_error(m), code(c) {}
};
[[noreturn]] void fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
void set_last_error(const std::string& m);

#define QTIP_HIP(expr)                                                                              \
  do {                                                                                              \
    hipError_t e_ = (expr);                                                                         \
    if (e_ != hipSuccess)                                                                           \
      ::qtipmi::fail(QTIP_E_HIP, "%s:%d: %s -> %s", __FILE__, __LINE__, #expr, hipGetErrorString(e_)); \
  } while (0)
#define QTIP_REQUIRE(cond, ...)                              \
  do {                                                       \
    if (!(cond)) ::qtipmi::fail(QTIP_E_ARG, __VA_ARGS__);    \
  } while (0)

// hipMalloc; a host-only test can make the next calls fail (test_fail_next_device_allocs) without touching a GPU
hipError_t device_malloc(void** p, size_t bytes);
void test_fail_next_device_allocs(int count);
long test_device_alloc_calls();

// Device memory kept by a context instead of going back to the runtime.  hipFree waits for the whole device, every
// stream of every thread, and the per-group buffers of the quantizer are a dozen such waits per group: harmless
// while one group at a time uses the chip, but groups that run side by side on lanes would wait for each other at
// every one of them.  A thread that has made an arena current (ArenaScope) gets its DBuf allocations from the
// arena's idle blocks (smallest one that is large enough and at most twice the size; else a new hipMalloc) and hands
// them back on release, after waiting for the arena's own streams only - the streams the lane's kernels run on.
// The blocks are freed with the arena.
struct DeviceArena {
  DeviceArena();
  DeviceArena(const DeviceArena&) = delete;
  DeviceArena& operator=(const DeviceArena&) = delete;
  ~DeviceArena();
  hipError_t acquire(void** p, size_t bytes);
  void give_back(void* p);
  size_t idle_bytes() const;
  size_t trim();  // idle blocks back to the runtime; returns their bytes.  An idle block is one whose last user has waited for the arena's streams, so any thread may do this
  // a lane's arena names its context's arena as parent (set while no lane thread runs): an allocation that finds the
  // device out of memory trims the whole family before it gives up
  DeviceArena* parent = nullptr;
  std::vector<DeviceArena*> children;
  std::vector<hipStream_t*> streams;  // slots holding the streams whose work may use the blocks (null slots are skipped)
  struct Impl;
  Impl* impl;
};
DeviceArena* current_arena();
struct ArenaScope {  // makes `a` the calling thread's arena until the scope ends
  DeviceArena* prev;
  explicit ArenaScope(DeviceArena* a);
  ~ArenaScope();
  ArenaScope(const ArenaScope&) = delete;
  ArenaScope& operator=(const ArenaScope&) = delete;
};

// Device buffer released on scope exit.
template <class T>
struct DBuf {
  T* p = nullptr;
  size_t n = 0;
  DeviceArena* from = nullptr;  // the arena the block came from (null: hipMalloc)
  DBuf() = default;
  explicit DBuf(size_t count) { alloc(count); }
  DBuf(const DBuf&) = delete;
  DBuf& operator=(const DBuf&) = delete;
  ~DBuf() { release(); }
  void alloc(size_t count) {
    release();
    if (count) {
      DeviceArena* a = current_arena();
      QTIP_HIP(a ? a->acquire(reinterpret_cast<void**>(&p), count * sizeof(T))
                 : device_malloc(reinterpret_cast<void**>(&p), count * sizeof(T)));
      from = a;
    }
    n = count;  // only after the allocation succeeded: a failed one leaves an empty buffer that ensure() retries
  }
  void ensure(size_t count) {
    if (count > n) alloc(count);
  }
  void release() {
    if (p) {
      if (from) from->give_back(p);
      else (void)hipFree(p);
    }
    p = nullptr;
    n = 0;
    from = nullptr;
  }
  size_t bytes() const { return n * sizeof(T); }
  operator T*() const { return p; }
};

// Page-locked host buffer (staging for HRr / L), released on scope exit.
template <class T>
struct HBuf {
  T* p = nullptr;
  size_t n = 0;
  HBuf() = default;
  HBuf(const HBuf&) = delete;
  HBuf& operator=(const HBuf&) = delete;
  ~HBuf() { release(); }
  void alloc(size_t count) {
    release();
    if (count) QTIP_HIP(hipHostMalloc(reinterpret_cast<void**>(&p), count * sizeof(T), hipHostMallocDefault));
    n = count;
  }
  void release() {
    if (p) (void)hipHostFree(p);
    p = nullptr;
    n = 0;
  }
};

// ---- host-side number formats / streams (qtip_host.cpp)
uint16_t f32_to_fp16(float f);
float fp16_to_f32(uint16_t h);
uint16_t f32_to_bf16(float f);
float bf16_to_f32(uint16_t h);
struct SplitMix {
  uint64_t s;
  explicit SplitMix(uint64_t seed);
  uint64_t next();
  float sign();
};
int had_K(int n);
// K x K mixing matrix as +-1 int8: row k2 holds hadK[k2][k] (transpose=false) or hadK[k][k2] (transpose=true)
std::vector<int8_t> had_matrix(int K, bool transpose);

struct HostCodebook {
  float tlut[512][2];
  uint16_t tlut_h[512][2];
  // per distinct entry e = flip << 9 | idx: the two decoded components
  double entry_d[kLutEntries][2];
  float entry_f[kLutEntries][2];
  double lut_rms = 0;
  void build(const float* tlut_or_null);
  static inline uint32_t entry_of_state(uint32_t s) { return ((s * (s + 1)) >> 6) & 1023u; }
};

void pack_trellis_host(const uint16_t* states, long B, uint16_t* packed);
void unpack_trellis_host(const uint16_t* packed, long B, uint16_t* states);
bool swizzle_host(const uint16_t* packed, int m, int n, uint16_t* out);
bool unswizzle_host(const uint16_t* in, int m, int n, uint16_t* packed);

// Large host work buffer from a process-wide pool (2 MB aligned, huge-page advised, kept for the life of the
// process and handed out to one caller at a time): the fp64 LDL work matrix (6.6 GB at n = 28672) and its packed
// panels are not mapped and faulted in again for every group.  Contents are whatever the last user left.
struct HostScratch {
  void* p;
  explicit HostScratch(size_t bytes);
  ~HostScratch();
  HostScratch(const HostScratch&) = delete;
  HostScratch& operator=(const HostScratch&) = delete;
  void* get() const { return p; }
};

// fp64 block LDL on the host (host_ldl.cpp). A: n x n fp64, lower triangle used, destroyed. Returns false if not PD.
bool block_ldl_host(double* A, int n, float* L_out, int threads);
// The same factorization with the trailing matrix kept by someone else (the GPU): the host factors and solves one
// panel of ldl_panel_width() columns at a time.  fetch(k, kb) returns a buffer of row stride kb holding rows k .. n-1
// of the columns k .. k+kb-1 as updated so far; solved(k, kb, panel) receives it back with the final columns of the
// Cholesky factor: the rows kb .. n-k-1 of it are the operand of the rank-kb update of the trailing matrix, which
// must form every element as one chain acc = fma(x_ip, x_jp, acc), p = 0 .. kb-1 from zero, then c -= acc, for L to
// equal block_ldl_host's bit for bit.
struct PanelAssist {
  virtual double* fetch(int k, int kb) = 0;
  virtual void solved(int k, int kb, const double* panel) = 0;
  // optional: the kb x kb diagonal block of panel k is factored (lower triangle at diag, row stride ld); called before
  // the rows below it are solved
  virtual void factored(int k, int kb, const double* diag, long ld) {}
  // optional: rows row0 .. row0 + count - 1 of the matrix (below the panel) are solved, `rows` holds their kb values
  // (row stride ld).  Called from the team's threads, several at a time, while the rows are still in cache.
  virtual void rows_solved(int k, int kb, int row0, int count, const double* rows, long ld) {}
  // the columns k .. k+kb-1 of L_out are final (all n rows)
  virtual void assembled(int k, int kb) {}
  virtual ~PanelAssist() = default;
};
int ldl_panel_width();
bool block_ldl_assisted(int n, float* L_out, int threads, PanelAssist& assist);
bool block_ldl_assisted_on_host(const float* HRr, int n, float* L_out, int threads);
// the scalar LDL of the NVFP4 calibration through the same panels: L_ij = C_ij / C_jj, dw_j = C_jj^2
bool scalar_ldl_assisted(int n, float* L_out, float* dw, int threads, PanelAssist& assist);
// lower Cholesky in place (lower triangle of the n x n fp64 matrix A); false if not positive definite
bool cholesky_lower_host(double* A, int n, int threads);
// A[i][j] = (HRr[i][j] + HRr[j][i]) / 2 in fp64, lower triangle
void symmetrize_lower_host(const float* HRr, int n, double* A, int threads);

// ---- layer-file writer (layer_file.cpp); the struct behind the C handle is defined there
qtip_st_writer* st_new();
void st_delete(qtip_st_writer* w);
void st_add(qtip_st_writer* w, const char* name, const char* dtype, const int64_t* shape, int rank, const void* data,
            size_t bytes);
void st_add_qtip_linear(qtip_st_writer* w, const char* prefix, const qtip_linear_out* out, int m, int n,
                        const uint16_t* tlut_f16);
size_t st_write(const qtip_st_writer* w, const char* path, const char* const* meta_kv, int nmeta);

// ---- GPU launchers (viterbi.hip, rht.hip, ldlq.hip)
struct TileJob {
  // inputs: either X (tiles x 256 fp32, sequence order) or the LDLQ feedback operands below
  const float* X = nullptr;
  long tiles = 0;
  // LDLQ feedback (X null): tile t covers weight rows 16 t .. 16 t + 15 and the columns col0 .. col0 + 15; the
  // target of (row j, column col0 + c) is
  //   WT[(col0 + c) * ldw + j] + prod[(col0 + c - prod_row0) * ldp + j]
  //     + sum over k = col0 + 16 .. bufend - 1 (ascending) of L[k * ldl + col0 + c] * (WT - hatWT)[k * ldw + j],
  // accumulated in the type of prod (prod64 or prod32, whichever is set) and rounded to fp32, then to fp16.
  const float* WT = nullptr;
  const float* L = nullptr;
  long ldl = 0;
  int bufend = 0;
  const double* prod64 = nullptr;
  const float* prod32 = nullptr;
  long prod_row0 = 0;
  long ldp = 0;  // row stride of prod (0: ldw)
  // prod as the split-K partial slabs of the gathered product: prod[s * prod_split_stride + ...], s < prod_splits,
  // added in this order (what the product's own reduction kernel would have done)
  int prod_splits = 1;
  long prod_split_stride = 0;
  // outputs (any may be null)
  uint16_t* states = nullptr;  // state words of tile t at states[(t * q_tile_stride + q_offset) * 128]
  long q_tile_stride = 1, q_offset = 0;
  uint16_t* packed = nullptr;  // tiles x 32, pack_trellis layout
  float* hatWT = nullptr;      // scatter of decoded values: hatWT[(col0 + c) * ldw + 16 * t + r]
  long ldw = 0, col0 = 0;
  // with hatWT and WT: the residual WT - hatWT of the decoded values as bf16 hi / lo bit patterns, weight row major:
  // dimg[(16 t + r) * ldd + col0 + c] (the operand images of the split-bf16 gathered product)
  uint16_t *dimg_h = nullptr, *dimg_l = nullptr;
  long ldd = 0;
  // LDLQ: a workgroup takes its tile row through `blocks` consecutive 16-column blocks, from the last (columns
  // col0 + 16 (blocks - 1) ..) down to the first (col0 ..), state words at q_offset + block: the blocks of a tile row
  // depend on each other only through that row's own hatWT values, so nothing has to wait for another workgroup
  int blocks = 1;
  // 0: both passes run on 32-bit metrics first and a pass whose traced decisions are not all won by `margin` units of
  // 2^-26 is run again on fp64 metrics (same results as mode 1, bit for bit); 1: fp64 metrics only
  int mode = 0;
  // workgroups of 512 threads per tile instead of 256 (mode 0 only; same results): -1 = where the launch has at most
  // a third as many tiles as the device has workgroup slots, 0 = never, 1 = always
  int wide = -1;
  uint32_t margin = kViterbiMargin;
  unsigned* stats = nullptr;  // device counters (optional): [0], [1] += passes of the first / second kind run again
};
size_t viterbi_workspace_bytes(int slots);
int viterbi_max_slots(int device);
// start / stop (optional): events stamped at the kernel's own start and end
void launch_viterbi_tiles(const TileJob& job, const double* d_entry_d, const float* d_entry_f, void* workspace,
                          int slots, hipStream_t s, hipEvent_t start = nullptr, hipEvent_t stop = nullptr);
// Kept-metrics slots that are part of the code object (no allocation): viterbi_static_scratch_init looks up the
// array's address on `device`, which must be current, once; viterbi_static_scratch returns it (null before that).
int viterbi_static_slots();
void viterbi_static_scratch_init(int device);
void* viterbi_static_scratch(int device);
void launch_decode_states(const uint16_t* states, long B, float* hat, const float* d_entry_f, hipStream_t s);
// keeps the stream busy for about `microseconds` (one wave watching the clock, with a bound on its turns)
void launch_delay(double microseconds, hipStream_t s);

}  // namespace qtipmi

