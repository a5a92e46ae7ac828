// Host-side pieces of the group quantizer: number formats, sign streams, codebook expansion, Hadamard factor
// selection, trellis packing.  Semantics follow the reference files named at each function.
#include <sys/mman.h>

#include <atomic>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <vector>

#include "data/qtip_tables.h"
#include "qtip_internal.hpp"

namespace qtipmi {

static thread_local std::string g_last_error;
void set_last_error(const std::string& m) { g_last_error = m; }
const std::string& last_error_ref() { return g_last_error; }
void fail(int code, const char* fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  std::vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  throw Error(code, buf);
}

// hipMalloc behind one door, so that a host-only test can see an allocation fail and be retried without a GPU
static std::atomic<int> g_fail_allocs{0};
static std::atomic<long> g_alloc_calls{0};
hipError_t device_malloc(void** p, size_t bytes) {
  g_alloc_calls.fetch_add(1);
  int left = g_fail_allocs.load();
  while (left > 0 && !g_fail_allocs.compare_exchange_weak(left, left - 1)) {}
  if (left > 0) return hipErrorOutOfMemory;
  return hipMalloc(p, bytes);
}
void test_fail_next_device_allocs(int count) { g_fail_allocs.store(count); }
long test_device_alloc_calls() { return g_alloc_calls.load(); }

struct DeviceArena::Impl {
  struct Block {
    void* p;
    size_t cap;
    bool busy;
  };
  std::mutex mu;
  std::vector<Block> blocks;
};
DeviceArena::DeviceArena() : impl(new Impl()) {}
DeviceArena::~DeviceArena() {
  for (auto& b : impl->blocks) (void)hipFree(b.p);
  delete impl;
}
hipError_t DeviceArena::acquire(void** p, size_t bytes) {
  {
    std::lock_guard<std::mutex> lk(impl->mu);
    Impl::Block* fit = nullptr;
    for (auto& b : impl->blocks)
      if (!b.busy && b.cap >= bytes && b.cap / 2 <= bytes && (!fit || b.cap < fit->cap)) fit = &b;
    if (fit) {
      fit->busy = true;
      *p = fit->p;
      return hipSuccess;
    }
  }
  // nothing idle fits: a new block.  Idle blocks go back to the runtime first when they hold more than 32 GiB (groups
  // of many different shapes would otherwise pile them up), and all of them when the device is out of memory
  const size_t cap = (bytes + 255) / 256 * 256;
  if (idle_bytes() > (size_t(32) << 30)) trim();
  hipError_t rc = device_malloc(p, cap);
  if (rc == hipErrorOutOfMemory) {
    // the idle blocks of the whole family go back first: a lane's arena may be empty while its parent's or a
    // sibling's holds the memory of an earlier, larger call
    (void)hipGetLastError();
    DeviceArena* root = this;
    while (root->parent) root = root->parent;
    root->trim();
    for (DeviceArena* a : root->children) a->trim();
    rc = device_malloc(p, cap);
  }
  if (rc != hipSuccess) return rc;
  std::lock_guard<std::mutex> lk(impl->mu);
  impl->blocks.push_back(Impl::Block{*p, cap, true});
  return hipSuccess;
}
size_t DeviceArena::idle_bytes() const {
  std::lock_guard<std::mutex> lk(impl->mu);
  size_t idle = 0;
  for (auto& b : impl->blocks)
    if (!b.busy) idle += b.cap;
  return idle;
}
size_t DeviceArena::trim() {
  std::vector<Impl::Block> gone;
  {
    std::lock_guard<std::mutex> lk(impl->mu);
    for (size_t i = impl->blocks.size(); i-- > 0;)
      if (!impl->blocks[i].busy) {
        gone.push_back(impl->blocks[i]);
        impl->blocks.erase(impl->blocks.begin() + long(i));
      }
  }
  size_t bytes = 0;
  for (auto& b : gone) {
    (void)hipFree(b.p);
    bytes += b.cap;
  }
  return bytes;
}
void DeviceArena::give_back(void* p) {
  // the next user of the block may run on another of the arena's streams: everything queued on them so far is over
  // before the block counts as idle (hipFree would have waited for the whole device)
  for (hipStream_t* s : streams)
    if (s && *s) (void)hipStreamSynchronize(*s);
  std::lock_guard<std::mutex> lk(impl->mu);
  for (auto& b : impl->blocks)
    if (b.p == p) b.busy = false;
}
static thread_local DeviceArena* g_arena = nullptr;
DeviceArena* current_arena() { return g_arena; }
ArenaScope::ArenaScope(DeviceArena* a) : prev(g_arena) { g_arena = a; }
ArenaScope::~ArenaScope() { g_arena = prev; }

// IEEE binary16 <-> binary32, round to nearest even (src/common.hpp:49-78 of the reference)
uint16_t f32_to_fp16(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  const uint32_t sign = (u >> 16) & 0x8000u, mag = u & 0x7fffffffu;
  if (mag >= 0x7f800000u) return uint16_t(sign | 0x7c00u | (mag > 0x7f800000u ? 0x200u : 0u));
  if (mag >= 0x477ff000u) return uint16_t(sign | 0x7c00u);  // rounds to infinity
  if (mag < 0x38800000u) {                                  // below the smallest normal half: fixed point in 2^-24
    const uint32_t e = mag >> 23;
    if (e < 102) return uint16_t(sign);                     // < 2^-25: rounds to zero (2^-25 itself ties to even = 0)
    const uint32_t sig = (mag & 0x7fffffu) | 0x800000u;     // 24-bit significand, value = sig * 2^(e-150)
    const int shift = int(126 - e);                         // result = sig >> shift, in units of 2^-24
    const uint32_t q = sig >> shift, rem = sig & ((1u << shift) - 1u), half = 1u << (shift - 1);
    uint32_t r = q;
    if (rem > half || (rem == half && (q & 1u))) ++r;
    return uint16_t(sign | r);
  }
  uint32_t h = (((mag >> 23) - 112u) << 10) | ((mag & 0x7fffffu) >> 13);
  const uint32_t rem = mag & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) ++h;
  return uint16_t(sign | h);
}
float fp16_to_f32(uint16_t h) {
  const uint32_t s = (h >> 15) & 1u, e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
  float v;
  if (e == 0) v = std::ldexp(float(m), -24);
  else if (e == 31) v = m ? NAN : INFINITY;
  else v = std::ldexp(float(m | 0x400u), int(e) - 25);
  return s ? -v : v;
}
uint16_t f32_to_bf16(float f) {  // src/common.hpp:42-48
  uint32_t u;
  std::memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return uint16_t((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return uint16_t(u >> 16);
}
float bf16_to_f32(uint16_t h) {
  const uint32_t u = uint32_t(h) << 16;
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

// splitmix64 stream of the reference (src/common.hpp:91-107)
SplitMix::SplitMix(uint64_t seed) : s(seed * 0x9E3779B97F4A7C15ull + 0x1234567ull) {}
uint64_t SplitMix::next() {
  uint64_t z = (s += 0x9E3779B97F4A7C15ull);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
float SplitMix::sign() { return (next() >> 63) ? -1.0f : 1.0f; }

// get_hadK (src/qtip_core.cpp:77-81): the first factor size of the fixed order that divides n decides
int had_K(int n) {
  auto pow2 = [](long v) { return v > 0 && (v & (v - 1)) == 0; };
  if (n <= 0) return 0;
  for (int i = 0; i < QTIP_NUM_HAD; ++i) {
    const int K = qtip_had_order[i];
    if (n % K == 0) return pow2(n / K) ? K : 0;
  }
  return pow2(n) ? 1 : 0;
}
std::vector<int8_t> had_matrix(int K, bool transpose) {
  const uint32_t* bits = qtip_had_bits(K);
  if (!bits) fail(QTIP_E_ARG, "no Hadamard factor of size %d", K);
  std::vector<int8_t> m(size_t(K) * K);
  for (int r = 0; r < K; ++r)
    for (int k = 0; k < K; ++k)
      m[size_t(r) * K + k] = int8_t(transpose ? qtip_had_entry(bits, K, k, r) : qtip_had_entry(bits, K, r, k));
  return m;
}

// quantlut_sym expansion (src/qtip_core.cpp:18-46): state s reads entry e(s) = bits 6..15 of s*(s+1);
// bit 9 of e is the sign fold of component 0, the low 9 bits index the fp16-rounded tlut.
void HostCodebook::build(const float* t) {
  for (int i = 0; i < 512; ++i)
    for (int v = 0; v < 2; ++v) {
      float f;
      if (t) f = t[i * 2 + v];
      else std::memcpy(&f, &qtip_hyb_tlut_bits[i * 2 + v], 4);
      tlut[i][v] = f;
      tlut_h[i][v] = f32_to_fp16(f);
    }
  for (int e = 0; e < kLutEntries; ++e) {
    const int idx = e & 511;
    uint16_t h0 = tlut_h[idx][0];
    if (e >> 9) h0 ^= 0x8000u;
    entry_f[e][0] = fp16_to_f32(h0);
    entry_f[e][1] = fp16_to_f32(tlut_h[idx][1]);
    entry_d[e][0] = entry_f[e][0];
    entry_d[e][1] = entry_f[e][1];
  }
  double ss = 0;  // same accumulation order as the reference: ascending state
  for (uint32_t s = 0; s < uint32_t(kStates); ++s) {
    const uint32_t e = entry_of_state(s);
    ss += double(entry_f[e][0]) * entry_f[e][0] + double(entry_f[e][1]) * entry_f[e][1];
  }
  lut_rms = std::sqrt(ss / (2.0 * kStates));
}

// Bit stream of one trellis, MSB first: the 16 bits of state 0, then the 4 new bits of states 1..127, cut at
// 512 bits (src/qtip_core.cpp:194-208).  Written nibble-wise: word w holds stream nibbles 4w..4w+3.
void pack_trellis_host(const uint16_t* states, long B, uint16_t* packed) {
#pragma omp parallel for schedule(static) if (B > 4096)
  for (long b = 0; b < B; ++b) {
    const uint16_t* st = states + b * kSteps;
    uint16_t* out = packed + b * kWords;
    out[0] = st[0];
    for (int w = 1; w < kWords; ++w) {
      uint32_t v = 0;
      for (int k = 0; k < 4; ++k) v = (v << 4) | (st[4 * w + k - 3] & 15u);  // stream nibble q (q >= 4) is state q-3
      out[w] = uint16_t(v);
    }
  }
}
void unpack_trellis_host(const uint16_t* packed, long B, uint16_t* states) {
#pragma omp parallel for schedule(static) if (B > 4096)
  for (long b = 0; b < B; ++b) {
    const uint16_t* in = packed + b * kWords;
    uint16_t* st = states + b * kSteps;
    auto nib = [&](int q) -> uint32_t {
      q &= 127;  // the stream wraps (tail-biting)
      return (in[q >> 2] >> (12 - 4 * (q & 3))) & 15u;
    };
    for (int t = 0; t < kSteps; ++t) st[t] = uint16_t((nib(t) << 12) | (nib(t + 1) << 8) | (nib(t + 2) << 4) | nib(t + 3));
  }
}
// Kernel layout (src/qtip_core.cpp:230-253): word c of tile (2*i0+i1, 2*j0+j1) goes to
// out[(((i0*(n/32)+j0)*32 + c)*2 + j1)*2 + i1]
bool swizzle_host(const uint16_t* packed, int m, int n, uint16_t* out) {
  if (m % 32 || n % 32) return false;
  const long nb = n / 16, M2 = m / 32, N2 = n / 32;
#pragma omp parallel for schedule(static)
  for (long i0 = 0; i0 < M2; ++i0)
    for (long j0 = 0; j0 < N2; ++j0) {
      uint16_t* o = out + (i0 * N2 + j0) * 128;
      for (int i1 = 0; i1 < 2; ++i1)
        for (int j1 = 0; j1 < 2; ++j1) {
          const uint16_t* src = packed + ((2 * i0 + i1) * nb + 2 * j0 + j1) * 32;
          for (int c = 0; c < 32; ++c) o[(c * 2 + j1) * 2 + i1] = src[c];
        }
    }
  return true;
}
bool unswizzle_host(const uint16_t* in, int m, int n, uint16_t* packed) {
  if (m % 32 || n % 32) return false;
  const long nb = n / 16, M2 = m / 32, N2 = n / 32;
#pragma omp parallel for schedule(static)
  for (long i0 = 0; i0 < M2; ++i0)
    for (long j0 = 0; j0 < N2; ++j0) {
      const uint16_t* o = in + (i0 * N2 + j0) * 128;
      for (int i1 = 0; i1 < 2; ++i1)
        for (int j1 = 0; j1 < 2; ++j1) {
          uint16_t* dst = packed + ((2 * i0 + i1) * nb + 2 * j0 + j1) * 32;
          for (int c = 0; c < 32; ++c) dst[c] = o[(c * 2 + j1) * 2 + i1];
        }
    }
  return true;
}

namespace {
// Large host work buffers, kept for the life of the process and handed out one caller at a time.
struct HostPool {
  struct Slot {
    void* p;
    size_t cap;
    bool busy;
  };
  std::mutex mu;
  std::vector<Slot> slots;
  void* acquire(size_t bytes) {
    std::lock_guard<std::mutex> lk(mu);
    Slot* fit = nullptr;  // smallest idle buffer that is large enough
    for (auto& s : slots)
      if (!s.busy && s.p && s.cap >= bytes && (!fit || s.cap < fit->cap)) fit = &s;
    if (fit) {
      fit->busy = true;
      return fit->p;
    }
    for (auto& s : slots)  // an idle but smaller buffer is replaced rather than kept beside the new one
      if (!s.busy) {
        std::free(s.p);
        s.p = nullptr;
        s.cap = 0;
      }
    void* p = nullptr;
    const size_t huge = size_t(2) << 20;
    const size_t cap = (bytes + huge - 1) / huge * huge;
    if (posix_memalign(&p, huge, cap) != 0 || !p) throw Error(QTIP_E_NOMEM, "out of host memory for the LDL work matrix");
    (void)madvise(p, cap, MADV_HUGEPAGE);
    for (auto& s : slots)
      if (!s.p) {
        s = Slot{p, cap, true};
        return p;
      }
    slots.push_back(Slot{p, cap, true});
    return p;
  }
  void release(void* p) {
    std::lock_guard<std::mutex> lk(mu);
    for (auto& s : slots)
      if (s.p == p) s.busy = false;
  }
};
HostPool& host_pool() {
  static HostPool pool;
  return pool;
}
}  // namespace
HostScratch::HostScratch(size_t bytes) : p(host_pool().acquire(bytes)) {}
HostScratch::~HostScratch() { host_pool().release(p); }

}  // namespace qtipmi
