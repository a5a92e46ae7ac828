// Small data-movement kernels of the group path: source-weight decoding (bf16, FP8 E4M3 with a per-row bf16
// scale; reference src/kernels.hip:31-60), row/column scaling (src/kernels.hip:67-75) and the packer that turns
// the per-tile state paths into the kernel-layout trellis words (pack_trellis + swizzle_for_kernel,
// src/qtip_core.cpp:194-243, done on the device so only 64 bytes per tile cross PCIe).
#include "misc.hpp"
#include "qtip_internal.hpp"

namespace qtipmi {
namespace {

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) { return __uint_as_float(uint32_t(h) << 16); }
// OCP FP8 E4M3 "fn": bias 7, no infinities, 0x7f / 0xff are NaN
__device__ __forceinline__ float fp8e4m3_to_f32(uint8_t b) {
  const uint32_t s = b >> 7, e = (b >> 3) & 0xfu, m = b & 7u;
  float v;
  if (e == 0) v = ldexpf(float(m), -9);
  else if (e == 15 && m == 7) v = __builtin_nanf("");
  else v = ldexpf(float(m | 8u), int(e) - 10);
  return s ? -v : v;
}

__global__ void bf16_to_f32_kernel(const uint16_t* __restrict__ in, float* __restrict__ out, long count) {
  const long i = long(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < count) out[i] = bf16_bits_to_f32(in[i]);
}
__global__ void fp8_to_f32_kernel(const uint8_t* __restrict__ w, const uint16_t* __restrict__ sc,
                                  float* __restrict__ out, long rows, long cols) {
  const long i = long(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= rows * cols) return;
  const float v = fp8e4m3_to_f32(w[i]);
  out[i] = sc ? v * bf16_bits_to_f32(sc[i / cols]) : v;
}
__global__ void scale_rc_kernel(float* __restrict__ X, long rows, long cols, long ld, const float* __restrict__ rs,
                                const float* __restrict__ cs) {
  const long i = long(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= rows * cols) return;
  const long r = i / cols, c = i % cols;
  float v = X[r * ld + c];
  if (rs) v *= rs[r];
  if (cs) v *= cs[c];
  X[r * ld + c] = v;
}

// One thread per output word.  Q holds the state paths of a linear's tiles, tile (tr, tc) at Q[(tr*nblk+tc)*128].
// Word c of a tile: c == 0 -> state 0; else the low nibbles of states 4c-3 .. 4c.
__global__ void pack_swizzle_kernel(const uint16_t* __restrict__ Q, long tile_rows, long nblk,
                                    uint16_t* __restrict__ out) {
  const long idx = long(blockIdx.x) * blockDim.x + threadIdx.x;
  const long total = tile_rows * nblk * 32;
  if (idx >= total) return;
  // idx = (((i0*N2 + j0)*32 + c)*2 + j1)*2 + i1
  const int i1 = int(idx & 1), j1 = int((idx >> 1) & 1), c = int((idx >> 2) & 31);
  const long blk = idx >> 7, N2 = nblk / 2, i0 = blk / N2, j0 = blk % N2;
  const uint16_t* st = Q + ((2 * i0 + i1) * nblk + 2 * j0 + j1) * 128;
  uint32_t v;
  if (c == 0) v = st[0];
  else {
    v = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) v = (v << 4) | (st[4 * c + k - 3] & 15u);
  }
  out[idx] = uint16_t(v);
}

inline unsigned blocks_for(long count) { return unsigned((count + 255) / 256); }

}  // namespace

void launch_bf16_to_f32(const uint16_t* in, float* out, long count, hipStream_t s) {
  if (count <= 0) return;
  bf16_to_f32_kernel<<<blocks_for(count), 256, 0, s>>>(in, out, count);
  QTIP_HIP(hipGetLastError());
}
void launch_fp8_to_f32(const uint8_t* w, const uint16_t* scale_bf16, float* out, long rows, long cols, hipStream_t s) {
  if (rows * cols <= 0) return;
  fp8_to_f32_kernel<<<blocks_for(rows * cols), 256, 0, s>>>(w, scale_bf16, out, rows, cols);
  QTIP_HIP(hipGetLastError());
}
void launch_scale_rc(float* X, long rows, long cols, long ld, const float* rs, const float* cs, hipStream_t s) {
  if (rows * cols <= 0) return;
  scale_rc_kernel<<<blocks_for(rows * cols), 256, 0, s>>>(X, rows, cols, ld, rs, cs);
  QTIP_HIP(hipGetLastError());
}
void launch_pack_swizzle(const uint16_t* Q, long m, long n, uint16_t* out, hipStream_t s) {
  QTIP_REQUIRE(m % 32 == 0 && n % 32 == 0, "kernel layout needs m, n multiples of 32 (m=%ld n=%ld)", m, n);
  const long total = (m / 16) * (n / 16) * 32;
  if (total <= 0) return;
  pack_swizzle_kernel<<<blocks_for(total), 256, 0, s>>>(Q, m / 16, n / 16, out);
  QTIP_HIP(hipGetLastError());
}

}  // namespace qtipmi
