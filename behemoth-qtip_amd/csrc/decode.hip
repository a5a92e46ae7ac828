// Decoder of the kernel-layout trellis: the 2-bit code words of a linear back to its rotated, Wscale-free weight
// hatWr (m x n fp32, row-major).  Reference: decode_tile / decode_rows, runtime/src/qtip.cpp:83-118, with the word
// addressing of HostLinear::word, runtime/include/behemoth/qtip.hpp:63-67; it is the inverse of pack_trellis +
// swizzle_for_kernel (src/qtip_core.cpp:194-243) followed by the codebook lookup.
//
// HBM-bound: 0.25 bytes read and 4 bytes written per weight.  A 256-thread workgroup takes a 32-row x 128-column
// patch (2 x 8 tiles) at a time: its code words are 1 KB contiguous in the kernel layout, the codebook entries are
// looked up in an LDS copy of the table, the decoded patch is staged in LDS and leaves as 512-byte row segments.
#include "misc.hpp"
#include "qtip_internal.hpp"

namespace qtipmi {
namespace {

constexpr int kLdsStride = 132;  // floats per staged patch row: 128 columns + padding, 16-byte aligned

__global__ __launch_bounds__(256) void decode_trellis_kernel(const uint16_t* __restrict__ trellis, long n2 /* n / 32 */,
                                                            long patches_per_row, long patches,
                                                            const float* __restrict__ entry_f,
                                                            float* __restrict__ out, long ld) {
  __shared__ float2 table[kLutEntries];      // the 1024 codebook entries: random lookups stay inside the CU
  __shared__ uint32_t words[256];            // 4 blocks x 128 u16, as stored
  __shared__ float patch[32 * kLdsStride];
  const int u = threadIdx.x;
#pragma unroll
  for (int k = 0; k < kLutEntries / 256; ++k) table[u + 256 * k] = reinterpret_cast<const float2*>(entry_f)[u + 256 * k];
  const uint16_t* w16 = reinterpret_cast<const uint16_t*>(words);
  for (long p = blockIdx.x; p < patches; p += gridDim.x) {
    const long i0 = p / patches_per_row, jb0 = (p % patches_per_row) * 4;
    const int nj = int(n2 - jb0 < 4 ? n2 - jb0 : 4);  // 32-column blocks in this patch
    __syncthreads();  // table ready / previous patch written out
    if (u < 64 * nj) words[u] = reinterpret_cast<const uint32_t*>(trellis)[(i0 * n2 + jb0) * 64 + u];
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int item = u + 256 * k, tile = item >> 7, t = item & 127;
      const int jb = tile >> 2, j1 = (tile >> 1) & 1, i1 = tile & 1;
      if (jb >= nj) continue;
      // 16-bit window at bit 4t of the tile's 512-bit tail-biting stream (MSB first)
      const int i = t >> 2, sh = 4 * (t & 3);
      const uint16_t* tw = w16 + jb * 128 + j1 * 2 + i1;  // word c of this tile at tw[4 * c]
      const uint32_t two = uint32_t(tw[4 * i]) << 16 | tw[4 * ((i + 1) & 31)];
      const uint32_t s = (two >> (16 - sh)) & 0xffffu;
      const uint32_t e = ((s * (s + 1u)) >> 6) & 1023u;
      // tile position of sequence element pair t = A*16 + B*4 + C*2 + D: row D*8 + A, columns C*8 + B*2 + {0, 1}
      const int A = t >> 4, B = (t >> 2) & 3, C = (t >> 1) & 1, D = t & 1;
      const int r = 16 * i1 + D * 8 + A, col = 32 * jb + 16 * j1 + C * 8 + B * 2;
      *reinterpret_cast<float2*>(&patch[r * kLdsStride + col]) = table[e];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int idx = u + 256 * k, row = idx >> 5, c4 = (idx & 31) * 4;
      if (c4 < 32 * nj)
        *reinterpret_cast<float4*>(&out[(32 * i0 + row) * ld + jb0 * 32 + c4]) =
            *reinterpret_cast<const float4*>(&patch[row * kLdsStride + c4]);
    }
  }
}

}  // namespace

void launch_decode_trellis(const uint16_t* trellis, long m, long n, const float* entry_f, float* out, long ld,
                           hipStream_t s) {
  QTIP_REQUIRE(m > 0 && n > 0 && m % 32 == 0 && n % 32 == 0, "kernel layout needs m, n multiples of 32 (m=%ld n=%ld)", m, n);
  QTIP_REQUIRE(ld >= n && ld % 4 == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0,
               "decode: output rows must be 16-byte aligned (ld=%ld)", ld);
  const long n2 = n / 32, per_row = (n2 + 3) / 4, patches = per_row * (m / 32);
  const unsigned grid = unsigned(patches < 4096 ? patches : 4096);  // workgroups walk over the patches
  decode_trellis_kernel<<<dim3(grid), dim3(256), 0, s>>>(trellis, n2, per_row, patches, entry_f, out, ld);
  QTIP_HIP(hipGetLastError());
}

}  // namespace qtipmi
