// Scalar codec of the NVFP4 format (reference: the format definition in src/nvfp4.hpp:15-57 and its use in
// src/nvfp4.cpp:12-70, src/nvfp4_gpu.hip:16-63), shared by the host quantizer and the device kernels.  Everything is
// done on the bit patterns: E4M3 by rounding the fp32 pattern to nearest even at its third mantissa bit (a carry runs
// into the exponent by itself), E2M1 by comparing with the seven midpoints between neighbouring magnitudes.
#pragma once
#include <cstdint>

#if defined(__HIPCC__)
#define QTIP_NV_FN __host__ __device__ __forceinline__
#else
#define QTIP_NV_FN inline
#endif

namespace qtipmi {
namespace nvcodec {

QTIP_NV_FN uint32_t bits_of(float f) { return __builtin_bit_cast(uint32_t, f); }
QTIP_NV_FN float float_of(uint32_t u) { return __builtin_bit_cast(float, u); }

constexpr uint32_t kE4M3Top = 126;            // 448, the largest finite E4M3 code
constexpr uint32_t kBits448 = 0x43e00000u;    // 448.0f
constexpr uint32_t kBitsMinNormal = 0x3c800000u;  // 2^-6, the smallest normal E4M3 magnitude

// E4M3 code (0 .. 126) of |x| for a float that is not NaN; magnitudes above 448, infinity included, give 126
QTIP_NV_FN uint32_t e4m3_of_magnitude(float x) {
  uint32_t u = bits_of(x) & 0x7fffffffu;
  if (u > kBits448) u = kBits448;
  if (u < kBitsMinNormal) {
    // fixed point with step 2^-9: adding 1.5 * 2^23 leaves the rounding (to nearest, ties to even) to the adder;
    // 8 is the first normal code
    return bits_of(float_of(u) * 512.f + 12582912.f) & 15u;
  }
  u += 0x7ffffu + ((u >> 20) & 1u);
  return (u >> 20) - (120u << 3);  // exponent bias 127 -> 7
}

// value of the E4M3 code c <= 126
QTIP_NV_FN float e4m3_value(uint32_t c) {
  const uint32_t e = c >> 3, m = c & 7u;
  return e ? float_of(((e + 120u) << 23) | (m << 20)) : float(m) * 0.001953125f;
}

// magnitudes of the E2M1 codes 0 .. 7: 0, 0.5, 1, 1.5, 2, 3, 4, 6
QTIP_NV_FN float e2m1_value(uint32_t c) {
  const uint32_t e = c >> 1, m = c & 1u;
  return e ? float_of(((e + 126u) << 23) | (m << 22)) : 0.5f * float(m);
}

// E2M1 code of the magnitude nearest to a >= 0 (0 for NaN); a midpoint goes to the even code of its two neighbours,
// so the comparison is strict where the upper neighbour is odd.  The last step, 4 against 6, compares the two fp32
// distances themselves: up to 2^25 that is a > 5, and beyond it, where 4 and 6 are no further apart than the spacing
// of the floats, it gives what a nearest-value search in fp32 gives (src/nvfp4.cpp:27-38), 4 for every other float.
QTIP_NV_FN uint32_t e2m1_of_magnitude(float a) {
  const float to6 = a - 6.f, to4 = a - 4.f;
  return uint32_t(a > 0.25f) + uint32_t(a >= 0.75f) + uint32_t(a > 1.25f) + uint32_t(a >= 1.75f) +
         uint32_t(a > 2.5f) + uint32_t(a >= 3.5f) + uint32_t((to6 < 0 ? -to6 : to6) < (to4 < 0 ? -to4 : to4));
}

// what execution sees of a product: fp32 rounded to bf16 (nearest even), as fp32
QTIP_NV_FN float through_bf16(float f) {
  uint32_t u = bits_of(f);
  u += 0x7fffu + ((u >> 16) & 1u);
  return float_of(u & 0xffff0000u);
}

}  // namespace nvcodec
}  // namespace qtipmi
