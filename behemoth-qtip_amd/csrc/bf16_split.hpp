// bf16 hi/lo split of an fp32 value, as bit patterns: x = hi + lo + O(2^-16 |x|) with hi = bf16(x) and
// lo = bf16(x - hi), both rounded to nearest even (the operand form of the reference's prod-cache GEMM,
// src/quantizer.cpp:66-76, split_kernel / diff_split_kernel).  Device code only.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace qtipmi {

__device__ __forceinline__ uint32_t bf16_rne_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}

__device__ __forceinline__ void bf16_split_bits(float x, uint32_t& hi, uint32_t& lo) {
  hi = bf16_rne_bits(x);
  lo = bf16_rne_bits(x - __uint_as_float(hi << 16));
}

}  // namespace qtipmi
