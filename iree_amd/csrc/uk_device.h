// Device-side helpers shared by the kernel translation units.
#ifndef IREE_AMD_CSRC_UK_DEVICE_H_
#define IREE_AMD_CSRC_UK_DEVICE_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace uk {

// 16-bit float -> f32 with the reference's generic-path semantics
// (common.h:665-699): a zero exponent field (zeros AND subnormals) widens to a
// signed zero, NaNs become the all-ones-mantissa quiet NaN. EBITS is 5 for
// f16, 8 for bf16.
template <int EBITS>
__host__ __device__ __forceinline__ float widen16(uint16_t h) {
  constexpr int MBITS = 15 - EBITS;
  constexpr uint32_t EMAX = (1u << EBITS) - 1u;
  const uint32_t sign = (uint32_t)(h >> 15) << 31;
  const uint32_t e = (h >> MBITS) & EMAX;
  const uint32_t m = h & ((1u << MBITS) - 1u);
  uint32_t bits;
  if (e == EMAX) {
    bits = sign | 0x7F800000u | (m ? 0x007FFFFFu : 0u);
  } else if (e == 0) {
    bits = sign;
  } else {
    bits = sign | ((e + 127u - ((1u << (EBITS - 1)) - 1u)) << 23) | (m << (23 - MBITS));
  }
  return __builtin_bit_cast(float, bits);
}

// f32 -> 16-bit float, round to nearest even, with the reference's quirks
// (common.h:701-770): f32 subnormals and results below the exponent range give
// zero, overflow gives infinity, and the lowest in-range exponent is encoded
// with exponent field 0 plus the rounded mantissa bits. This is the
// conversion spelled out step by step; narrow16 below is what the kernels call.
template <int EBITS>
__host__ __device__ __forceinline__ uint16_t narrow16_by_steps(float f) {
  constexpr int MBITS = 15 - EBITS;
  constexpr int HALF = 1 << (EBITS - 1);
  constexpr uint32_t EMASK = ((1u << EBITS) - 1u) << MBITS;
  constexpr uint32_t MMASK = (1u << MBITS) - 1u;
  const uint32_t bits = __builtin_bit_cast(uint32_t, f);
  const uint32_t sign = (bits >> 31) << 15;
  const uint32_t e32 = (bits >> 23) & 0xFFu;
  const uint32_t m32 = bits & 0x007FFFFFu;
  if (e32 == 0xFFu) return (uint16_t)(sign | EMASK | (m32 ? MMASK : 0u));
  if (e32 == 0) return (uint16_t)sign;
  int e = (int)e32 - 128;
  if (e >= HALF) return (uint16_t)(sign | EMASK);
  if (e < -HALF) return (uint16_t)sign;
  constexpr uint32_t EVEN = 1u << (23 - MBITS);
  constexpr uint32_t ODD = EVEN >> 1;
  uint32_t m = m32 + ((m32 & EVEN) ? ODD : ODD - 1u);
  if (m > 0x007FFFFFu) {
    m = 0;
    ++e;
  }
  return (uint16_t)(sign | ((uint32_t)(e + HALF) << MBITS) | (m >> (23 - MBITS)));
}

// The same function without branches (an epilogue that rounds 256 accumulators
// per lane with the steps above took 23 us of a 154 us f16f16f16 4096^3
// launch). For every f32 exponent field that the steps treat as in range
// (1 .. 254 for bf16, which has f32's exponent range; 112 .. 143 for f16) they
// amount to adding the rounding bias to the whole word, letting the mantissa
// carry into the exponent (common.h:741-752 says as much), and rebasing the
// exponent; that includes the reference's encodings at both ends of the f16
// range (field 0 with mantissa bits for 2^-15 <= |x| < 2^-14, field 31 with
// mantissa bits for 2^16 <= |x| < 2^17, and the carry out of that into bit
// 15). Below the range: signed zero; above: infinity; NaN: all mantissa bits.
// (The hardware's v_cvt_f16_f32 agrees with the steps between the smallest
// normal f16 and overflow only; a test of the range in front of it, as a
// branch per value, per four values or per wavefront, was slower than this.)
template <int EBITS>
__host__ __device__ __forceinline__ uint16_t narrow16(float f) {
  constexpr int MBITS = 15 - EBITS;
  constexpr int SHIFT = 23 - MBITS;                              // mantissa bits dropped
  constexpr uint32_t LOWEST = 128u - (1u << (EBITS - 1));        // lowest in-range f32 exponent field (0 for bf16)
  constexpr uint32_t EMASK = ((1u << EBITS) - 1u) << MBITS, MMASK = (1u << MBITS) - 1u;
  const uint32_t bits = __builtin_bit_cast(uint32_t, f);
  const uint32_t mag = bits & 0x7FFFFFFFu, sign = (bits >> 16) & 0x8000u;
  uint32_t r = ((mag + ((1u << (SHIFT - 1)) - 1u) + ((mag >> SHIFT) & 1u)) >> SHIFT) - (LOWEST << MBITS);
  if constexpr (EBITS == 8) {
    r = mag < 0x00800000u ? 0u : r;                              // zeros and f32 subnormals
  } else {
    r = mag < (LOWEST << 23) ? 0u : r;                           // below the range (zeros, f32 subnormals included)
    r = mag >= ((LOWEST + (2u << (EBITS - 1))) << 23) ? EMASK : r;   // above it, infinity included
  }
  r = mag == 0x7F800000u ? EMASK : r;
  r = mag > 0x7F800000u ? (EMASK | MMASK) : r;
  return (uint16_t)(sign | r);
}

}  // namespace uk

#endif  // IREE_AMD_CSRC_UK_DEVICE_H_
