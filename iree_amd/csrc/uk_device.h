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
__device__ __forceinline__ float widen16(uint16_t h) {
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
  return __uint_as_float(bits);
}

// f32 -> 16-bit float, round to nearest even, with the reference's quirks
// (common.h:701-770): f32 subnormals and results below the exponent range give
// zero, overflow gives infinity, and the lowest in-range exponent is encoded
// with exponent field 0 plus the rounded mantissa bits.
template <int EBITS>
__device__ __forceinline__ uint16_t narrow16(float f) {
  constexpr int MBITS = 15 - EBITS;
  constexpr int HALF = 1 << (EBITS - 1);
  constexpr uint32_t EMASK = ((1u << EBITS) - 1u) << MBITS;
  constexpr uint32_t MMASK = (1u << MBITS) - 1u;
  const uint32_t bits = __float_as_uint(f);
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

}  // namespace uk

#endif  // IREE_AMD_CSRC_UK_DEVICE_H_
