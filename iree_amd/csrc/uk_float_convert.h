// Software conversions between f32 and the 16-bit float formats, with the
// exact behaviour of the CPU ukernels' routines
// (runtime/src/iree/builtins/ukernel/common.h:651-792). Device code.
#ifndef IREE_UK_AMD_UK_FLOAT_CONVERT_H_
#define IREE_UK_AMD_UK_FLOAT_CONVERT_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace uk {

// 16-bit float with EB exponent bits -> f32: exponent field 0 (zero and
// subnormals) gives a signed zero, NaN gives a quiet NaN with all mantissa
// bits set (runtime/src/iree/builtins/ukernel/common.h:665-699).
template <int EB>
__device__ __forceinline__ float small16_to_f32(uint16_t v) {
  constexpr int MB = 15 - EB;
  const uint32_t sign = (uint32_t)(v >> 15) << 31;
  const uint32_t e = (v >> MB) & ((1u << EB) - 1);
  const uint32_t m = v & ((1u << MB) - 1);
  uint32_t bits;
  if (e == (1u << EB) - 1) {
    bits = sign | 0x7F800000u | (m ? 0x007FFFFFu : 0u);
  } else if (e == 0) {
    bits = sign;
  } else {
    bits = sign | ((e + 128u - (1u << (EB - 1))) << 23) | (m << (23 - MB));
  }
  return __uint_as_float(bits);
}

// f32 -> 16-bit float, round to nearest even, with the exponent-range
// behaviour of runtime/src/iree/builtins/ukernel/common.h:701-770 (the range
// tests sit one binade late; f32 subnormals give zero).
template <int EB>
__device__ __forceinline__ uint16_t f32_to_small16(float value) {
  constexpr int MB = 15 - EB;
  const uint32_t u = __float_as_uint(value);
  const uint32_t sign16 = (u >> 31) << 15;
  const uint32_t e32 = (u >> 23) & 0xFF;
  const uint32_t m32 = u & 0x007FFFFFu;
  constexpr uint32_t emask16 = ((1u << EB) - 1) << MB;
  constexpr uint32_t mmask16 = (1u << MB) - 1;
  if (e32 == 0xFF) return (uint16_t)(sign16 | emask16 | (m32 ? mmask16 : 0));
  if (e32 == 0) return (uint16_t)sign16;
  int ex = (int)e32 - 128;
  constexpr int half_range = 1 << (EB - 1);
  if (ex >= half_range) return (uint16_t)(sign16 | emask16);
  if (ex < -half_range) return (uint16_t)sign16;
  constexpr int drop = 23 - MB;
  constexpr uint32_t even_bit = 1u << drop;
  constexpr uint32_t odd_bit = even_bit >> 1;
  uint32_t biased = m32 + ((m32 & even_bit) ? odd_bit : odd_bit - 1);
  if (biased > 0x007FFFFFu) {
    biased = 0;
    ++ex;
  }
  return (uint16_t)(sign16 | ((uint32_t)(ex + half_range) << MB) | (biased >> drop));
}

}  // namespace uk

#endif  // IREE_UK_AMD_UK_FLOAT_CONVERT_H_
