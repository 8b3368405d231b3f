// Shared device-side helpers for the gfx950 ukernel translation units.
#ifndef IREE_UK_AMD_DEVICE_COMMON_H_
#define IREE_UK_AMD_DEVICE_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace uk {

// Unsigned 32-bit division by a runtime constant through a multiply-high:
// n / d == umulhi(n, mul) >> shift for every n < 2^31 (round-up method with a
// 32-bit multiplier; exact on that range for every d in [1, 2^31)).
struct FastDiv {
  uint32_t mul;
  uint32_t shift;
  uint32_t d;
  FastDiv() : mul(0), shift(0), d(1) {}
  explicit FastDiv(uint32_t divisor) : d(divisor) {
    if (divisor <= 1) {
      mul = 0;
      shift = 0;
      d = 1;
      return;
    }
    uint32_t l = 0;
    while ((1ull << l) < divisor) ++l;  // l = ceil(log2(d))
    // mul = floor(2^(32+l-1) / d) + 1 fits 32 bits and is exact for n < 2^31.
    uint64_t m = ((1ull << (32 + l - 1)) / divisor) + 1;
    mul = (uint32_t)m;
    shift = l - 1;
  }
  __host__ __device__ __forceinline__ uint32_t div(uint32_t n) const {
    if (d == 1) return n;
#if defined(__HIP_DEVICE_COMPILE__)
    return __umulhi(n, mul) >> shift;
#else
    return (uint32_t)(((uint64_t)n * mul) >> 32) >> shift;
#endif
  }
  __host__ __device__ __forceinline__ void divmod(uint32_t n, uint32_t& q,
                                                  uint32_t& r) const {
    q = div(n);
    r = n - q * d;
  }
};

// Largest power of two <= cap that divides v (v == 0 counts as divisible).
inline int64_t pow2_divisor(int64_t v, int64_t cap) {
  int64_t p = cap;
  if (v < 0) v = -v;
  while (p > 1 && (v % p) != 0) p >>= 1;
  return p;
}

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace uk

#endif  // IREE_UK_AMD_DEVICE_COMMON_H_
