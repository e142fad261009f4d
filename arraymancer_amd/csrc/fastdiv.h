// Unsigned 32-bit division by a divisor that is fixed for a whole launch: the host derives a multiplier and two shift
// counts once, the kernel divides with a high multiply, a subtraction, two shifts and an addition instead of the
// twenty-odd instructions of a division by a value the compiler does not know. Exact for every 32-bit dividend and
// every divisor from 1 to 2^31 (the round-up method of Granlund and Montgomery, "Division by invariant integers
// using multiplication", 1994, figure 4.1). Plain C++: the same code runs on the host, where the tests check it.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define AM_HD __host__ __device__ __forceinline__
#else
#define AM_HD inline
#endif

namespace am {

struct FastDiv {
  uint32_t d, m, s1, s2;

  FastDiv() : d(1), m(1), s1(0), s2(0) {}
  explicit FastDiv(uint32_t divisor) : d(divisor ? divisor : 1) {
    uint32_t l = 0;                                   // ceil(log2 d)
    while (l < 32 && ((uint64_t)1 << l) < d) ++l;
    m = (uint32_t)((((uint64_t)1 << 32) * (((uint64_t)1 << l) - d)) / d + 1);
    s1 = l < 1 ? l : 1;
    s2 = l - s1;
  }
  AM_HD uint32_t div(uint32_t n) const {
    const uint32_t t = (uint32_t)(((uint64_t)m * n) >> 32);
    return (t + ((n - t) >> s1)) >> s2;
  }
  // quotient, and the remainder through `rem`
  AM_HD uint32_t divmod(uint32_t n, uint32_t& rem) const {
    const uint32_t q = div(n);
    rem = n - q * d;
    return q;
  }
};

}  // namespace am
