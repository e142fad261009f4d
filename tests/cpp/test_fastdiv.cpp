// Host check of arraymancer_amd/csrc/fastdiv.h against the machine's own division: every divisor up to 4096 and a
// spread of larger ones (powers of two and their neighbours, primes, 2^31), each against dividends at the places
// where a wrong multiplier or shift shows: multiples of the divisor and their neighbours, the ends of the 32-bit
// range, and a pseudo-random sample.
#include <cstdio>
#include <cstdint>
#include <vector>
#include "../../arraymancer_amd/csrc/fastdiv.h"

int main() {
  std::vector<uint32_t> divisors;
  for (uint32_t d = 1; d <= 4096; ++d) divisors.push_back(d);
  for (int b = 12; b <= 31; ++b)
    for (int64_t off = -2; off <= 2; ++off) {
      const int64_t d = ((int64_t)1 << b) + off;
      if (d >= 1 && d <= ((int64_t)1 << 31)) divisors.push_back((uint32_t)d);
    }
  for (uint32_t d : {4099u, 36864u, 65521u, 65537u, 1000003u, 16777259u, 268435399u, 2147483647u, 3u * 715827881u}) divisors.push_back(d);
  uint64_t checked = 0, bad = 0, x = 88172645463325252ull;
  for (uint32_t d : divisors) {
    if (d > (1u << 31)) continue;
    const am::FastDiv f(d);
    std::vector<uint32_t> ns = {0u, 1u, 2u, d - 1, d, d + 1, 2 * d - 1, 2 * d, 0x7fffffffu, 0x80000000u, 0x80000001u, 0xfffffffeu, 0xffffffffu};
    const uint32_t top = 0xffffffffu / d;
    for (uint32_t k : {top, top - 1, top / 2, top / 3 + 1})
      for (int64_t off = -1; off <= 1; ++off) {
        const int64_t n = (int64_t)k * d + off;
        if (n >= 0 && n <= 0xffffffffll) ns.push_back((uint32_t)n);
      }
    for (int i = 0; i < 64; ++i) {
      x ^= x << 13; x ^= x >> 7; x ^= x << 17;
      ns.push_back((uint32_t)x);
      ns.push_back((uint32_t)(x >> 32) % (d < 0x10000u ? d * 65536u : 0xffffffffu));
    }
    for (uint32_t n : ns) {
      uint32_t r;
      const uint32_t q = f.divmod(n, r);
      ++checked;
      if (q != n / d || r != n % d) {
        if (++bad <= 10) std::printf("FAILED %u / %u: got %u rem %u, want %u rem %u\n", n, d, q, r, n / d, n % d);
      }
    }
  }
  std::printf("%llu divisions checked, %llu wrong\n", (unsigned long long)checked, (unsigned long long)bad);
  return bad ? 1 : 0;
}
