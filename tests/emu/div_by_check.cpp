// Host check of amoe::div_by (csrc/common.h: one multiplication and two fused multiply-adds with y = 1/b) against the
// correctly rounded IEEE quotient a / b, over the operand ranges of the DAC stage (|a| <= |b| scaled, b a positive
// input range or quantisation step).  Built on demand by tests/test_oracle.py with the stand-in headers of tests/emu.
#include <cstdint>
#include <cstring>
#include <cmath>
#include "common.h"

static inline float bits_f(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }
static inline uint32_t f_bits(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
static inline bool same(float a, float b) { return f_bits(a) == f_bits(b); }

extern "C" {

// every one of the 2^23 mantissas of the dividend (both signs, three binades) against one divisor
long long div_by_mismatches_all_mantissas(float b) {
  const float y = 1.0f / b;
  long long bad = 0;
  for (uint32_t m = 0; m < (1u << 23); m++) {
    for (uint32_t e : {126u, 127u, 120u}) {
      const float a = bits_f((e << 23) | m);
      if (!same(amoe::div_by(a, b, y), a / b)) bad++;
      if (!same(amoe::div_by(-a, b, y), -a / b)) bad++;
    }
  }
  return bad;
}

static inline uint64_t next(uint64_t& s) { s ^= s << 13; s ^= s >> 7; s ^= s << 17; return s; }

// n random (dividend, divisor) pairs; kind 0: any mantissas, divisor in [2^-8, 2^8), |dividend| <= divisor (the clip
// before the first division); kind 1: divisor with an all-ones mantissa tail; kind 2: divisor next to a power of two;
// kind 3: divisors 1 / (2^j - 1) and 2 / (2^j - 2), the quantisation steps, dividend in [-1, 1]
long long div_by_mismatches_random(uint64_t seed, long long n, int kind) {
  uint64_t s = seed * 0x9E3779B97F4A7C15ull + 1;
  long long bad = 0;
  for (long long i = 0; i < n; i++) {
    const uint64_t r1 = next(s), r2 = next(s);
    uint32_t mb = (uint32_t)(r1 & 0x7fffff);
    const uint32_t eb = 119 + (uint32_t)((r1 >> 23) % 16);
    if (kind == 1) mb |= 0x7fffffu >> ((r1 >> 40) % 12);
    if (kind == 2) mb = ((r1 >> 40) & 1) ? (uint32_t)((r1 >> 41) % 8) : 0x7fffffu - (uint32_t)((r1 >> 41) % 8);
    float b = bits_f((eb << 23) | mb);
    float a;
    if (kind == 3) {
      const int j = 2 + (int)((r1 >> 30) % 12);
      b = ((r1 >> 50) & 1) ? 1.0f / (float)((1 << j) - 1) : 2.0f / (float)((1 << j) - 2);
      a = (float)((double)(r2 >> 11) / 9007199254740992.0 * 2.0 - 1.0);
    } else {
      a = b * (float)((double)(r2 >> 11) / 9007199254740992.0 * 2.0 - 1.0);     // |a| <= b
      if ((r2 & 7) == 0) a = (r2 & 8) ? b : -b;                                    // the clipped values themselves
    }
    if (!same(amoe::div_by(a, b, 1.0f / b), a / b)) bad++;
  }
  return bad;
}

}  // extern "C"
