/*
 * Host checks of the short correctly rounded sequences of the fused kernel's exact parameter
 * update (sqrt_rn, div_by_reciprocal, div_rn in quantfour_adamw_cuda_amd/csrc/q4adamw_device.h),
 * restated here in C with the same operations (fmaf is a correctly rounded fma).
 *
 * 1. Division.
 *     y  = RN(1/c)                 (given: computed in fp64 on the host for a uniform divisor,
 *                                   or the hardware estimate plus one Newton step, which the
 *                                   GPU walk of every divisor shows to be RN(1/c))
 *     q0 = RN(x * y)
 *     r  = fma(-c, q0, x)
 *     q  = fma(r, y, q0)           claimed: q == RN(x / c) for all x, c without under/overflow
 *
 * Argument.  With t = x/c, d = y - 1/c (|d| <= half an ulp of 1/c) the last fma rounds
 * t + r*d (+ r's own rounding when q0 is more than an ulp off).  |r| <= 3 ulp(t), so the
 * rounded value is within 4.5 * 2^-24 ulp(t) of t, and q == RN(t) unless t lies within that
 * distance of a midpoint of two neighbouring floats.  Scale x = X * 2^-23, c = C * 2^-23
 * with integers 2^23 <= X, C < 2^24 (signs and exponents do not matter).  The midpoints are
 * M / 2^25 (t < 1) or M / 2^24 (t >= 1) with M odd, and
 *     |t - midpoint| = |X * 2^25 - M * C| / (C * 2^25)     resp.  |X * 2^24 - M * C| / (C * 2^24)
 * so "within 4.5 * 2^-24 ulp" means |e| <= 9 for the integer e = X * 2^k - M * C, e != 0.
 * For every divisor C and every |e| <= kMaxE (16) this program solves that congruence for
 * (X, M), i.e. it lists EVERY numerator whose quotient comes that close to a midpoint, and
 * runs the sequence on it with real fp32 arithmetic.  All of them must come out correctly
 * rounded; together with the bound above that covers all 2^46 mantissa pairs.
 * It also runs a few 10^8 random pairs, and shows that the rule fails when y is off by one
 * ulp (the reason the GPU walk has to establish y == RN(1/c) for the hardware path).
 *
 * 2. Square root.  sqrt_rn takes an estimate s within one ulp of the root and decides between
 * s and its two neighbours by the signs of s_dn * s - v and s_up * s - v.  Every mantissa of
 * two neighbouring binades (which cover every parity of the exponent) is run with the estimate
 * set to the correctly rounded root and to each of its neighbours.
 *
 * Prints "ok ..." and exits 0, or prints the first failures and exits 1.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

enum { kMaxE = 16 };

static inline uint32_t f2b(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static inline float div3(float x, float c, float y) {
  const float q0 = x * y;
  const float r = fmaf(-c, q0, x);
  return fmaf(r, y, q0);
}

static inline float rn_reciprocal(float c) { return (float)(1.0 / (double)c); }

static inline float b2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* sqrt_rn with the estimate passed in */
static inline float sqrt_fix(float v, float s) {
  const uint32_t s_dn = f2b(s) - 1u, s_up = f2b(s) + 1u;
  const uint32_t above_dn = f2b(fmaf(b2f(s_dn), s, -v)) >> 31;
  const uint32_t above_up = f2b(fmaf(b2f(s_up), s, -v)) >> 31;
  return b2f(s_dn + above_dn + above_up);
}

static long g_cases, g_bad;

static void try_pair(uint32_t X, uint32_t C) {
  const float x = (float)X, c = (float)C;   /* both exact: 24-bit integers */
  const float want = x / c, got = div3(x, c, rn_reciprocal(c));
  ++g_cases;
  if (f2b(want) != f2b(got)) {
    if (g_bad < 10) printf("FAIL X=%u C=%u got %08x want %08x\n", X, C, f2b(got), f2b(want));
    ++g_bad;
  }
}

/* inverse of an odd number modulo 2^32 */
static uint32_t inv32(uint32_t a) {
  uint32_t x = a;   /* correct to 3 bits */
  for (int i = 0; i < 5; ++i) x *= 2u - a * x;
  return x;
}

int main(int argc, char **argv) {
  const long random_pairs = argc > 1 ? atol(argv[1]) : 200000000L;
  for (uint32_t C = 1u << 23; C < (1u << 24); ++C) {
    int a = 0;
    while (!((C >> a) & 1u)) ++a;
    if ((1 << a) > kMaxE) continue;   /* e is a multiple of 2^a */
    const uint32_t Cp = C >> a, inv = inv32(Cp);
    for (int ep = -(kMaxE >> a); ep <= (kMaxE >> a); ++ep) {
      if (ep == 0) continue;
      const int64_t e = (int64_t)ep * (1 << a);
      /* k = 25: quotients below 1; k = 24: quotients from 1 on.  M * C' = -e' modulo 2^(k-a) */
      for (int k = 24; k <= 25; ++k) {
        const int bits = k - a;
        const uint32_t mask = (bits >= 32) ? 0xffffffffu : ((1u << bits) - 1u);
        const uint32_t M0 = ((uint32_t)(-(int32_t)ep) * inv) & mask;
        for (uint64_t M = M0; M < (1ull << 25); M += (1ull << bits)) {
          if (!(M & 1) || M <= (1ull << 24)) continue;
          const uint64_t num = M * (uint64_t)C + (uint64_t)e;   /* M*C >= 2^47, |e| small */
          if (num & ((1ull << k) - 1)) continue;
          const uint64_t X = num >> k;
          if (X < (1u << 23) || X >= (1u << 24)) continue;
          if (k == 25 ? X >= C : X < C) continue;
          try_pair((uint32_t)X, C);
        }
      }
    }
  }
  const long worst = g_cases;
  /* random pairs, divisors with all-ones and all-zero mantissas among them */
  uint64_t s = 0x9E3779B97F4A7C15ull;
  for (long i = 0; i < random_pairs; ++i) {
    s ^= s << 13; s ^= s >> 7; s ^= s << 17;
    uint32_t X = (1u << 23) | (uint32_t)(s & 0x7fffffu), C = (1u << 23) | (uint32_t)((s >> 23) & 0x7fffffu);
    if ((i & 15) == 0) C = (1u << 24) - 1u - (uint32_t)((s >> 50) & 3u);
    if ((i & 15) == 1) C = (1u << 23) + (uint32_t)((s >> 50) & 3u);
    try_pair(X, C);
  }
  /* the premise matters: with a reciprocal one ulp off, 1 / (2 - 2^-23) comes out wrong */
  {
    const float c = 1.99999988079071044921875f, y = rn_reciprocal(c);
    float y_off; uint32_t u = f2b(y) - 1u; memcpy(&y_off, &u, 4);
    if (f2b(div3(1.0f, c, y)) != f2b(1.0f / c) || f2b(div3(1.0f, c, y_off)) == f2b(1.0f / c)) {
      printf("FAIL the all-ones divisor behaves differently from what this check documents\n");
      ++g_bad;
    }
  }
  /* square roots: every mantissa of [0.5, 2), estimates RN - 1 ulp, RN, RN + 1 ulp */
  long roots = 0;
  for (uint32_t u = 0x3f000000u; u < 0x40000000u; ++u) {
    const float v = b2f(u), t = sqrtf(v);
    for (int k = -1; k <= 1; ++k) {
      ++roots;
      if (f2b(sqrt_fix(v, b2f(f2b(t) + (uint32_t)k))) != f2b(t)) {
        if (g_bad < 10) printf("FAIL sqrt v=%08x estimate %+d ulp\n", u, k);
        ++g_bad;
      }
    }
  }
  if (g_bad) { printf("%ld failures in %ld cases\n", g_bad, g_cases + roots); return 1; }
  printf("ok %ld near-midpoint quotients, %ld random, %ld square roots\n", worst, g_cases - worst, roots);
  return 0;
}
