// Exhaustive host check of the first-moment tables in csrc/q4adamw_tables.h, over every fp32
// bit pattern a quotient can take (|q| <= 1 plus a margin).  Built and run by
// tests/test_abi_and_tables.py with g++ -fopenmp; prints one line per check, "ok" last.
//
// 1. Nearest rounding: wherever the 256-entry half-indexed bucket table decides a code on
//    its own ((q > hi) == (q > lo)), every value within kSlack ulps of q -- the fused
//    kernel's quotient is within 3 ulps of the exactly divided one -- has that code under
//    the closed form  code = #{j : mid[j] < x}.
// 2. Stochastic rounding: base + (q >= thr) equals #{j : Q[j] <= q} exactly.
#include <cmath>
#include <cstdint>
#include <cstdio>

#include "../../quantfour_adamw_cuda_amd/csrc/q4adamw_tables.h"

using namespace q4;

static const int kSlack = 3;

// high byte of q converted to half precision toward zero (v_cvt_pkrtz_f16_f32)
static inline uint32_t half_index(float q) {
  const uint32_t b = f2bits(q), sign = b >> 31, mag = b & 0x7fffffffu, e8 = mag >> 23;
  if (e8 >= 113u) return (sign << 7) | ((e8 - 112u) << 2) | ((mag >> 21) & 3u);   // normal half, |q| < 65536
  const uint32_t m = (uint32_t)std::floor(std::fabs((double)q) * 16777216.0);    // subnormal half: 10-bit mantissa
  return (sign << 7) | (m >> 8);
}

// order-preserving map between floats and unsigned integers
static inline uint32_t to_key(uint32_t b) { return (b & 0x80000000u) ? ~b : (b | 0x80000000u); }
static inline uint32_t from_key(uint32_t k) { return (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k; }

static inline int exact_code(float x) {
  int c = 0;
  for (int j = 0; j < 15; ++j) c += bits2f(kQmidMBits[j]) < x;
  return c;
}

int main() {
  static MtabEntry table[256];
  static SrEntry sr[256];
  for (uint32_t h = 0; h < 256; ++h) {
    table[h] = mtab_entry(half_index_bucket(h));
    sr[h] = sr_entry(h);
  }
  const uint32_t lo_key = to_key(f2bits(-1.0000019f)), hi_key = to_key(f2bits(1.0000019f));   // +-16 ulps beyond 1
  long long decided = 0, undecided = 0, bad = 0, bad_sr = 0;
#pragma omp parallel for schedule(static) reduction(+ : decided, undecided, bad, bad_sr)
  for (long long k = lo_key; k <= (long long)hi_key; ++k) {
    const float q = bits2f(from_key((uint32_t)k));
    const uint32_t h = half_index(q);
    const MtabEntry e = table[h];
    const bool above_hi = q > bits2f(e.hi), above_lo = q > bits2f(e.lo);   // the base nibble is part of the bound, as in the kernel
    if (above_hi == above_lo) {
      const int code = (int)(e.lo & 15u) + (above_hi ? 1 : 0);
      ++decided;
      // the sign of a quotient is exact, so the neighbourhood does not cross zero
      uint32_t k_lo = (uint32_t)k - kSlack, k_hi = (uint32_t)k + kSlack;
      const uint32_t zero_neg = to_key(0x80000000u), zero_pos = to_key(0u);
      if ((uint32_t)k <= zero_neg) { if (k_hi > zero_neg) k_hi = zero_neg; }
      else if (k_lo < zero_pos) k_lo = zero_pos;
      if (exact_code(bits2f(from_key(k_lo))) != code || exact_code(bits2f(from_key(k_hi))) != code) ++bad;
    } else {
      ++undecided;
    }
    int k_raw = 0;
    for (int j = 0; j < 16; ++j) k_raw += bits2f(kQmapMBits[j]) <= q;
    // -0.0 is in the negative zero bucket (base 7) although 0 <= -0.0 holds: both readings
    // give the same final code (see q4adamw_tables.h), so it is exempt here
    if (f2bits(q) != 0x80000000u && (int)(sr[h].base + (q >= bits2f(sr[h].thr) ? 1u : 0u)) != k_raw) ++bad_sr;
  }
  std::printf("nearest: %lld decided, %lld undecided, %lld wrong\n", decided, undecided, bad);
  std::printf("stochastic: %lld wrong interval numbers\n", bad_sr);
  if (bad || bad_sr || undecided <= 0 || undecided > 15 * (2 * 6 + 40)) return 1;
  std::printf("ok\n");
  return 0;
}
