// Code books, midpoint tables and the first-moment bucket table of the fused 4-bit
// AdamW step.  Usable from host and device code; no torch, no HIP runtime types.
//
// The four tables carry the values of the reference's constant arrays
// (optim/cuda_adamw_kernels.cu:25-98) as exact fp32 bit patterns.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define Q4_HD __host__ __device__
#else
#define Q4_HD
#endif

namespace q4 {

Q4_HD constexpr float bits2f(uint32_t u) { return __builtin_bit_cast(float, u); }
Q4_HD constexpr uint32_t f2bits(float f) { return __builtin_bit_cast(uint32_t, f); }

// first moment: signed dynamic-exponent map (cuda_adamw_kernels.cu:25-42)
constexpr uint32_t kQmapMBits[16] = {
    0xbf633333u, 0xbf29999au, 0xbee00000u, 0xbe59999au, 0xbd9eb852u, 0xbd051eb8u,
    0xbbb43958u, 0x00000000u, 0x3bb43958u, 0x3d051eb8u, 0x3d9eb852u, 0x3e59999au,
    0x3ee00000u, 0x3f29999au, 0x3f633333u, 0x3f800000u};
// decision thresholds between neighbouring entries (cuda_adamw_kernels.cu:44-61);
// entries 3 and 10 are one ulp below the fp32 mean of their neighbours: the literal
// table is authoritative
constexpr uint32_t kQmidMBits[15] = {
    0xbf466666u, 0xbf0ccccdu, 0xbea66666u, 0xbe147ae1u, 0xbd6147aeu,
    0xbc9ba5e3u, 0xbb343958u, 0x3b343958u, 0x3c9ba5e3u, 0x3d6147aeu,
    0x3e147ae1u, 0x3ea66666u, 0x3f0ccccdu, 0x3f466666u, 0x3f71999au};
// second moment: (k+1)/16 (cuda_adamw_kernels.cu:63-80) and thresholds (2k+1)/32,
// k = 1..15 (cuda_adamw_kernels.cu:82-98); all exact in fp32
Q4_HD constexpr float qmap_v(int k) { return (float)(k + 1) * 0.0625f; }
Q4_HD constexpr float qmid_v(int k) { return (float)(2 * k + 3) * 0.03125f; }

// ---------------------------------------------------------------------------
// Bucket table for the first-moment quantizer.
//
// The code of a normalised value q is the number of thresholds strictly below it
// (closed form of the binary search at cuda_adamw_kernels.cu:167-194).  The top
// eleven bits of q's fp32 pattern (sign, exponent, two mantissa bits) select one
// of 2048 buckets; no bucket holds more than one of the fifteen thresholds, so
//     code = base + (thr < q)
// with base = number of thresholds below the whole bucket and thr = the threshold
// inside it, if any.
//
// The fused kernel's fast path knows q only to within three ulps (it multiplies by a
// refined reciprocal instead of dividing), so each entry stores a guard band
// around thr instead of thr itself:
//     x = fp32 "lo" bound, at least kGuardUlps below thr, low four bits = base
//     y = fp32 "hi" bound, kGuardUlps above thr
// q > hi  => the exactly divided value is above thr as well
// q <= lo => the exactly divided value is not above thr
// anything in between is decided by the exact path.
// Buckets without a threshold use a bound that no normalised value exceeds.
// ---------------------------------------------------------------------------
constexpr uint32_t kMtabEntries = 2048;
constexpr uint32_t kGuardUlps = 6;
constexpr uint32_t kNoThr = 0x7f000000u;  // 1.7e38

struct MtabEntry {
  uint32_t lo;  // fp32 bits, low nibble = base
  uint32_t hi;  // fp32 bits
};

Q4_HD constexpr MtabEntry mtab_entry(uint32_t idx) {
  const uint32_t sign = (idx >> 10) & 1u, mag = idx & 1023u, e = mag >> 2;
  uint32_t base = 0, thr = 0;
  bool has = false;
  if (e == 255u) {           // nan (an infinite quotient only occurs in blocks that take the
    base = 0u;               // exact path): no threshold is below a nan
  } else if (e >= 128u) {    // |q| >= 2: beyond every threshold
    base = sign ? 0u : 15u;
  } else if (e < 118u) {     // |q| < 2^-9 < 0.00275: the seven negative thresholds are below
    base = 7u;
  } else {
    const float lo = bits2f(mag << 21), hi = bits2f((mag + 1u) << 21);
    for (int j = 0; j < 15; ++j) {
      const float t = bits2f(kQmidMBits[j]);
      if (!sign) {           // bucket holds q in [lo, hi)
        if (t < lo) ++base;
        else if (t < hi) { thr = kQmidMBits[j]; has = true; }
      } else {               // bucket holds q in (-hi, -lo]
        if (t <= -hi) ++base;
        else if (t < -lo) { thr = kQmidMBits[j]; has = true; }
      }
    }
  }
  MtabEntry out{};
  if (!has) {
    out.lo = kNoThr | base;
    out.hi = kNoThr;
    return out;
  }
  const uint32_t s = thr & 0x80000000u, m = thr & 0x7fffffffu;
  if (!s) {  // positive threshold: lower bound has the smaller magnitude
    const uint32_t want = m - kGuardUlps;
    uint32_t c = (want & ~15u) | base;
    if (c > want) c -= 16u;
    out.lo = c;
    out.hi = m + kGuardUlps;
  } else {   // negative threshold: lower bound has the larger magnitude
    const uint32_t want = m + kGuardUlps;
    uint32_t c = (want & ~15u) | base;
    if (c < want) c += 16u;
    out.lo = c | s;
    out.hi = (m - kGuardUlps) | s;
  }
  return out;
}

// ---------------------------------------------------------------------------
// The table a workgroup of the fused kernel holds in LDS: 256 entries.
//
// The kernel converts a quotient to half precision with round-toward-zero
// (v_cvt_pkrtz_f16_f32, two quotients per instruction) and takes the high byte of
// the half (sign, five exponent bits, two mantissa bits) as the entry index.
// Truncation keeps the leading bits, so for |q| in [2^-14, 65536) that byte names
// the same bucket as the top eleven bits of the fp32 pattern, with the exponent
// re-biased by 112; every smaller magnitude (a subnormal half, exponent field 0) is
// below the smallest threshold (2.7e-3) and shares the bucket of zero, which is why
// the kernel needs no clamp.  Exponent field 31 (inf, nan) maps to the bucket of the
// same fp32 class.
// ---------------------------------------------------------------------------
constexpr uint32_t kHalfTableEntries = 256;

// bucket of the 2048-entry table that half-index h (0..255) stands for
Q4_HD constexpr uint32_t half_index_bucket(uint32_t h) {
  const uint32_t sign = (h >> 7) & 1u, e5 = (h >> 2) & 31u, m2 = h & 3u;
  const uint32_t e8 = e5 == 0u ? 0u : e5 == 31u ? 255u : e5 + 112u;
  return (sign << 10) | (e8 << 2) | (e5 == 0u ? 0u : m2);
}
static_assert((113u << 2) < 471u, "the lowest bucket that holds a threshold must be a normal half");

struct HalfTable {
  MtabEntry e[kHalfTableEntries];
};

constexpr HalfTable make_half_table() {
  HalfTable t{};
  for (uint32_t h = 0; h < kHalfTableEntries; ++h) t.e[h] = mtab_entry(half_index_bucket(h));
  return t;
}

// ---------------------------------------------------------------------------
// Stochastic rounding (first moment): the interval of a normalised value among the code
// book's entries.  k_raw = number of entries <= q (0..16); entry [k_raw] of the interval
// table holds the interval's lower end and its width, extended at both ends so that no
// case split is needed: below the first entry the width is 0 (always "up", from code -1
// to code 0), at or above the last one it is infinite (never "up").
//
// The half-indexed table gives k_raw as base + (q >= thr): thr is the code-book entry
// inside the bucket, if any (no bucket holds two).  No guard band: a value within a few
// ulps of an entry gets the same final code from either neighbouring interval.
// ---------------------------------------------------------------------------
struct SrEntry {
  uint32_t thr;   // fp32 bits of the entry inside the bucket; kNoThr if none
  uint32_t base;  // number of entries below the whole bucket
};

Q4_HD constexpr SrEntry sr_entry(uint32_t half_index) {
  const uint32_t idx = half_index_bucket(half_index);
  const uint32_t sign = (idx >> 10) & 1u, mag = idx & 1023u, e = mag >> 2;
  SrEntry out{kNoThr, 0u};
  if (e == 255u) {            // nan: interval 1 makes "up" false and the code 1 - 1 + 0 = 0
    out.base = 1u;
    return out;
  }
  if (e >= 128u) {            // |q| >= 2
    out.base = sign ? 0u : 16u;
    return out;
  }
  if (mag == 0u) {            // the bucket of zero and of every |q| < 2^-14
    out.base = sign ? 7u : 8u;
    return out;
  }
  const float lo = bits2f(mag << 21), hi = bits2f((mag + 1u) << 21);
  for (int j = 0; j < 16; ++j) {
    const float t = bits2f(kQmapMBits[j]);
    if (!sign) {              // bucket holds q in [lo, hi)
      if (t < lo) ++out.base;
      else if (t < hi) out.thr = kQmapMBits[j];
    } else {                  // bucket holds q in (-hi, -lo]
      if (t <= -hi) ++out.base;
      else if (t <= -lo) out.thr = kQmapMBits[j];
    }
  }
  return out;
}

// The table as the kernels keep it: the interval number k_raw leads to entry [k_raw] of the
// 8-byte affine table below, so a bucket's entry carries the two byte offsets it can lead to
// as the halves of one word, 8 * base in the low half (q below the bucket's code-book entry,
// or no entry in the bucket) and 8 * (base + 1) in the high half.
struct SrSlot {
  uint32_t thr;      // as SrEntry::thr
  uint32_t offsets;  // 8 * base | 8 * (base + 1) << 16
};

struct SrHalfTable {
  SrSlot e[kHalfTableEntries];
};

constexpr SrHalfTable make_sr_half_table() {
  SrHalfTable t{};
  for (uint32_t h = 0; h < kHalfTableEntries; ++h) {
    const SrEntry e = sr_entry(h);
    t.e[h] = SrSlot{e.thr, (e.base * 8u) | ((e.base + 1u) * 8u) << 16};
  }
  return t;
}

// number of code-book entries that some bucket names as its threshold: must be all that
// are not zero (zero sits on the boundary between the two zero buckets)
constexpr int sr_thresholds_found() {
  int n = 0;
  for (uint32_t h = 0; h < kHalfTableEntries; ++h) n += sr_entry(h).thr != kNoThr ? 1 : 0;
  return n;
}
static_assert(sr_thresholds_found() == 15, "every non-zero code-book entry needs a bucket of its own");

struct SrInterval {
  float lower, width;
};

Q4_HD constexpr SrInterval sr_interval_m(uint32_t k_raw) {  // k_raw 0..16
  if (k_raw == 0u) return SrInterval{-3.4028234663852886e38f, 0.0f};
  const float lower = bits2f(kQmapMBits[k_raw - 1u]);
  if (k_raw == 16u) return SrInterval{lower, __builtin_inff()};
  return SrInterval{lower, bits2f(kQmapMBits[k_raw]) - lower};
}

struct SrIntervalTable {
  SrInterval e[17];
};

constexpr SrIntervalTable make_sr_interval_table() {
  SrIntervalTable t{};
  for (uint32_t k = 0; k < 17; ++k) t.e[k] = sr_interval_m(k);
  return t;
}

// The fast path's form of the same decision: inside interval k_raw = 1..15 the code is
// floor(k_raw + (q - lower) / width - noise), an affine function of q minus the noise, so
// entry [k_raw] holds {1 / width, k_raw - lower / width} (from the exact interval in
// double precision, rounded once).  Below the first entry {0, 1} gives floor(1 - noise) = 0,
// at or above the last one {0, 16} gives floor(16 - noise) = 15.
struct SrAffine {
  float a, c;
};

Q4_HD constexpr SrAffine sr_affine_m(uint32_t k_raw) {  // k_raw 0..16
  if (k_raw == 0u) return SrAffine{0.0f, 1.0f};
  if (k_raw == 16u) return SrAffine{0.0f, 16.0f};
  const double lower = (double)bits2f(kQmapMBits[k_raw - 1u]);
  const double width = (double)bits2f(kQmapMBits[k_raw]) - lower;
  return SrAffine{(float)(1.0 / width), (float)((double)k_raw - lower / width)};
}

struct SrAffineTable {
  SrAffine e[17];
};

constexpr SrAffineTable make_sr_affine_table() {
  SrAffineTable t{};
  for (uint32_t k = 0; k < 17; ++k) t.e[k] = sr_affine_m(k);
  return t;
}

// The error of the affine form, in units of one code, is the quotient's relative error
// times |q| / width: the guard band of the fast path is sized for a ratio below 9.
constexpr bool sr_affine_ratio_ok() {
  for (uint32_t k = 1; k < 16; ++k) {
    const double lo = (double)bits2f(kQmapMBits[k - 1u]), hi = (double)bits2f(kQmapMBits[k]);
    const double big = (lo < 0 ? -lo : lo) > (hi < 0 ? -hi : hi) ? (lo < 0 ? -lo : lo) : (hi < 0 ? -hi : hi);
    if (big / (hi - lo) >= 9.0) return false;
  }
  return true;
}
static_assert(sr_affine_ratio_ok(), "first-moment code book: an interval too narrow for the guard band");

}  // namespace q4
