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
// The kernel's fast path knows q only to within three ulps (it multiplies by a
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
  if (e >= 128u) {           // |q| >= 2, inf, nan: beyond every threshold
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

// Only the buckets that can hold a threshold differ from "no threshold, base 7":
// per sign, buckets kBucketFloor .. kBucketTop (|q| from 1.75 * 2^-10 to 1.25).
// The kernel clamps smaller magnitudes up to the floor bucket and builds just these
// entries in LDS, at their natural index, leaving the rest of the table untouched.
constexpr uint32_t kBucketFloor = 471;                                  // exponent 117, mantissa 11b
constexpr uint32_t kBucketTop = 508;                                    // exponent 127, mantissa 00b
constexpr uint32_t kBucketsPerSign = kBucketTop - kBucketFloor + 1;     // 38
constexpr uint32_t kNegativeBuckets = 1024;                             // index offset of the sign bit

// What the first 128 threads of a workgroup copy into LDS, one 8-byte entry each:
// slots 0..37   : positive buckets kBucketFloor.. (a = lo bound | base, b = hi bound)
// slots 38..75  : negative buckets
// slots 76..95  : padding (written to the unused entries 0..19)
// slots 96..111 : first-moment code book  (a = fp32 bits) -> entries 2048..2063
// slots 112..127: second-moment code book (a = fp32 bits) -> entries 2064..2079
// entry[] is the index of the 8-byte LDS entry the slot goes to.
struct WorkgroupTables {
  uint32_t a[128];
  uint32_t b[128];
  uint32_t entry[128];
};

// slot j of the compact table <-> bucket index in the full table
Q4_HD constexpr uint32_t compact_slot_bucket(uint32_t j) {
  return j < kBucketsPerSign ? kBucketFloor + j
                             : kNegativeBuckets + kBucketFloor + (j - kBucketsPerSign);
}

constexpr WorkgroupTables make_workgroup_tables() {
  WorkgroupTables t{};
  for (uint32_t j = 0; j < 2 * kBucketsPerSign; ++j) {
    const MtabEntry e = mtab_entry(compact_slot_bucket(j));
    t.a[j] = e.lo;
    t.b[j] = e.hi;
  }
  for (uint32_t k = 0; k < 16; ++k) {
    t.a[96 + k] = kQmapMBits[k];
    t.a[112 + k] = f2bits(qmap_v((int)k));
  }
  for (uint32_t j = 0; j < 128; ++j) {
    t.entry[j] = j < 2 * kBucketsPerSign ? compact_slot_bucket(j)
                 : j < 96                ? j - 2 * kBucketsPerSign
                                         : kMtabEntries + (j - 96);
  }
  return t;
}

}  // namespace q4
