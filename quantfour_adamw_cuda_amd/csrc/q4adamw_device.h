// Device helpers of the 4-bit AdamW kernels: address spaces and buffer resources, wave
// reductions, 16-bit element conversion, element loads and stores, the exact quantizers, the
// rounding noise, the correctly rounded square root and quotients of the exact parameter
// update, the tensor search.
#pragma once
#include "q4adamw_args.h"

namespace q4 {

// ---------------------------------------------------------------------------
// device helpers
// ---------------------------------------------------------------------------
// Pointers that arrive inside a descriptor are generic; every tensor lives in
// global memory, so say so and get global_load/global_store instead of flat ones.
template <typename T>
using gptr = __attribute__((address_space(1))) T *;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <typename T>
__device__ __forceinline__ gptr<T> as_global(const void *p) {
  return (gptr<T>)(uintptr_t)p;
}

// Memory that no kernel of the running launch writes, read through the scalar unit when
// the address is uniform.
template <typename T>
using cptr = __attribute__((address_space(4))) T *;
template <typename T>
__device__ __forceinline__ cptr<T> as_constant(const void *p) {
  return (cptr<T>)(uintptr_t)p;
}

// Full tiles go through buffer instructions: the tile's base address sits in a
// scalar resource descriptor and each lane supplies a 32-bit byte offset, so no
// vector ALU work goes into addresses.  Cache policy of the streamed tensors: the
// non-temporal hint (bit 1) plus system scope (sc1, bit 4); every datum is touched
// once, and with the wider scope the streams measure 1.5 % faster than with the hint
// alone (and 11 % faster than without either).
typedef __amdgpu_buffer_rsrc_t rsrc_t;
constexpr int kNt = 2 | 16;
// Stores to a tensor that does not start on a 16-byte boundary: a wave's first and last line
// are shared with its neighbours, and without sc1 the halves meet in the cache instead of
// reaching memory as two partial writes (fp32 parameters one element off a boundary, 2^28
// elements: 0.540 ms against 0.668 with sc1; aligned tensors: 0.531 against 0.510).
constexpr int kNtSharedLines = 2;
constexpr int kNtReadOnly = 2;  // a pure read stream (the gradient norm) measures the same with and without sc1

__device__ __forceinline__ rsrc_t tile_rsrc(const void *base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, -1, 0x00020000);
}

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_umax(uint32_t x) {
  const uint32_t y = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, CTRL, 0xf, 0xf, true);
  return x > y ? x : y;
}

// Abs-max of both moments over the 32 lanes of a quantization block (lanes 0-31 or
// 32-63), results in every lane of the block.  The inputs are non-negative floats,
// so their bit patterns order like unsigned integers.  One v_permlane16_swap pairs
// lane i of the block's first row with lane i of its second row and leaves the
// first-moment partial max in the first row and the second-moment partial max in
// the second row; four DPP steps then reduce both rows at once; a second swap
// hands each row the other row's result.
__device__ __forceinline__ void block_max32_pair(float &am, float &av) {
  // after the swap: a = [am.r0, av.r0, am.r2, av.r2], b = [am.r1, av.r1, am.r3, av.r3]
  const auto s1 = __builtin_amdgcn_permlane16_swap(f2bits(am), f2bits(av), false, false);
  uint32_t u = s1[0] > s1[1] ? s1[0] : s1[1];
  u = dpp_umax<0xB1>(u);   // quad_perm [1,0,3,2]
  u = dpp_umax<0x4E>(u);   // quad_perm [2,3,0,1]
  u = dpp_umax<0x141>(u);  // row_half_mirror
  u = dpp_umax<0x140>(u);  // row_mirror
  // u = [max am, max av, max am, max av] per row; spread: a = rows (0,0,2,2), b = rows (1,1,3,3)
  const auto s2 = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  am = bits2f(s2[0]);
  av = bits2f(s2[1]);
}

// Max of a non-negative float over the 16 lanes of a DPP row, result in every lane.
__device__ __forceinline__ float row_max16(float x) {
  uint32_t u = f2bits(x);
  u = dpp_umax<0xB1>(u);
  u = dpp_umax<0x4E>(u);
  u = dpp_umax<0x141>(u);
  u = dpp_umax<0x140>(u);
  return bits2f(u);
}

// Element types of parameters and gradients, by the tags of include/q4adamw.h:
// 0 = fp32, 1 = bf16, 2 = fp16.  A non-zero tag is a 16-bit type.
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// one 16-bit pattern -> fp32 (exact)
template <int DT>
__device__ __forceinline__ float widen_bits(uint32_t h) {
  static_assert(DT == Q4ADAMW_BF16 || DT == Q4ADAMW_FP16, "a 16-bit element type");
  if (DT == Q4ADAMW_BF16) return bits2f(h << 16);
  return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

// fp32 -> one 16-bit pattern, round to nearest even
template <int DT>
__device__ __forceinline__ uint32_t narrow_bits(float f) {
  static_assert(DT == Q4ADAMW_BF16 || DT == Q4ADAMW_FP16, "a 16-bit element type");
  if (DT == Q4ADAMW_BF16) return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f);
  return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);
}

// two fp32 -> two 16-bit values (round to nearest even) in one 32-bit word, lo in the low half
template <int DT>
__device__ __forceinline__ uint32_t pack_pair(float lo, float hi) {
  if (DT == Q4ADAMW_BF16) return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, bf16x2));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, f16x2));
}

template <int DT>
__device__ __forceinline__ void widen_pair(uint32_t w, float &lo, float &hi) {
  if (DT == Q4ADAMW_BF16) {
    lo = bits2f(w << 16);
    hi = bits2f(w & 0xffff0000u);
  } else {
    const f32x2 f = __builtin_convertvector(__builtin_bit_cast(f16x2, w), f32x2);
    lo = f.x;
    hi = f.y;
  }
}

// element i of an array of element type DT, as fp32
template <int DT>
__device__ __forceinline__ float load_scalar(const void *base, int64_t i) {
  if constexpr (DT == Q4ADAMW_FP32) return as_global<const float>(base)[i];
  else return widen_bits<DT>(as_global<const uint16_t>(base)[i]);
}

template <int DT>
__device__ __forceinline__ void store_scalar(void *base, int64_t i, float x) {
  if constexpr (DT == Q4ADAMW_FP32) as_global<float>(base)[i] = x;
  else as_global<uint16_t>(base)[i] = (uint16_t)narrow_bits<DT>(x);
}

// N consecutive elements (N = 4 or 8) starting at element e0 of the tile at base
template <int DT, int N, bool FULL>
__device__ __forceinline__ void load_elems(const void *base, uint32_t e0, int nv, float (&x)[N]) {
  if (FULL) {
    if constexpr (DT != 0 && N == 4) {
      const u32x2 w = __builtin_amdgcn_raw_buffer_load_b64(tile_rsrc(base), e0 * 2, 0, kNt);
      widen_pair<DT>(w.x, x[0], x[1]);
      widen_pair<DT>(w.y, x[2], x[3]);
    } else if constexpr (DT != 0) {
      const u32x4 w = __builtin_amdgcn_raw_buffer_load_b128(tile_rsrc(base), e0 * 2, 0, kNt);
      widen_pair<DT>(w.x, x[0], x[1]);
      widen_pair<DT>(w.y, x[2], x[3]);
      widen_pair<DT>(w.z, x[N - 4], x[N - 3]);
      widen_pair<DT>(w.w, x[N - 2], x[N - 1]);
    } else {
#pragma unroll
      for (int k = 0; k < N; k += 4) {
        const u32x4 a = __builtin_amdgcn_raw_buffer_load_b128(tile_rsrc(base), (e0 + k) * 4, 0, kNt);
        x[k] = bits2f(a.x); x[k + 1] = bits2f(a.y); x[k + 2] = bits2f(a.z); x[k + 3] = bits2f(a.w);
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < N; ++j) {
      x[j] = 0.0f;
      if (j < nv) {
        x[j] = load_scalar<DT>(base, e0 + j);
      }
    }
  }
}

template <int POLICY>
__device__ __forceinline__ void store_b64(u32x2 w, const void *base, uint32_t offset) {
  __builtin_amdgcn_raw_buffer_store_b64(w, tile_rsrc(base), offset, 0, POLICY);
}
template <int POLICY>
__device__ __forceinline__ void store_b128(u32x4 w, const void *base, uint32_t offset) {
  __builtin_amdgcn_raw_buffer_store_b128(w, tile_rsrc(base), offset, 0, POLICY);
}

// whether a tensor's lines are shared between neighbouring waves (uniform: the low bits of a
// tile's address are those of its tensor's)
__device__ __forceinline__ bool shares_lines(const void *base) {
  return __builtin_expect((reinterpret_cast<uintptr_t>(base) & 15u) != 0, 0);
}

template <int DT, int N, bool FULL>
__device__ __forceinline__ void store_elems(void *base, uint32_t e0, int nv, const float (&x)[N]) {
  if (FULL) {
    const bool shared = shares_lines(base);
    if constexpr (DT != 0 && N == 4) {
      u32x2 w;
      w.x = pack_pair<DT>(x[0], x[1]);
      w.y = pack_pair<DT>(x[2], x[3]);
      if (shared) store_b64<kNtSharedLines>(w, base, e0 * 2);
      else store_b64<kNt>(w, base, e0 * 2);
    } else if constexpr (DT != 0) {
      u32x4 w;
      w.x = pack_pair<DT>(x[0], x[1]);
      w.y = pack_pair<DT>(x[2], x[3]);
      w.z = pack_pair<DT>(x[N - 4], x[N - 3]);
      w.w = pack_pair<DT>(x[N - 2], x[N - 1]);
      if (shared) store_b128<kNtSharedLines>(w, base, e0 * 2);
      else store_b128<kNt>(w, base, e0 * 2);
    } else {
#pragma unroll
      for (int k = 0; k < N; k += 4) {
        const u32x4 w = {f2bits(x[k]), f2bits(x[k + 1]), f2bits(x[k + 2]), f2bits(x[k + 3])};
        if (shared) store_b128<kNtSharedLines>(w, base, (e0 + k) * 4);
        else store_b128<kNt>(w, base, (e0 + k) * 4);
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < N; ++j) {
      if (j < nv) {
        store_scalar<DT>(base, e0 + j, x[j]);
      }
    }
  }
}

// zeros over the N elements that load_elems<DT, N, FULL> read
template <int DT, int N, bool FULL>
__device__ __forceinline__ void zero_elems(void *base, uint32_t e0, int nv) {
  if (FULL) {
    const u32x4 z4 = {0u, 0u, 0u, 0u};
    const bool shared = shares_lines(base);
    if (DT && N == 4) {
      const u32x2 z2 = {0u, 0u};
      if (shared) store_b64<kNtSharedLines>(z2, base, e0 * 2);
      else store_b64<kNt>(z2, base, e0 * 2);
    } else if (DT) {
      if (shared) store_b128<kNtSharedLines>(z4, base, e0 * 2);
      else store_b128<kNt>(z4, base, e0 * 2);
    } else {
#pragma unroll
      for (int k = 0; k < N; k += 4) {
        if (shared) store_b128<kNtSharedLines>(z4, base, (e0 + k) * 4);
        else store_b128<kNt>(z4, base, (e0 + k) * 4);
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < N; ++j) {
      if (j < nv) {
        if (DT) as_global<uint16_t>(base)[e0 + j] = 0;
        else as_global<float>(base)[e0 + j] = 0.0f;
      }
    }
  }
}

// Zeros over one tile of a gradient tensor: what is left of a step's work when an
// overflow flag cancels it and the caller asked for the gradients to be cleared.
template <int DT, int N>
__device__ __forceinline__ void zero_tile(const void *g, int64_t tile, int64_t numel, int lane) {
  constexpr int64_t kTile = 64 * N;
  const int64_t tb = tile * kTile;
  if (tb >= numel) return;
  void *g_tile = static_cast<char *>(const_cast<void *>(g)) + tb * (DT ? 2 : 4);
  const uint32_t e0 = (uint32_t)lane * N;
  if (tb + kTile <= numel) {
    zero_elems<DT, N, true>(g_tile, e0, N);
  } else {
    const int64_t rem = numel - tb - (int64_t)e0;
    zero_elems<DT, N, false>(g_tile, e0, rem >= N ? N : (rem > 0 ? (int)rem : 0));
  }
}

template <int N>
struct Vals {
  float x[N];
};

// Exact quantization of N values of one state: IEEE division by the block scale,
// then the number of thresholds strictly below the quotient
// (cuda_adamw_kernels.cu:167-194 in closed form).  0/0 is NaN and gets code 0.
template <bool SECOND, int N>
__device__ __forceinline__ uint32_t quantize_exact(const Vals<N> &v, float scale) {
  uint32_t word = 0;
#pragma unroll
  for (int j = 0; j < N; ++j) {
    const float q = v.x[j] / scale;
    uint32_t c = 0;
#pragma unroll
    for (int k = 0; k < 15; ++k) {
      const float t = SECOND ? qmid_v(k) : bits2f(kQmidMBits[k]);
      c += (t < q) ? 1u : 0u;
    }
    word |= c << (4 * j);
  }
  return word;
}

// The same for the second moment with a scale per element (rank-1 scaling).
template <int N>
__device__ __forceinline__ uint32_t quantize_exact_scales(const Vals<N> &v, const Vals<N> &scale) {
  uint32_t word = 0;
#pragma unroll
  for (int j = 0; j < N; ++j) {
    const float q = v.x[j] / scale.x[j];
    uint32_t c = 0;
#pragma unroll
    for (int k = 0; k < 15; ++k) c += (qmid_v(k) < q) ? 1u : 0u;
    word |= c << (4 * j);
  }
  return word;
}

// Adds element j's code to a lane's word of 4-bit codes.  Four elements per lane: the code
// (0..15 and no other bits) goes to its place.  Eight: every code enters at the top and
// moves down four bits per later element.
template <int N>
__device__ __forceinline__ uint32_t append_code(uint32_t word, uint32_t code, int j) {
  if (N == 4) return j == 0 ? code : ((code << (4 * j)) | word);
  return __builtin_amdgcn_alignbit(code, word, 4);
}

// A 32-bit integer mixer (two multiply-xorshift rounds) for the rounding noise.
__host__ __device__ __forceinline__ uint32_t lowbias32(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7FEB352Du;
  x ^= x >> 15;
  x *= 0x846CA68Bu;
  x ^= x >> 16;
  return x;
}

// lowbias32 without its last step: lowbias32(x) == y ^ (y >> 16) for y = lowbias32_open(x).
// The step kernel takes the two 16-bit halves of the hash as floats and lets the conversions
// do that step: the high half of y ^ (y >> 16) is y's own, the low half is y's two halves
// xor-ed, and both selections ride on the instructions' operand selectors.
__device__ __forceinline__ uint32_t lowbias32_open(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7FEB352Du;
  x ^= x >> 15;
  x *= 0x846CA68Bu;
  return x;
}

__device__ __forceinline__ float hash_high_half_as_float(uint32_t y) {
  float r;
  asm("v_cvt_f32_u32_sdwa %0, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:WORD_1" : "=v"(r) : "v"(y));
  return r;
}

__device__ __forceinline__ float hash_low_half_as_float(uint32_t y) {
  uint32_t lo;
  asm("v_xor_b32_sdwa %0, %1, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:WORD_1 src1_sel:WORD_0" : "=v"(lo) : "v"(y));
  return (float)lo;
}

// halves' high 16 bits if q >= thr, else its low 16 bits (a NaN on either side: the low half).
// The select reads the halves through its operand selectors, so the choice between two small
// numbers kept in one word costs a compare and one more instruction.  On this target a vector
// instruction that reads VCC needs two wait states after the vector instruction that wrote it;
// the compiler keeps that distance in its own code and does not look into this block, hence
// the s_nop (it holds back this wave only: the other waves of the SIMD issue meanwhile).
__device__ __forceinline__ uint32_t high_half_if_ge(float q, float thr, uint32_t halves) {
  uint32_t r;
  asm("v_cmp_ge_f32_e32 vcc, %1, %2\n\t"
      "s_nop 1\n\t"
      "v_cndmask_b32_sdwa %0, %3, %3, vcc dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:WORD_0 src1_sel:WORD_1"
      : "=v"(r)
      : "v"(q), "v"(thr), "v"(halves)
      : "vcc");
  return r;
}

// noise in (0, 1) from a 16-bit number (as a float): (2 n + 1) / 2^17, exact
constexpr float kNoiseStep = 1.52587890625e-05f;     // 2^-16
__device__ __forceinline__ float sr_noise_value(float n16) {
  return __builtin_fmaf(n16, kNoiseStep, 0.5f * kNoiseStep);
}

// Stochastic rounding, exact form (the closed form of quantize_bsearch<STOCHASTIC>,
// optim/adamw_fourbit_triton.py:1050-1075, without its division): IEEE quotient, its
// interval [Q[k], Q[k+1]) among the code-book entries, upper code iff
// noise * (Q[k+1] - Q[k]) < q - Q[k].  0/0 is NaN and gets code 0.
template <bool SECOND>
__device__ __forceinline__ uint32_t sr_code_exact(float q, float noise) {
  uint32_t k_raw = 0;
#pragma unroll
  for (int k = 0; k < 16; ++k) {
    const float t = SECOND ? qmap_v(k) : bits2f(kQmapMBits[k]);
    k_raw += (t <= q) ? 1u : 0u;
  }
  float lower, width;
  if (SECOND) {
    lower = k_raw == 0u ? -3.4028234663852886e38f : (float)k_raw * 0.0625f;
    width = k_raw == 0u ? 0.0f : (k_raw == 16u ? __builtin_inff() : 0.0625f);
  } else {
    const SrInterval iv = kSrIntervals.e[k_raw];
    lower = iv.lower;
    width = iv.width;
  }
  const bool up = noise * width < q - lower;
  int c = (int)k_raw - 1 + (up ? 1 : 0);
  c = c < 0 ? 0 : (c > 15 ? 15 : c);
  return (uint32_t)c;
}

template <bool SECOND, int N>
__device__ __forceinline__ uint32_t quantize_exact_sr(const Vals<N> &v, float scale, const Vals<N> &noise) {
  uint32_t word = 0;
#pragma unroll
  for (int j = 0; j < N; ++j) word |= sr_code_exact<SECOND>(v.x[j] / scale, noise.x[j]) << (4 * j);
  return word;
}

// The same for the second moment with a scale per element (rank-1 scaling).
template <int N>
__device__ __forceinline__ uint32_t quantize_exact_sr_scales(const Vals<N> &v, const Vals<N> &scale,
                                                             const Vals<N> &noise) {
  uint32_t word = 0;
#pragma unroll
  for (int j = 0; j < N; ++j) word |= sr_code_exact<true>(v.x[j] / scale.x[j], noise.x[j]) << (4 * j);
  return word;
}

// (x & mask) | base as one v_and_or_b32: the mask travels in a scalar register (the
// compiler splits the operation when the mask is a literal, which a VOP3 encoding
// cannot hold).
__device__ __forceinline__ uint32_t and_or(uint32_t x, uint32_t mask, uint32_t base) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "s"(mask), "v"(base));
  return r;
}

// Byte BYTE of x shifted left by `shift` (the byte offset of a table entry of 1 << shift
// bytes), as one SDWA shift; the shift amount travels in a register.
template <int BYTE>
__device__ __forceinline__ uint32_t byte_shifted(uint32_t x, uint32_t shift) {
  static_assert(BYTE >= 0 && BYTE <= 3, "");
  uint32_t r;
#define Q4_SDWA_SHIFT(SEL)                                                                          \
  asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:" SEL \
      : "=v"(r) : "v"(shift), "v"(x))
  if (BYTE == 0) Q4_SDWA_SHIFT("BYTE_0");
  else if (BYTE == 1) Q4_SDWA_SHIFT("BYTE_1");
  else if (BYTE == 2) Q4_SDWA_SHIFT("BYTE_2");
  else Q4_SDWA_SHIFT("BYTE_3");
#undef Q4_SDWA_SHIFT
  return r;
}

// byte_shifted with the byte chosen by a loop index of an unrolled loop
__device__ __forceinline__ uint32_t entry_offset(uint32_t x, int byte, uint32_t shift) {
  switch (byte) {
    case 0: return byte_shifted<0>(x, shift);
    case 1: return byte_shifted<1>(x, shift);
    case 2: return byte_shifted<2>(x, shift);
    default: return byte_shifted<3>(x, shift);
  }
}

// 1/s to within half an ulp for s in [2^-100, 2^100]: hardware estimate plus one
// Newton step
__device__ __forceinline__ float refined_rcp(float s) {
  const float r0 = __builtin_amdgcn_rcpf(s);
  const float e = __builtin_fmaf(-s, r0, 1.0f);
  return __builtin_fmaf(e, r0, r0);
}

// ---------------------------------------------------------------------------
// The parameter update with every operation rounded as IEEE 754 rounds it
// (optim/cuda_adamw_kernels.cu:334,351: sqrtf, /, +, /, *, *, -), without the scaling and the
// special-case instructions of the general expansions: the three functions below are exact
// inside the ranges they name, the caller checks the ranges per lane and takes the general
// expansions (`sqrtf`, `/`) outside them.
// ---------------------------------------------------------------------------
// RN(sqrt(v)) for 2^-96 <= v <= 2^100 (or NaN).  The hardware's estimate s is within one ulp,
// so the answer is s or one of its neighbours s_dn, s_up, and the residuals against the two
// midpoints decide: the root lies below the midpoint of s_dn and s iff v <= s_dn * s (the
// midpoint's square exceeds that product by a quarter ulp squared, less than v's spacing),
// above the midpoint of s and s_up iff v > s_up * s.  Each residual is one fma (only its
// sign matters, so its rounding does not); written as s_dn * s - v >= 0 and s_up * s - v < 0
// the two decisions are the residuals' sign bits (an fma never returns -0 for an exact zero),
// and the answer's bit pattern is s_dn's plus one for each set sign bit.  Below 2^-96 the
// residuals' operands leave the normal range.
__device__ __forceinline__ float sqrt_rn(float v) {
  const float s = __builtin_amdgcn_sqrtf(v);
  const uint32_t s_dn = f2bits(s) - 1u, s_up = f2bits(s) + 1u;
  const uint32_t above_dn = f2bits(__builtin_fmaf(bits2f(s_dn), s, -v)) >> 31;   // v >  s_dn * s
  const uint32_t above_up = f2bits(__builtin_fmaf(bits2f(s_up), s, -v)) >> 31;   // v >  s_up * s
  return bits2f(s_dn + above_dn + above_up);
}

// RN(x / c) given y = RN(1/c), for 2^-60 <= |x|, c <= 2^60: quotient, exact residual, one
// correction.  The corrected value is t + r * (y - 1/c) with t the true quotient, within
// 4.5 * 2^-24 ulp of t, so the result can differ from RN(t) only where t comes that close to
// the midpoint of two floats; tests/native/check_exact_update.c lists every such (x, c) -- for all
// 2^23 divisor mantissas -- and shows that the sequence rounds each of them correctly.
__device__ __forceinline__ float div_by_reciprocal(float x, float c, float y) {
  const float q0 = x * y;
  const float r = __builtin_fmaf(-c, q0, x);
  return __builtin_fmaf(r, y, q0);
}

// RN(m / d) for 2^-60 <= |m|, d <= 2^60.  One Newton step takes the hardware's estimate of 1/d
// (within one ulp) to RN(1/d): a property of this GPU's v_rcp_f32, established by walking every
// divisor (tests/test_gpu_exact_update.py); arithmetic alone only promises it for divisors
// whose mantissa is not all ones.
__device__ __forceinline__ float div_rn(float m, float d) {
  const float y0 = __builtin_amdgcn_rcpf(d);
  const float y = __builtin_fmaf(__builtin_fmaf(-d, y0, 1.0f), y0, y0);
  return div_by_reciprocal(m, d, y);
}

constexpr float kExactLo = 8.673617379884035e-19f;   // 2^-60
constexpr float kExactHi = 1.152921504606847e+18f;   // 2^60
constexpr float kExactVLo = 1.262177448353619e-29f;  // 2^-96
constexpr float kExactVHi = 1.2379400392853803e+27f; // 2^90

// The update as the reference writes it; `sqrtf` and `/` are the compiler's general
// correctly rounded expansions, products and sums stay apart (-ffp-contract=off).
__device__ __forceinline__ float param_update_ieee(float p, float m, float v, const StepConsts &sc) {
  const float den = __builtin_sqrtf(v) / sc.c2s + sc.eps;
  return p * sc.wdu - sc.ss * (m / den);
}

constexpr float kScaleLo = 7.888609052210118e-31f;   // 2^-100
constexpr float kScaleHi = 1.2676506002282294e+30f;  // 2^100
// 16 / scale at or above this (2^103.5) means a scale at the lower end of the range or below
// it (16 / kScaleLo is 2^104 give or take the reciprocal's ulp)
constexpr float kInvScaleLo16 = 1.4340386889e+31f;
constexpr float kVGuard = 7.62939453125e-06f;        // 2^-17, in units of 16*q
static_assert(kVGuard == 0.5f * kNoiseStep, "the fast path lets the noise's offset cancel the guard band");

// Uniform search of the launch's tensor list: the last tensor whose first chunk is
// <= chunk.  first_chunk[0] is 0, so the result is never negative.  Chunk indices and
// table entries are below 2^31, so bit 31 of (x - chunk - 1) says x <= chunk: plain
// integer arithmetic that stays on the scalar unit.
template <typename Args>
__device__ __forceinline__ int find_tensor(const Args &a, uint32_t chunk) {
  uint32_t group = 0;
#pragma unroll
  for (int k = 1; k < Args::kPivots; ++k) group += (a.pivot[k] - chunk - 1u) >> 31;
  uint32_t within = 0;
#pragma unroll
  for (int k = 0; k < 8; ++k) within += (a.first_chunk[group * 8 + k] - chunk - 1u) >> 31;
  return (int)(group * 8 + within) - 1;
}

// LDS of a workgroup, one array of 8-byte entries:
//   [0, 256)    the waves' private dequantization tables, as two arrays of 256 floats: the
//               first moment's at float 0, the second moment's at float kLdsSecondMoment;
//               per wave 64 entries of each, per quantization block 16 (code book value *
//               block scale * beta), so that dequantizing an element is one 4-byte read
//               per moment and an entry number fits a byte
//   [256, 512)  bucket table of the first-moment quantizer, indexed by the high byte
//               of the quotient as a half
//   [512, 529)  stochastic rounding only: the first moment's intervals as affine maps
constexpr uint32_t kLdsBuckets = 64 * kWaves;
constexpr uint32_t kLdsSecondMoment = 64 * kWaves;   // in floats: the second array of the dequantization tables
constexpr uint32_t kLdsIntervals = kLdsBuckets + kHalfTableEntries;
constexpr uint32_t kLdsEntries = kLdsIntervals + 32;
static_assert(kLdsBuckets == 256, "dequantization entry numbers must fit a byte");
static_assert(kThreads == (int)kHalfTableEntries, "one bucket table entry per thread");

// What a thread fetches from the constant tables as the very first thing it does.
struct TableSlot {
  uint2 entry;     // bucket table entry number tid
  float qm;        // first-moment code-book value number (lane & 15)
  uint2 interval;  // stochastic rounding: affine table entry number tid (tid < 17)
};

template <bool SR>
__device__ __forceinline__ TableSlot request_table_slot(int tid) {
  TableSlot s;
  if (SR) {
    const SrSlot e = kSrHalfTable.e[tid];
    s.entry = make_uint2(e.thr, e.offsets);
    const SrAffine af = kSrAffine.e[tid < 17 ? tid : 0];
    s.interval = make_uint2(f2bits(af.a), f2bits(af.c));
  } else {
    const MtabEntry e = kHalfTable.e[tid];
    s.entry = make_uint2(e.lo, e.hi);
    s.interval = make_uint2(0u, 0u);
  }
  s.qm = bits2f(kQmapMDev[tid & 15]);
  return s;
}

// Writes the slot into LDS and waits for the whole workgroup.  Called by every wave
// exactly once, after it has issued its global loads, so that the latencies overlap.
// The fences order LDS only: a full __syncthreads() would also drain the outstanding
// global loads.
template <bool SR>
__device__ __forceinline__ void setup_tables(uint2 *lds, int tid, const TableSlot &s) {
  lds[kLdsBuckets + tid] = s.entry;
  if (SR && tid < 17) lds[kLdsIntervals + tid] = s.interval;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// The launch's gradient multiplier; false if the launch is to do nothing.
// The step's derived scalars: the launch's arguments, or what device_step_kernel left in
// device memory for a step whose number the host does not know (a captured graph).
__device__ __forceinline__ StepConsts step_consts(const StepConsts &from_args, const GradOps &go) {
  static_assert(sizeof(StepConsts) == 48, "twelve floats; device_step_kernel writes them in the order read here, the step number between them");
  StepConsts sc = from_args;
  if (go.sc_dev) {
    const cptr<const float> f = as_constant<const float>(go.sc_dev);
    sc.b1 = f[0]; sc.b2 = f[1]; sc.r1 = f[2]; sc.r2 = f[3]; sc.wdu = f[4];
    sc.ss = f[5]; sc.c2s = f[6]; sc.eps = f[7]; sc.den_scale = f[8]; sc.den_eps = f[9];
    sc.c2s_rcp = f[11];   // f[10] is the step number
    sc.exact_short = as_constant<const uint32_t>(go.sc_dev)[12];
  }
  return sc;
}

// The noise salt of a tensor in this step (q4adamw_sr_tensor_salt: the tensor's own salt,
// the step number and the two halves of the seed, hashed in turn).  The host has finished the
// chain when it knows the step number; otherwise it has hashed the tensor's salt and the
// kernel goes on with the number device_step_kernel left behind its scalars.
__device__ __forceinline__ uint32_t step_salt(uint32_t from_args, const GradOps &go, uint32_t seed_lo,
                                              uint32_t seed_hi) {
  if (!go.sc_dev) return from_args;
  const uint32_t step = as_constant<const uint32_t>(go.sc_dev)[10];
  return lowbias32(lowbias32(lowbias32(from_args ^ step) ^ seed_hi) ^ seed_lo);
}

__device__ __forceinline__ bool grad_ops_begin(const GradOps &go, float &gscale) {
  if (go.skip && *as_global<const float>(go.skip) != 0.0f) return false;
  gscale = go.scale;
  if (go.scale_dev) gscale *= *as_global<const float>(go.scale_dev);
  return true;
}

// Minimum and maximum of non-negative, non-NaN floats (scales, maxima) through their bit
// patterns: one integer instruction each, where fminf / fmaxf on loaded values would
// first canonicalise both operands.
__device__ __forceinline__ float min_nonneg(float a, float b) {
  const uint32_t x = f2bits(a), y = f2bits(b);
  return bits2f(x < y ? x : y);
}

__device__ __forceinline__ float max_nonneg(float a, float b) {
  const uint32_t x = f2bits(a), y = f2bits(b);
  return bits2f(x > y ? x : y);
}

// Atomic maximum of non-negative floats through their bit patterns.
__device__ __forceinline__ void atomic_max_nonneg(const float *addr, float x) {
  // non-negative floats order like their bit patterns
  atomicMax(reinterpret_cast<unsigned int *>(const_cast<float *>(addr)), f2bits(x));
}

}  // namespace q4
